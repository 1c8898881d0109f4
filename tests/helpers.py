"""Shared checks for the parity tests (host side, numpy only)."""
import numpy as np


def ordered_int(a):
    """float32 array -> int64 whose integer order is the float order
    (-0 and +0 both map to 0), so |difference| is a distance in ulps."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    return np.where(u < 0, -(u & 0x7FFFFFFF), u)


def ulp_diff(a, b):
    """Element-wise distance in float32 ulps; NaN vs NaN counts as 0,
    NaN vs number as a huge distance."""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    d = np.abs(ordered_int(a) - ordered_int(b))
    an, bn = np.isnan(a), np.isnan(b)
    d = np.where(an & bn, 0, d)
    d = np.where(an ^ bn, 1 << 40, d)
    return d


def half_ulp_diff(a, b):
    """Distance in binary16 ulps between two float16 (or uint16-bit) arrays;
    NaN vs NaN counts as 0, NaN vs number as a huge distance."""
    def bits(h):
        h = np.asarray(h)
        return h.view(np.uint16) if h.dtype == np.float16 else h
    def oi(h):
        s = bits(h).astype(np.int64)
        return np.where(s & 0x8000, -(s & 0x7FFF), s)
    def nan(h):
        return (bits(h) & 0x7FFF) > 0x7C00
    d = np.abs(oi(a) - oi(b))
    an, bn = nan(a), nan(b)
    d = np.where(an & bn, 0, d)
    return np.where(an ^ bn, 1 << 40, d)


def topk_brute(x, k, axis=-1, largest=True):
    """Stable-sort brute force of the tie rule (value order, then lower index);
    NaN ranks as the largest value.  Returns (values, int32 indices)."""
    x = np.asarray(x)
    xm = np.moveaxis(x, axis, -1)
    xf = xm.astype(np.float32)
    nan = np.isnan(xf)
    key = np.where(nan, np.inf, xf) + np.float32(0.0)  # -0 -> +0
    # rank NaN strictly above +inf through a second key
    n = xf.shape[-1]
    idx = np.broadcast_to(np.arange(n), xf.shape)
    if largest:
        order = np.lexsort((idx, -key, ~nan), axis=-1)
    else:
        order = np.lexsort((idx, key, nan), axis=-1)
    order = order[..., :k]
    vals = np.take_along_axis(xm, order, axis=-1)
    return np.moveaxis(vals, -1, axis), np.moveaxis(order.astype(np.int32), -1, axis)


def check_topk_invariants(x, vals, idx, k, largest=True):
    """Structural properties any correct top-k along the last axis has,
    whatever the data: values are copies of x[idx], ordered, indices unique,
    nothing left out beats the k-th, equal values in increasing index order."""
    x = np.asarray(x, dtype=np.float32)
    rows = x.reshape(-1, x.shape[-1])
    v = np.asarray(vals, dtype=np.float32).reshape(rows.shape[0], k)
    ix = np.asarray(idx).reshape(rows.shape[0], k)
    for r in range(rows.shape[0]):
        assert ix[r].min() >= 0 and ix[r].max() < rows.shape[1]
        assert len(set(ix[r].tolist())) == k
        assert np.array_equal(rows[r][ix[r]].view(np.uint32), v[r].view(np.uint32))
        s = v[r] if largest else -v[r]
        assert np.all(s[:-1] >= s[1:])
        same = s[:-1] == s[1:]
        assert np.all(ix[r][1:][same] > ix[r][:-1][same])
        rest = np.ones(rows.shape[1], bool)
        rest[ix[r]] = False
        if rest.any():
            rs = rows[r][rest] if largest else -rows[r][rest]
            assert rs.max() <= s[-1]
            tied = np.nonzero(rest & ((rows[r] if largest else -rows[r]) == s[-1]))[0]
            if tied.size:
                last_sel = ix[r][s == s[-1]].max()
                assert tied.min() > last_sel


def reference_float_tolerance_ok(out, exp):
    """The reference harness's own three-band float32 tolerance
    (tests/setup.hpp:241-263): a floor every result must also meet."""
    out = np.asarray(out, dtype=np.float32).ravel()
    exp = np.asarray(exp, dtype=np.float32).ravel()
    a = np.abs(exp)
    thr = np.where(a > 1.0, a * 0.01, np.where(a > 1e-3, np.maximum(0.003, a * 0.02), 0.002))
    return bool(np.all(~np.isnan(out)) and np.all(np.abs(out - exp) <= thr))


def reference_half_tolerance_ok(out, exp):
    """tests/setup.hpp:215-233: |d| <= max(0.02, 2 %) on the widened halves."""
    out = np.asarray(out).view(np.float16).astype(np.float32).ravel()
    exp = np.asarray(exp).view(np.float16).astype(np.float32).ravel()
    a = np.abs(exp)
    thr = np.where(a > 1.0, a * 0.02, 0.02)
    return bool(np.all(~np.isnan(out)) and np.all(np.abs(out - exp) <= thr))


def check_fused_invariants(x_row, vals_row, idx_row):
    """What any correct fused softmax -> top-k (largest first) of one row satisfies,
    whatever row sum the implementation arrived at, because a probability is a
    non-decreasing function of its logit: returned probabilities do not increase;
    equal returned probabilities come in increasing index order; a larger logit never
    has a smaller returned probability; nothing left out has a logit at or above that
    of a returned entry whose probability exceeds the last one; and anything left out
    whose logit reaches the smallest logit of the last probability's group (it then
    has that same probability) has a higher index than every returned member of the
    group.  Rows holding NaN / +inf (all-NaN results) are not for this check.
    Raises AssertionError naming the property that fails."""
    x = np.asarray(x_row, dtype=np.float32)
    p = np.asarray(vals_row, dtype=np.float32)
    ix = np.asarray(idx_row).astype(np.int64)
    k = len(ix)
    assert len(set(ix.tolist())) == k and ix.min() >= 0 and ix.max() < len(x), "indices not distinct / in range"
    assert np.all(p[:-1] >= p[1:]), "probabilities increase along the result"
    same = p[:-1] == p[1:]
    assert np.all(ix[1:][same] > ix[:-1][same]), "equal probabilities not in increasing index order"
    lx = x[ix]
    order = np.argsort(-lx, kind="stable")
    assert np.all(np.diff(p[order]) <= 0), "a larger logit has a smaller probability"
    rest = np.ones(len(x), bool)
    rest[ix] = False
    if not rest.any():
        return
    last = p[-1]
    group = p == last
    above = ~group
    if above.any():
        assert x[rest].max() < lx[above].min(), "an element left out beats a returned one with a larger probability"
    reach = rest & (x >= lx[group].min())
    if reach.any():
        assert np.nonzero(reach)[0].min() > ix[group].max(), "a tie at the last place was not settled by lower index"


def well_separated_cut(probs_row, logits_row, k, min_ulp=4):
    """True when the row's k+1 largest probabilities (an oracle's) are pairwise either at
    least min_ulp apart or equal with equal logits: then an implementation within a
    couple of ulp of them must return exactly the oracle's indices."""
    pr = np.asarray(probs_row, dtype=np.float32)
    lg = np.asarray(logits_row, dtype=np.float32)
    if np.isnan(pr).any():
        return False
    order = np.lexsort((np.arange(len(pr)), -pr))[:k + 1]
    top, tl = pr[order], lg[order]
    d = ulp_diff(top[:-1], top[1:])
    ok = (d >= min_ulp) | ((d == 0) & (tl[:-1] == tl[1:]))
    return bool(np.all(ok))
