"""Pins the CPU oracle (oracle/vkop_oracle.c) before anything is compared with it.

Sources of truth used here, none of which is the oracle's own formula:
libtorch 2.10.0 CPU results frozen from the reference tests' seeds and shapes
(tests/SoftmaxTest.cpp:193-231, tests/TopkTest.cpp:91-128), numpy's float16
conversions, closed forms, an extended-precision evaluation of the
mathematical softmax on inputs whose differences are exact, a stable-sort brute
force of the tie rule, and structural invariants.
"""
import numpy as np
import pytest

import oracle
from helpers import (check_topk_invariants, half_ulp_diff, reference_float_tolerance_ok,
                     reference_half_tolerance_ok, topk_brute, ulp_diff)

# ----------------------------------------------------------------------------
# binary16 conversions
# ----------------------------------------------------------------------------


def test_half_to_float_exhaustive():
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = oracle.half_to_float(h)
    exp = h.view(np.float16).astype(np.float32)
    nan = np.isnan(exp)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), exp[~nan].view(np.uint32))


def test_float_to_half_against_numpy():
    rng = np.random.default_rng(7)
    pieces = [
        rng.standard_normal(20000).astype(np.float32) * 3,
        (rng.standard_normal(5000) * 1e-5).astype(np.float32),         # half subnormals
        (rng.standard_normal(5000) * 3e4).astype(np.float32),          # near overflow
        rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 65519.99, 65520.0, 65536.0,
                  2.0 ** -24, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                  2.0 ** -14, np.nextafter(np.float32(2.0 ** -14), np.float32(0)), 1e-10, -1e-10], dtype=np.float32),
    ]
    # every half value and the float just above / below every rounding midpoint
    allh = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid = ((allh[:-1].astype(np.float64) + allh[1:].astype(np.float64)) / 2).astype(np.float32)
    pieces += [allh, mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)), -mid]
    x = np.concatenate(pieces)
    got = oracle.float_to_half(x)
    with np.errstate(over="ignore"):
        exp = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x3FF) != 0)
    assert np.array_equal(got[~nan], exp[~nan])


# ----------------------------------------------------------------------------
# softmax
# ----------------------------------------------------------------------------


@pytest.mark.parametrize("case", range(6))
def test_softmax_libtorch_goldens_f32(golden, case):
    x = golden["softmax%d_f32_in" % case]
    exp = golden["softmax%d_f32_out" % case]
    got = oracle.softmax(x, int(golden["softmax%d_axis" % case]))
    assert got.shape == exp.shape
    assert reference_float_tolerance_ok(got, exp)          # the reference's own bar
    # lines are <= 1000 long here, where libtorch's lane-wise float sum is still
    # within a few ulp of an exact sum
    assert ulp_diff(got, exp).max() <= 8, ulp_diff(got, exp).max()


@pytest.mark.parametrize("case", range(6))
def test_softmax_libtorch_goldens_f16(golden, case):
    x = golden["softmax%d_f16_in" % case]
    exp = golden["softmax%d_f16_out" % case]
    got = oracle.softmax(x.view(np.float16), int(golden["softmax%d_axis" % case]))
    assert reference_half_tolerance_ok(got, exp)
    assert half_ulp_diff(got, exp).max() <= 1


def test_softmax_closed_forms():
    for n in list(range(1, 70)) + [127, 128, 129, 1000, 4097]:
        for c in (0.0, -3.25, 100.0, -1e30):
            y = oracle.softmax(np.full((2, n), c, np.float32))
            assert np.all(y.view(np.uint32) == np.float32(1.0 / n).view(np.uint32)), (n, c)
    # two elements: logistic function, evaluated in extended precision
    d = np.linspace(-30, 30, 241).astype(np.float32)
    x = np.stack([d, np.zeros_like(d)], axis=1)
    y = oracle.softmax(x)
    ld = d.astype(np.longdouble)
    exact0 = (1 / (1 + np.exp(-ld)))
    exact1 = (1 / (1 + np.exp(ld)))
    assert ulp_diff(y[:, 0], exact0.astype(np.float32)).max() <= 1
    assert ulp_diff(y[:, 1], exact1.astype(np.float32)).max() <= 1
    # a dominant element: the rest underflow to exactly zero
    x = np.zeros((1, 50), np.float32)
    x[0, 17] = 200.0
    y = oracle.softmax(x)
    assert y[0, 17] == 1.0 and np.count_nonzero(y) == 1


def test_softmax_extended_precision_brute_force():
    """Inputs on a 2^-10 grid in [-8, 8]: x - max is exact in float32, so the
    mathematical softmax evaluated in 80-bit arithmetic is the target; the
    oracle may differ only by its float exp rounding and the final rounding."""
    rng = np.random.default_rng(11)
    for shape, axis in [((7, 33), 1), ((5, 12, 9), 1), ((3, 4, 5, 6), 2), ((300,), 0), ((2, 3, 4, 5), 0), ((6, 513), -1)]:
        x = (rng.integers(-8192, 8193, size=shape).astype(np.float32) / np.float32(1024))
        y = oracle.softmax(x, axis)
        xl = x.astype(np.longdouble)
        e = np.exp(xl - xl.max(axis=axis, keepdims=True))
        exact = e / e.sum(axis=axis, keepdims=True)
        assert ulp_diff(y, exact.astype(np.float32)).max() <= 1, (shape, axis)
        assert np.all(np.abs(y.astype(np.float64).sum(axis=axis) - 1) <= x.shape[axis] * 2.0 ** -24)


def test_softmax_invariants():
    rng = np.random.default_rng(12)
    x = rng.standard_normal((9, 257)).astype(np.float32)
    y = oracle.softmax(x)
    # shifting by a constant that keeps every x + c exact changes nothing
    xs = (rng.integers(-4096, 4096, size=(9, 257)).astype(np.float32) / np.float32(256))
    assert np.array_equal(oracle.softmax(xs).view(np.uint32), oracle.softmax(xs + np.float32(64)).view(np.uint32))
    # permuting a line permutes the result (double sum order may move the last bit)
    perm = rng.permutation(257)
    assert ulp_diff(oracle.softmax(x[:, perm]), y[:, perm]).max() <= 1
    # monotone in x within a line
    for r in range(9):
        o = np.argsort(x[r], kind="stable")
        assert np.all(np.diff(y[r][o]) >= 0)
    # a strided axis is the last-axis result moved back
    x4 = rng.standard_normal((2, 5, 7, 3)).astype(np.float32)
    for ax in range(4):
        via_last = np.moveaxis(oracle.softmax(np.ascontiguousarray(np.moveaxis(x4, ax, -1))), -1, ax)
        assert np.array_equal(oracle.softmax(x4, ax).view(np.uint32), np.ascontiguousarray(via_last).view(np.uint32))
    # rank 1 is one line (ops/Softmax.hpp:116-120)
    assert np.array_equal(oracle.softmax(x[0]).view(np.uint32), y[0].view(np.uint32))


def test_softmax_special_values():
    x = np.array([[1.0, np.nan, 2.0], [1.0, np.inf, 2.0], [-np.inf, 0.0, 0.0], [-np.inf, -np.inf, -np.inf]], np.float32)
    with np.errstate(invalid="ignore"):
        y = oracle.softmax(x)
    assert np.all(np.isnan(y[0])) and np.all(np.isnan(y[1])) and np.all(np.isnan(y[3]))
    assert np.array_equal(y[2], np.array([0.0, 0.5, 0.5], np.float32))
    with np.errstate(invalid="ignore"):
        y = oracle.softmax(x, nan_where=1, nan_value=0.25)
    assert np.all(y[0] == 0.25) and np.all(y[3] == 0.25) and np.array_equal(y[2], np.array([0.0, 0.5, 0.5], np.float32))


# ----------------------------------------------------------------------------
# top-k
# ----------------------------------------------------------------------------


def _tie_free(row_vals_kplus1):
    return len(np.unique(row_vals_kplus1)) == len(row_vals_kplus1)


@pytest.mark.parametrize("tag", ["f32", "f16"])
@pytest.mark.parametrize("case", range(5))
def test_topk_libtorch_goldens(golden, case, tag):
    x = golden["topk%d_%s_in" % (case, tag)]
    k = int(golden["topk%d_k" % case])
    xin = x.view(np.float16) if tag == "f16" else x
    v, ix = oracle.topk(xin, k, int(golden["topk%d_axis" % case]), True)
    ev, eix = golden["topk%d_%s_val" % (case, tag)], golden["topk%d_%s_idx" % (case, tag)]
    vb = v.view(np.uint16) if tag == "f16" else v.view(np.uint32)
    eb = ev if tag == "f16" else ev.view(np.uint32)
    assert np.array_equal(vb, eb)                      # values: always bit-equal
    compared = 0
    for r in range(x.shape[0]):
        top = np.sort(xin[r].astype(np.float32))[::-1][:k + 1]
        if _tie_free(top):                             # libtorch's tie order is not a target
            assert np.array_equal(ix[r], eix[r])
            compared += 1
    if tag == "f32":
        assert compared == x.shape[0]                  # randn float32 rows are tie free


def test_topk_brute_force_ties_axes_and_smallest():
    rng = np.random.default_rng(21)
    cases = [((4, 300), 1, 17), ((4, 300), 0, 3), ((3, 40, 5), 1, 40), ((2, 3, 64, 4), 2, 9), ((500,), 0, 1), ((6, 64), -1, 64)]
    for shape, axis, k in cases:
        for largest in (True, False):
            x = (rng.integers(-6, 7, size=shape).astype(np.float32) / np.float32(4))   # heavy ties
            x.ravel()[rng.integers(0, x.size, 3)] = -0.0
            v, ix = oracle.topk(x, k, axis, largest)
            bv, bix = topk_brute(x, k, axis, largest)
            assert np.array_equal(ix, bix), (shape, axis, k, largest)
            assert np.array_equal(v.view(np.uint32), bv.view(np.uint32))
            xm = np.ascontiguousarray(np.moveaxis(x, axis, -1))
            check_topk_invariants(xm, np.moveaxis(v, axis, -1), np.moveaxis(ix, axis, -1), k, largest)
    # half precision rows
    xh = (rng.standard_normal((5, 777)) * 2).astype(np.float16)
    v, ix = oracle.topk(xh, 33)
    bv, bix = topk_brute(xh, 33)
    assert np.array_equal(ix, bix) and np.array_equal(v.view(np.uint16), bv.view(np.uint16))


def test_topk_nan_inf_ranking():
    x = np.array([[1.0, np.nan, np.inf, -np.inf, 3.0, np.nan, -0.0, 0.0]], np.float32)
    v, ix = oracle.topk(x, 8, -1, True)
    assert ix[0].tolist() == [1, 5, 2, 4, 0, 6, 7, 3]
    v, ix = oracle.topk(x, 8, -1, False)
    assert ix[0].tolist() == [3, 6, 7, 0, 4, 2, 1, 5]
    bv, bix = topk_brute(x, 8, -1, True)
    assert bix[0].tolist() == [1, 5, 2, 4, 0, 6, 7, 3]
    v, ix = oracle.topk(x, 0)
    assert v.shape == (1, 0)


def test_topk_downsized_grid_workload(golden):
    x, k = golden["c4_in"], int(golden["c4_k"])
    v, ix = oracle.topk(x, k)
    assert np.array_equal(v.view(np.uint32), golden["c4_val"].view(np.uint32))   # libtorch values
    bv, bix = topk_brute(x, k)
    assert np.array_equal(ix, bix)
    check_topk_invariants(x, v, ix, k)


# ----------------------------------------------------------------------------
# fused softmax -> top-k, reduce max, CPU post-proc restatement
# ----------------------------------------------------------------------------


@pytest.mark.parametrize("name", ["c1", "c2", "c3"])
def test_fused_against_libtorch(golden, name):
    x, k = golden[name + "_in"], int(golden[name + "_k"])
    v, ix, p = oracle.softmax_topk(x, k, return_probs=True)
    # composition property: exactly top-k of the oracle's own softmax
    assert np.array_equal(p.view(np.uint32), oracle.softmax(x).view(np.uint32))
    bv, bix = topk_brute(p, k)
    assert np.array_equal(ix, bix) and np.array_equal(v.view(np.uint32), bv.view(np.uint32))
    ev, eix = golden[name + "_val"], golden[name + "_idx"]
    assert reference_float_tolerance_ok(v, ev)
    assert ulp_diff(v, ev).max() <= (8 if x.shape[-1] <= 1000 else 64)
    for r in range(x.shape[0]):
        if _tie_free(np.sort(p[r])[::-1][:k + 1]) and _tie_free(ev[r]):
            assert np.array_equal(ix[r], eix[r])


def test_fused_half_against_libtorch(golden):
    x, k = golden["c2h_in"].view(np.float16), int(golden["c2h_k"])
    v, ix, p = oracle.softmax_topk(x, k, return_probs=True)
    assert half_ulp_diff(p, golden["c2h_prob"]).max() <= 1
    assert half_ulp_diff(v, golden["c2h_val"]).max() <= 1
    bv, bix = topk_brute(p, k)
    assert np.array_equal(ix, bix)


def test_detection_style_chain(golden):
    x, k = golden["c5_in"], int(golden["c5_k"])
    p = oracle.softmax(x, 1)
    m = oracle.reduce_max(p, 1)
    assert np.array_equal(m, p.max(axis=1))
    assert ulp_diff(m, golden["c5_max"]).max() <= 8
    v, ix = oracle.topk(m, k)
    for r in range(x.shape[0]):
        if _tie_free(np.sort(m[r])[::-1][:k + 1]) and np.array_equal(np.argsort(-golden["c5_max"][r], kind="stable")[:k], golden["c5_idx"][r]):
            # same ordering whenever neither side has ties and the few-ulp
            # differences do not swap neighbours
            if np.array_equal(np.argsort(-m[r], kind="stable")[:k], golden["c5_idx"][r]):
                assert np.array_equal(ix[r], golden["c5_idx"][r])
    # the class max of a softmax column is 1 / sum(exp(x - max))
    xm = x.max(axis=1, keepdims=True)
    s = np.exp((x - xm).astype(np.float64)).sum(axis=1)
    assert ulp_diff(m, (1.0 / s).astype(np.float32)).max() <= 2


def test_reduce_max_nan():
    x = np.array([[1.0, np.nan], [3.0, 2.0]], np.float32)
    m = oracle.reduce_max(x, 0)
    assert m[0] == 3.0 and np.isnan(m[1])


def test_get_top_k_predictions(golden):
    x = golden["c1_in"][0]
    got = oracle.get_top_k_predictions(x, 5)
    e = np.exp(x - x.max(), dtype=np.float32)
    s = np.float32(0)
    for t in e:                      # sequential float sum, core/function.cpp:157-160
        s = np.float32(s + t)
    p = (e / s).astype(np.float32)
    order = np.argsort(-p, kind="stable")[:5]
    assert [g[0] for g in got] == order.tolist()
    # libm expf vs numpy's float exp may differ in the last bit
    assert ulp_diff(np.array([g[1] for g in got], np.float32), p[order]).max() <= 2
    assert [g[0] for g in got] == golden["c1_idx"][0].tolist()
    assert len(oracle.get_top_k_predictions(x[:3], 5)) == 3


# ---- non-maximum suppression (the detection chain's last operator) -------------------------------

def _reference_like_boxes(rng, B, N):
    """Boxes the way tests/NmsTest.cpp:38-56 draws them: centre in [0,1)^2, size in [0,1.3)^2, clamped."""
    c = rng.random((B, N, 2)).astype(np.float32)
    s = (rng.random((B, N, 2)) * 1.3).astype(np.float32)
    lo = np.clip(c - s / 2, 0.0, 1.0)
    hi = np.clip(c + s / 2, 0.0, 1.0)
    return np.concatenate([lo, hi], axis=-1).astype(np.float32)


def _nms_like_the_reference_test(boxes, scores, iou_threshold, score_threshold):
    """The expectation tests/NmsTest.cpp:62-160 computes, written with whole-array
    operations (argsort + an IoU matrix) instead of its nested scalar loops."""
    out = []
    B, C, N = scores.shape
    for b in range(B):
        bx = boxes[b].astype(np.float32)
        area = (bx[:, 2] - bx[:, 0]) * (bx[:, 3] - bx[:, 1])
        w = np.maximum(np.float32(0), np.minimum(bx[:, None, 2], bx[None, :, 2]) - np.maximum(bx[:, None, 0], bx[None, :, 0]))
        h = np.maximum(np.float32(0), np.minimum(bx[:, None, 3], bx[None, :, 3]) - np.maximum(bx[:, None, 1], bx[None, :, 1]))
        inter = (w * h).astype(np.float32)
        union = (area[:, None] + area[None, :] - inter).astype(np.float32)
        iou = np.where(union > np.float32(1e-8), inter / np.where(union > 0, union, 1), 0).astype(np.float32)
        for c in range(C):
            order = np.argsort(-scores[b, c], kind="stable")
            order = order[scores[b, c][order] >= score_threshold]
            alive = np.ones(len(order), bool)
            for p, i in enumerate(order):
                if not alive[p]:
                    continue
                out.append((b, c, int(i)))
                alive[p + 1:] &= ~(iou[i, order[p + 1:]] > iou_threshold)
    return np.array(out, dtype=np.int32).reshape(-1, 3)


@pytest.mark.parametrize("box_shape,score_shape,max_per_class,iou_thr,score_thr", [
    ((1, 10, 4), (1, 2, 10), 0, 0.5, 0.5), ((1, 200, 4), (1, 1, 200), 0, 0.7, 0.4), ((1, 50, 4), (1, 7, 50), 0, 0.3, 0.2),
    ((3, 300, 4), (3, 5, 300), 0, 0.45, 0.25)])
def test_nms_matches_the_reference_tests_expectation(box_shape, score_shape, max_per_class, iou_thr, score_thr):
    """Shapes and thresholds of tests/NmsTest.cpp:165-169 (its expectation ignores the per-class limit, so 0 here)."""
    rng = np.random.default_rng(box_shape[1])
    boxes = _reference_like_boxes(rng, box_shape[0], box_shape[1])
    scores = rng.random(score_shape).astype(np.float32)
    got = oracle.nms(boxes, scores, iou_thr, score_thr, max_per_class)
    want = _nms_like_the_reference_test(boxes, scores, np.float32(iou_thr), np.float32(score_thr))
    assert np.array_equal(got, want)


def test_nms_invariants_and_closed_forms():
    rng = np.random.default_rng(9)
    boxes = _reference_like_boxes(rng, 2, 120)
    scores = rng.random((2, 3, 120)).astype(np.float32)
    sel = oracle.nms(boxes, scores, 0.4, 0.3)

    def iou(a, b):
        x1, y1, x2, y2 = max(a[0], b[0]), max(a[1], b[1]), min(a[2], b[2]), min(a[3], b[3])
        if x2 <= x1 or y2 <= y1:
            return 0.0
        inter = (x2 - x1) * (y2 - y1)
        return inter / ((a[2] - a[0]) * (a[3] - a[1]) + (b[2] - b[0]) * (b[3] - b[1]) - inter)
    for b in range(2):
        for c in range(3):
            mine = [int(r[2]) for r in sel if r[0] == b and r[1] == c]
            s = scores[b, c]
            assert all(s[i] > 0.3 for i in mine) and list(s[mine]) == sorted(s[mine], reverse=True)
            for p, i in enumerate(mine):                       # no two selected boxes overlap too much
                assert all(iou(boxes[b, i], boxes[b, j]) <= 0.4 + 1e-6 for j in mine[:p])
            for j in np.nonzero(s > 0.3)[0]:                   # every rejected candidate lost to a better selected box
                if j not in mine:
                    assert any(s[i] >= s[j] and iou(boxes[b, i], boxes[b, j]) > 0.4 - 1e-6 for i in mine)
    # identical boxes: only the best survives; disjoint boxes: all, best first
    same = np.tile(np.array([[0.1, 0.1, 0.6, 0.7]], np.float32), (1, 8, 1))
    sc = np.array([[[0.3, 0.9, 0.5, 0.7, 0.2, 0.8, 0.6, 0.4]]], np.float32)
    assert oracle.nms(same, sc, 0.5, 0.0).tolist() == [[0, 0, 1]]
    apart = np.array([[[i, 0, i + 0.5, 1] for i in range(8)]], np.float32)
    assert oracle.nms(apart, sc, 0.5, 0.0)[:, 2].tolist() == [1, 5, 3, 6, 2, 7, 0, 4]
    # IoU can never exceed 1: a threshold of 1 keeps every candidate; a score threshold above all keeps none
    assert len(oracle.nms(same, sc, 1.0, 0.25)) == 7 and len(oracle.nms(same, sc, 0.5, 0.95)) == 0
    # per-class limit, centre format, candidate limit (the first by box index)
    assert oracle.nms(apart, sc, 0.5, 0.0, max_output_boxes_per_class=3)[:, 2].tolist() == [1, 5, 3]
    centre = np.stack([(apart[..., 0] + apart[..., 2]) / 2, (apart[..., 1] + apart[..., 3]) / 2,
                       apart[..., 2] - apart[..., 0], apart[..., 3] - apart[..., 1]], -1).astype(np.float32)
    assert np.array_equal(oracle.nms(centre, sc, 0.5, 0.0, center_point_box=1), oracle.nms(apart, sc, 0.5, 0.0))
    assert oracle.nms(apart, sc, 0.5, 0.0, max_candidates=4)[:, 2].tolist() == [1, 3, 2, 0]


# ---- nucleus (top-p) cut: not in the reference, pinned on closed forms and numpy's sequential cumsum --------------

def test_topp_count_closed_forms_and_cumsum():
    eighths = np.full((1, 8), 0.125, dtype=np.float32)              # every partial sum exact
    for p, want in [(0.0, 1), (0.125, 1), (0.126, 2), (0.5, 4), (0.51, 5), (1.0, 8), (1.5, 8), (-1.0, 1)]:
        assert oracle.topp_count(eighths, p).tolist() == [want], p
    rng = np.random.default_rng(3)
    x = rng.standard_normal((64, 4000)).astype(np.float32) * 3
    probs = oracle.softmax(x, -1)
    v, _ = oracle.topk(probs, 50, -1)
    running = np.cumsum(v, axis=-1, dtype=np.float32)               # numpy accumulates front to back in float32
    last = 0
    for p in (0.05, 0.3, 0.5, 0.8, 0.9, 0.99, 1.0):
        got = oracle.topp_count(v, p)
        reached = running >= np.float32(p)
        want = np.where(reached.any(axis=-1), reached.argmax(axis=-1) + 1, 50)
        assert np.array_equal(got, want), p
        assert (got >= last).all()                                  # a larger p never needs fewer values
        last = got
    bad = v.copy()
    bad[3, 2] = np.nan                                              # a NaN in the sum: nothing is ever reached after it
    assert oracle.topp_count(bad, 0.9999)[3] == 50
    half = v.astype(np.float16)
    assert np.array_equal(oracle.topp_count(half, 0.7), oracle.topp_count(half.astype(np.float32), 0.7))


# ------------------------------------------------ sampling-style fused variant --

def test_sampling_variant_scale_and_count_pins():
    """vkop_oracle_softmax_topk_sampling_*: not the formula retyped, but facts that fix it.
    scale = 1 is the plain fused oracle bit for bit; a power-of-two scale multiplies
    exactly, so the result is the plain oracle's on numpy's ldexp of the input; any scale
    is the plain oracle on numpy's own float32 product (one rounding per element, done by
    another implementation); the counts are topp_count (pinned above) on the returned
    values, with its closed forms: p <= first value -> 1, p above the total -> k."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((6, 3000)) * 2).astype(np.float32)
    x[1, ::7] = x[1, 3]                      # ties
    x[2, 100:] = -np.inf                     # fewer finite elements than most k
    for k in (1, 7, 50):
        v1, i1 = oracle.softmax_topk_sampling(x, k, 1.0)
        ev, ei = oracle.softmax_topk(x, k)
        assert np.array_equal(i1, ei) and np.array_equal(v1.view(np.uint32), ev.view(np.uint32))
        for j in (-2, 1, 3):
            v2, i2 = oracle.softmax_topk_sampling(x, k, 2.0 ** j)
            ev, ei = oracle.softmax_topk(np.ldexp(x, j).astype(np.float32), k)
            assert np.array_equal(i2, ei) and np.array_equal(v2.view(np.uint32), ev.view(np.uint32)), (k, j)
        for scale in (1.25, 0.7, 3.3333333):
            v3, i3, c3 = oracle.softmax_topk_sampling(x, k, scale, top_p=0.9)
            xs = (x * np.float32(scale)).astype(np.float32)
            ev, ei = oracle.softmax_topk(xs, k)
            assert np.array_equal(i3, ei) and np.array_equal(v3.view(np.uint32), ev.view(np.uint32)), (k, scale)
            assert np.array_equal(c3, oracle.topp_count(v3, 0.9))
        _, _, c = oracle.softmax_topk_sampling(x, k, 1.25, top_p=0.0)
        assert np.all(c == 1)
        _, _, c = oracle.softmax_topk_sampling(x, k, 1.25, top_p=1.5)
        assert np.all(c == k)
    # half precision: the same facts on the widened halves
    xh = x[:3].astype(np.float16)
    v, i = oracle.softmax_topk_sampling(xh, 9, 1.0)
    ev, ei = oracle.softmax_topk(xh, 9)
    assert np.array_equal(i, ei) and np.array_equal(v.view(np.uint16), ev.view(np.uint16))
    v, i, c = oracle.softmax_topk_sampling(xh, 9, 2.0, top_p=0.5)
    x2 = (xh.astype(np.float32) * np.float32(2.0)).astype(np.float16)   # exact in half away from overflow
    ev, ei = oracle.softmax_topk(x2, 9)
    assert np.array_equal(i, ei) and np.array_equal(v.view(np.uint16), ev.view(np.uint16))
    assert np.array_equal(c, oracle.topp_count(v.astype(np.float32), 0.5))


def test_fused_invariant_check_catches_a_wrong_tie_break():
    """tests/helpers.py: check_fused_invariants accepts the oracle's results and refuses a
    result whose tie at the last place went to a higher index, an entry left out that
    beats a returned one, and equal probabilities out of index order."""
    from helpers import check_fused_invariants, well_separated_cut
    rng = np.random.default_rng(0)
    x = (np.round(rng.standard_normal((4, 5000)) * 8) / 8).astype(np.float32)   # many equal logits
    v, ix = oracle.softmax_topk(x, 50)
    for r in range(4):
        check_fused_invariants(x[r], v[r], ix[r])
    r = 0
    group = np.nonzero(v[r] == v[r, -1])[0]
    level = x[r, ix[r, group]].min()
    left_out = [j for j in np.nonzero(x[r] == level)[0] if j not in ix[r]]
    assert left_out, "the case needs a tie across the last place"
    wrong = ix[r].copy()
    wrong[-1] = max(left_out)                               # same probability, higher index
    with pytest.raises(AssertionError, match="lower index"):
        check_fused_invariants(x[r], v[r], wrong)
    wrong = ix[r].copy()
    wrong[0] = int(np.argmin(x[r]))                         # the row's best element left out for its worst
    with pytest.raises(AssertionError):
        check_fused_invariants(x[r], v[r], wrong)
    pair = np.nonzero(v[r][:-1] == v[r][1:])[0]
    if pair.size:
        wrong = ix[r].copy()
        a = pair[0]
        wrong[a], wrong[a + 1] = wrong[a + 1], wrong[a]
        with pytest.raises(AssertionError, match="increasing index"):
            check_fused_invariants(x[r], v[r], wrong)
    y = rng.standard_normal((1, 4000)).astype(np.float32)
    assert well_separated_cut(oracle.softmax(y)[0], y[0], 10, 1) in (True, False)
    y[0, :20] = 9.0                                          # ties through equal logits count as separated
    assert well_separated_cut(oracle.softmax(y)[0], y[0], 10)
