"""Parity of the HIP path (through the C ABI) with the CPU oracle, on the GPU.

Bars: top-k indices and values bit-exact; float32 softmax within 2 ulp of the
oracle (correctly rounded exp terms, double sum); float16 within 1e-3 relative
(in practice 1 half ulp).  The distance to libtorch's own CPU softmax is
reported through the reference harness's tolerance, not gated tighter: libtorch
sums in ISA-dependent float lanes and is itself many ulp from an exact sum on
long rows.
"""
import os

import numpy as np
import pytest

import oracle
from helpers import (check_fused_invariants, check_topk_invariants, half_ulp_diff, reference_float_tolerance_ok,
                     reference_half_tolerance_ok, ulp_diff, well_separated_cut)
from vkop_amd import synth

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def ops():
    from vkop_amd import capi, ops as _ops
    capi.lib()              # raises if the HIP library is not built: no fallback
    capi.init(0)
    return _ops


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        a = a.view(np.float16)
    return torch.from_numpy(a).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def assert_softmax_close(got, x, axis, what=""):
    exp = oracle.softmax(x, axis)
    if got.dtype == np.float16:
        assert half_ulp_diff(got, exp).max() <= 1, what
        g, e = got.astype(np.float32), exp.astype(np.float32)
        with np.errstate(invalid="ignore"):
            ok = (np.abs(g - e) <= 1e-3 * np.abs(e) + 6e-8) | (np.isnan(g) & np.isnan(e))
        assert ok.all(), what
    else:
        d = ulp_diff(got, exp)
        assert d.max() <= 2, "%s: %d ulp" % (what, d.max())


# ------------------------------------------------------------------ softmax --

@pytest.mark.parametrize("tag", ["f32", "f16"])
@pytest.mark.parametrize("case", range(6))
def test_softmax_reference_test_shapes(ops, golden, case, tag):
    """tests/SoftmaxTest.cpp:193-231: same shapes, axes, seed-42 inputs."""
    x = golden["softmax%d_%s_in" % (case, tag)]
    axis = int(golden["softmax%d_axis" % case])
    xin = x.view(np.float16) if tag == "f16" else x
    got = host(ops.softmax(dev(xin), axis))
    assert got.shape == x.shape
    assert_softmax_close(got, xin, axis, "case %d %s" % (case, tag))
    exp = golden["softmax%d_%s_out" % (case, tag)]
    if tag == "f16":
        assert reference_half_tolerance_ok(got, exp)
    else:
        assert reference_float_tolerance_ok(got, exp)
        assert ulp_diff(got, exp).max() <= 8


@pytest.mark.parametrize("n", [1, 2, 3, 5, 63, 64, 65, 255, 256, 257, 1000, 1023, 1024, 4097, 20001])
def test_softmax_ragged_lengths(ops, n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal((3, n)) * 3).astype(np.float32)
    assert_softmax_close(host(ops.softmax(dev(x))), x, -1, "n=%d" % n)
    xh = x.astype(np.float16)
    assert_softmax_close(host(ops.softmax(dev(xh))), xh, -1, "n=%d half" % n)


@pytest.mark.parametrize("shape", [(1001, 197), (7, 64), (4099, 33), (513, 512), (12, 5, 197, 197), (70000, 8)])
def test_softmax_many_short_rows(ops, shape):
    """Rows of up to 512 elements take a wave each, four rows a workgroup: row counts that
    are not a multiple of four, rows that do not start on 16 bytes, an attention-shaped
    tensor, rows shorter than a wave; a NaN row, a +inf row and a row of -inf among them."""
    rng = np.random.default_rng(shape[0] + shape[-1])
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    flat = x.reshape(-1, shape[-1])
    flat[1, shape[-1] // 2] = np.nan
    flat[2, 0] = np.inf
    flat[3, :] = -np.inf
    assert_softmax_close(host(ops.softmax(dev(x))), x, -1, str(shape))
    xh = x.astype(np.float16)
    assert_softmax_close(host(ops.softmax(dev(xh))), xh, -1, str(shape) + " half")


@pytest.mark.parametrize("shape,axis", [((5, 7, 9), 0), ((5, 7, 9), 1), ((5, 7, 9), 2), ((2, 3, 4, 5), 0), ((2, 3, 4, 5), 1),
                                        ((2, 3, 4, 5), -2), ((300,), 0), ((4, 2500, 3), 1), ((3, 70, 130), 1), ((2, 5, 64), 1),
                                        ((2, 1000, 64), 1), ((1, 4096, 300), 1), ((2, 200, 7, 5), 1), ((3, 129, 2), 1),
                                        ((2, 777, 65), 1), ((5000, 33), 0), ((1, 8192, 3), 1), ((300, 200, 64), 1),
                                        ((40, 1000, 16), 1), ((1, 4100, 130), -2)])
def test_softmax_axes(ops, shape, axis):
    """Every axis of small tensors; lines along a non-last axis short (held in registers) and
    long (a tile of lines per workgroup, and -- with few tiles -- the tile's rows split over
    several workgroups in two launches), with tiles and row chunks that end ragged."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    if x.size > 4000:   # a NaN line, a +inf line, a line of -inf
        xv = np.moveaxis(x, axis, -1)
        xv[..., 0, 5] = np.nan
        xv[..., 1, 3] = np.inf
        xv[..., 2, :] = -np.inf
    assert_softmax_close(host(ops.softmax(dev(x), axis)), x, axis, str((shape, axis)))
    xh = x.astype(np.float16)
    assert_softmax_close(host(ops.softmax(dev(xh), axis)), xh, axis, str((shape, axis)) + " half")


@pytest.mark.parametrize("shape,axis", [((4096, 64), -1), ((4096, 1024), -1), ((8192, 512), -1), ((300, 2048), -1), ((64, 40000), -1),
                                        ((16, 80, 840), 1), ((2, 1000, 64), 1), ((8, 4096, 64), 1)])
def test_softmax_half_near_rounding_boundaries(ops, shape, axis):
    """Half tensors take their terms from the single-precision exponential (about 2^-22 relative
    before the rounding to 11 bits) and scale them in single precision.  Where the exact
    probability -- worked out here in float64 -- lies within 2^-14 relative of the boundary
    between two halves, either neighbour is a result within the bar (one unit of a half against
    the oracle); away from the boundaries the result must be the oracle's own, on every kernel
    that writes half tensors (a wave a row, a wave a row with 128-bit loads, a workgroup a row,
    chunked rows, strided lines in registers and in tiles, tiles split over workgroups)."""
    rng = np.random.default_rng(shape[0] * 7 + shape[-1])
    x = (rng.standard_normal(shape) * 2.5).astype(np.float16)
    got = host(ops.softmax(dev(x), axis))
    exp = oracle.softmax(x, axis)
    x64 = np.moveaxis(x.astype(np.float64), axis, -1)
    e64 = np.exp(x64 - x64.max(-1, keepdims=True))
    p64 = np.moveaxis(e64 / e64.sum(-1, keepdims=True), -1, axis)
    # distance of the exact probability to the nearest boundary between two halves, in units of its own size
    lo = p64.astype(np.float16)
    lo = np.where(lo.astype(np.float64) > p64, np.nextafter(lo, np.float16(0)), lo)     # the half at or below
    hi = np.nextafter(lo, np.float16(1))
    mid = (lo.astype(np.float64) + hi.astype(np.float64)) / 2
    near = np.abs(p64 - mid) <= p64 * 2.0 ** -14
    d = half_ulp_diff(got, exp)
    assert d.max() <= 1, "%s: %d units of a half" % (shape, d.max())
    assert near.sum() > 50, "the case holds no probability near a boundary"
    assert np.all(d[~near] == 0), "%s: %d results away from every boundary differ from the oracle" % (shape, int((d[~near] != 0).sum()))
    assert (d != 0).mean() < 0.01


@pytest.mark.parametrize("shape,axis", [((128, 33000), -1), ((16, 131072), -1), ((64, 40000), -1), ((8, 4096, 256), 1),
                                        ((32, 1000, 64), 1), ((300, 200, 64), 1), ((4096, 1024), -1)])
def test_softmax_of_one_repeated_value_and_a_few_peaks(ops, shape, axis):
    """Lines that are one value but for a peak in five thousand elements: the sum is that value's
    term times its count, the term being the float exponential of the ROUNDED difference to the
    maximum; the kernels that sum chunks against their own maxima count the copies of one value
    apart (the chunk's smallest; for strided tiles the line's first element in the chunk, where
    the second equals it), so that they enter the sum as defined (4 ulp otherwise)."""
    rng = np.random.default_rng(len(shape) + shape[-1])
    x = np.full(shape, 0.25, np.float32)
    x.ravel()[rng.integers(0, x.size, max(1, x.size // 5000))] = 6.0
    x.ravel()[rng.integers(0, x.size, 3)] = -np.inf
    assert_softmax_close(host(ops.softmax(dev(x), axis)), x, axis, str(shape))
    y = (x * np.float32(-1.0)).astype(np.float32)      # the repeated value on top, the rest far below
    y[np.isinf(y)] = -np.inf
    assert_softmax_close(host(ops.softmax(dev(y), axis)), y, axis, str(shape) + " flipped")


def test_softmax_special_values_and_nan_option(ops):
    x = np.zeros((5, 130), np.float32)
    x[0, 7] = np.nan
    x[1, 9] = np.inf
    x[2, :] = -np.inf
    x[3, 3] = -np.inf
    x[4, 100] = 300.0
    with np.errstate(invalid="ignore"):
        exp = oracle.softmax(x)
        expn = oracle.softmax(x, nan_where=1, nan_value=0.125)
    got = host(ops.softmax(dev(x)))
    assert np.array_equal(np.isnan(got), np.isnan(exp))
    assert ulp_diff(got, exp).max() <= 2
    assert got[4, 100] == 1.0 and np.count_nonzero(got[4]) == 1 and got[3, 3] == 0.0
    gotn = host(ops.softmax(dev(x), nan_where=True, nan_value=0.125))
    assert not np.isnan(gotn).any() and ulp_diff(gotn, expn).max() <= 2
    # all-equal rows give exactly 1/n
    c = np.full((2, 777), -3.5, np.float32)
    assert np.all(host(ops.softmax(dev(c))) == np.float32(1.0 / 777))


def test_softmax_in_place(ops):
    x = synth.classifier_logits(16, 1000, seed=3)
    xd = dev(x)
    ops.softmax(xd, out=xd)
    assert_softmax_close(host(xd), x, -1)


def test_softmax_workloads(ops):
    x2 = synth.classifier_logits(256, 1000, synth.SEEDS["C2"])
    assert_softmax_close(host(ops.softmax(dev(x2))), x2, -1, "C2 f32")
    x2h = x2.astype(np.float16)
    assert_softmax_close(host(ops.softmax(dev(x2h))), x2h, -1, "C2 f16")
    x3 = synth.llm_logits(64, 128256, synth.SEEDS["C3"])
    got = host(ops.softmax(dev(x3)))
    assert_softmax_close(got, x3, -1, "C3")
    assert np.abs(got.astype(np.float64).sum(-1) - 1).max() < 1e-5
    x4 = synth.grid_values(8, 262144, synth.SEEDS["C4"])
    assert_softmax_close(host(ops.softmax(dev(x4))), x4, -1, "C4")
    x5 = synth.detection_scores(16, 80, 8400, synth.SEEDS["C5"])
    assert_softmax_close(host(ops.softmax(dev(x5), 1)), x5, 1, "C5")


# -------------------------------------------------------------------- top-k --

def assert_topk_exact(ops, x, k, axis=-1, largest=True):
    v, ix = ops.topk(dev(x), k, axis, largest)
    v, ix = host(v), host(ix)
    ev, eix = oracle.topk(x, k, axis, largest)
    assert ix.dtype == np.int32 and ix.shape == eix.shape
    assert np.array_equal(ix, eix), (x.shape, k, axis, largest)
    bits = np.uint16 if x.dtype == np.float16 else np.uint32
    assert np.array_equal(v.view(bits), ev.view(bits))
    return v, ix


@pytest.mark.parametrize("tag", ["f32", "f16"])
@pytest.mark.parametrize("case", range(5))
def test_topk_reference_test_shapes(ops, golden, case, tag):
    """tests/TopkTest.cpp:91-128: same shapes, k, seed-56 inputs; libtorch's
    values always, its indices on rows without ties."""
    x = golden["topk%d_%s_in" % (case, tag)]
    k = int(golden["topk%d_k" % case])
    xin = x.view(np.float16) if tag == "f16" else x
    v, ix = assert_topk_exact(ops, xin, k, int(golden["topk%d_axis" % case]))
    ev, eix = golden["topk%d_%s_val" % (case, tag)], golden["topk%d_%s_idx" % (case, tag)]
    assert np.array_equal(v.view(ev.dtype) if tag == "f16" else v.view(np.uint32), ev if tag == "f16" else ev.view(np.uint32))
    for r in range(x.shape[0]):
        top = np.sort(xin[r].astype(np.float32))[::-1][:k + 1]
        if len(np.unique(top)) == len(top):
            assert np.array_equal(ix[r], eix[r])


@pytest.mark.parametrize("shape,axis,k", [((4, 300), 1, 17), ((4, 300), 0, 3), ((3, 40, 5), 1, 40), ((2, 3, 64, 4), 2, 9),
                                          ((500,), 0, 1), ((6, 64), -1, 64), ((2, 5000), -1, 2048), ((3, 1), -1, 1),
                                          ((2, 70000), -1, 100), ((5, 257), -1, 256)])
def test_topk_ties_axes_smallest(ops, shape, axis, k):
    rng = np.random.default_rng(31)
    for largest in (True, False):
        x = (rng.integers(-6, 7, size=shape).astype(np.float32) / np.float32(4))
        x.ravel()[rng.integers(0, x.size, 3)] = -0.0
        assert_topk_exact(ops, x, k, axis, largest)
        xr = rng.standard_normal(shape).astype(np.float32)
        assert_topk_exact(ops, xr, k, axis, largest)
        assert_topk_exact(ops, xr.astype(np.float16), k, axis, largest)


def test_topk_nan_inf(ops):
    x = np.random.default_rng(2).standard_normal((4, 500)).astype(np.float32)
    x[0, [3, 77]] = np.nan
    x[1, 5] = np.inf
    x[1, 6] = -np.inf
    x[2, :] = np.nan
    x[3, 10] = -np.nan
    for largest in (True, False):
        v, ix = ops.topk(dev(x), 9, -1, largest)
        ev, eix = oracle.topk(x, 9, -1, largest)
        assert np.array_equal(host(ix), eix)
        assert np.array_equal(np.isnan(host(v)), np.isnan(ev))


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("n,k", [(1000, 5), (256, 8), (1024, 32), (777, 20), (64, 16), (33, 33), (2048, 1)])
def test_topk_smallest_on_short_rows(ops, n, k, dtype):
    """The k smallest of rows that a wave holds (the one-wave kernel with its order keys turned
    round): spread-out rows, ties, constant rows, -0 and +0, rows of mostly +inf (the floor of
    that direction), -inf entries (its summit), NaN entries -- still the largest values, so they
    come last, also where the k smallest reach into them -- and sorted rows; against the oracle,
    in both directions."""
    rng = np.random.default_rng(n * 7 + k)
    rows = 12
    x = (rng.standard_normal((rows, n)) * 3).astype(np.float32)
    x[1] = np.round(x[1])                          # ties
    x[2] = 1.5                                     # constant
    x[3, ::2] = -0.0
    x[3, 1::2] = 0.0
    x[4, :] = np.inf
    x[4, rng.integers(0, n, max(1, k // 2))] = rng.standard_normal(max(1, k // 2))   # fewer numbers than k
    x[5, rng.integers(0, n, 5)] = -np.inf
    x[6, rng.integers(0, n, 7)] = np.nan
    x[7, :] = np.nan
    x[7, rng.integers(0, n, max(1, k - 2))] = rng.standard_normal(max(1, k - 2))     # the k smallest reach into the NaNs
    x[8] = np.sort(x[8])
    x[9] = np.sort(x[9])[::-1]
    x[10, :] = np.inf
    x[10, 3 % n] = np.nan                          # +inf, then the NaN
    x = x.astype(dtype)
    for largest in (False, True):
        v, ix = ops.topk(dev(x), k, -1, largest)
        ev, eix = oracle.topk(x.astype(np.float32), k, -1, largest)
        v, ix = host(v).astype(np.float32), host(ix)
        assert np.array_equal(ix, eix), (n, k, largest, np.argwhere(ix != eix)[:4])
        assert np.array_equal(np.isnan(v), np.isnan(ev))
        ok = ~np.isnan(ev)
        assert np.array_equal(v[ok].view(np.uint32), ev[ok].astype(np.float32).view(np.uint32))   # (bit copies: signs of zeros too)


def test_topk_workloads(ops, golden):
    x4 = synth.grid_values(8, 262144, synth.SEEDS["C4"])
    v, ix = assert_topk_exact(ops, x4, 1024)
    check_topk_invariants(x4, v, ix, 1024)
    x3 = synth.llm_logits(64, 128256, synth.SEEDS["C3"])
    assert_topk_exact(ops, x3, 50)
    x2 = synth.classifier_logits(256, 1000, synth.SEEDS["C2"])
    assert_topk_exact(ops, x2, 5)
    assert_topk_exact(ops, x2.astype(np.float16), 5)
    # libtorch values on the down-sized grid workload
    v, _ = assert_topk_exact(ops, golden["c4_in"], int(golden["c4_k"]))
    assert np.array_equal(v.view(np.uint32), golden["c4_val"].view(np.uint32))


@pytest.mark.parametrize("rows,n,k,largest,dtype", [
    (3, 20000, 300, True, np.float32), (3, 20000, 300, False, np.float32), (2, 16385, 2048, True, np.float32),
    (5, 40001, 256, True, np.float32), (2, 65536, 1000, True, np.float16), (3, 30003, 257, False, np.float16),
    (1, 262144, 1, False, np.float32)])
def test_topk_long_rows_large_k(ops, rows, n, k, largest, dtype):
    """Rows the multi-workgroup radix select takes: k above 255 or smallest-first,
    odd lengths (unaligned rows), half precision with its many equal values."""
    rng = np.random.default_rng(n + k)
    x = rng.standard_normal((rows, n)).astype(np.float32)
    x[0, ::7] = x[0, 3]            # a run of equal values across chunks
    x[-1, n // 2:] = np.round(x[-1, n // 2:] * 4) / 4   # a coarse grid: ties at the cut
    x = x.astype(dtype)
    v, ix = assert_topk_exact(ops, x, k, -1, largest)
    check_topk_invariants(x, v, ix, k, largest=largest)


def test_topk_long_rows_nan_inf(ops):
    x = np.random.default_rng(5).standard_normal((2, 50000)).astype(np.float32)
    x[0, [7, 40000]] = np.nan
    x[0, 123] = np.inf
    x[1, 10:20000] = -np.inf
    x[1, 49999] = -0.0
    assert_topk_exact(ops, x, 400)
    assert_topk_exact(ops, x, 400, -1, False)


# -------------------------------------------------------------------- fused --

def assert_fused(ops, x, k, axis=-1, largest=True, rows_may_differ=0):
    """rows_may_differ: how many rows of step (3) may come out in another order than the tensor
    route's -- by a probability tie that the two routes' row sums, an ulp apart, open or close; the
    ceiling a test passes is what its seeded inputs measure (0 on every case so far), so that a
    change that moves it shows."""
    v, ix, p = ops.softmax_topk(dev(x), k, axis, largest, return_probs=True)
    v, ix, p = host(v), host(ix), host(p)
    # (1) exactly the top-k of the softmax tensor the same call wrote
    ev, eix = oracle.topk(p, k, axis, largest)
    bits = np.uint16 if x.dtype == np.float16 else np.uint32
    assert np.array_equal(ix, eix), (x.shape, k)
    assert np.array_equal(v.view(bits), ev.view(bits))
    # (2) that tensor is the softmax, to the softmax bar
    assert_softmax_close(p, x, axis)
    # (3) without the tensor (the single-pass streaming kernel where it applies):
    # same ranking; its row sum is built from chunk partials, so a value may
    # round the other way
    v2, ix2 = ops.softmax_topk(dev(x), k, axis, largest)
    v2, ix2 = host(v2), host(ix2)
    same = np.array_equal(ix2, ix)
    if x.dtype == np.float16:
        assert half_ulp_diff(v2, v).max() <= 1
    else:
        assert ulp_diff(v2, v).max() <= 1
    pm = np.moveaxis(p, axis, -1).reshape(-1, x.shape[axis])
    i2 = np.moveaxis(ix2, axis, -1).reshape(-1, k)
    i1 = np.moveaxis(ix, axis, -1).reshape(-1, k)
    if not same:
        # only a probability tie that the 1-ulp difference opens or closes may
        # reorder: the ranking must still be exact for the values it returned
        tolerant = 0
        for r in range(pm.shape[0]):
            if not np.array_equal(i2[r], i1[r]):
                tolerant += 1
                assert sorted(pm[r][i2[r]].tolist()) == sorted(pm[r][i1[r]].tolist()), r
        assert tolerant <= rows_may_differ, "%s k=%d: %d of %d rows differ from the tensor route by a tie the row sum opened or closed (ceiling %d)" % (
            x.shape, k, tolerant, pm.shape[0], rows_may_differ)
    if largest:
        # whichever way such a tie went, the result is ranked by (probability, then lower
        # index) of a monotone function of the logits: checked on the logits themselves
        xm = np.moveaxis(x, axis, -1).reshape(-1, x.shape[axis]).astype(np.float32)
        v2m = np.moveaxis(v2, axis, -1).reshape(-1, k).astype(np.float32)
        for r in range(pm.shape[0]):
            if np.isfinite(v2m[r]).all():
                check_fused_invariants(xm[r], v2m[r], i2[r])
    # (4) against the oracle's own fused result: values to the softmax bar,
    # indices wherever the oracle's probabilities around the cut are distinct
    ov, oix, op = oracle.softmax_topk(x, k, axis, largest, return_probs=True)
    if x.dtype == np.float32:
        assert ulp_diff(v, ov).max() <= 2
        pm = np.moveaxis(op, axis, -1).reshape(-1, x.shape[axis])
        im, om = np.moveaxis(ix, axis, -1).reshape(-1, k), np.moveaxis(oix, axis, -1).reshape(-1, k)
        xm = np.moveaxis(x, axis, -1).reshape(-1, x.shape[axis])
        for r in range(pm.shape[0]):
            top = np.sort(xm[r])[::-1][:k + 1] if largest else np.sort(xm[r])[:k + 1]
            ptop = np.sort(pm[r])[::-1][:k + 1] if largest else np.sort(pm[r])[:k + 1]
            if len(np.unique(top)) == len(top) and len(np.unique(ptop)) == len(ptop) and not np.isnan(ptop).any():
                assert np.array_equal(im[r], om[r]), r
            # the streaming result: exactly the oracle's indices wherever the oracle's
            # probabilities around the cut are well apart (or tie through equal logits)
            if largest and well_separated_cut(pm[r], xm[r], k):
                assert np.array_equal(i2[r], om[r]), r
    return v, ix


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c2h"])
def test_fused_downsized_workloads(ops, golden, name):
    x, k = golden[name + "_in"], int(golden[name + "_k"])
    if name == "c2h":
        x = x.view(np.float16)
    v, ix = assert_fused(ops, x, k)
    ev, eix = golden[name + "_val"], golden[name + "_idx"]
    if name == "c2h":
        assert reference_half_tolerance_ok(v, ev)
    else:
        assert reference_float_tolerance_ok(v, ev)
        for r in range(x.shape[0]):
            if len(np.unique(ev[r])) == k:
                assert np.array_equal(ix[r], eix[r])


@pytest.mark.parametrize("shape,axis,k", [((7, 33), -1, 5), ((3, 50, 11), 1, 7), ((2, 3, 64, 4), 2, 64), ((1, 5), -1, 5),
                                          ((2, 20000), -1, 300), ((4, 1), -1, 1), ((9, 777), -1, 1)])
def test_fused_shapes_and_ties(ops, shape, axis, k):
    rng = np.random.default_rng(41)
    for largest in (True, False):
        assert_fused(ops, rng.standard_normal(shape).astype(np.float32) * 2, k, axis, largest)
        # grid data: many equal logits, hence many equal probabilities
        assert_fused(ops, rng.integers(-8, 9, size=shape).astype(np.float32) / np.float32(2), k, axis, largest)
        assert_fused(ops, (rng.standard_normal(shape) * 2).astype(np.float16), k, axis, largest)


def test_fused_probability_collisions(ops):
    """Distinct logits whose probabilities round to the same float: the
    reference order (top-k of the softmax tensor) puts the lower index first
    even when its logit is the smaller one."""
    n = 4096
    x = np.full((2, n), -20.0, np.float32)
    x[:, 100] = 12.0                                # max; ulp(x - 12) = 2^-20 near 0 logits
    base = np.float32(1.0)
    x[0, 900] = base                                # larger logit, higher index
    x[0, 50] = np.nextafter(base, np.float32(0))    # smaller logit, lower index
    x[1, 2000:2100] = np.float32(0.25) + np.arange(100, dtype=np.float32) * np.float32(2.0 ** -24)
    assert_fused(ops, x, 3)
    assert_fused(ops, x, 60)
    # underflow: most probabilities are exactly zero and tie by index
    y = np.random.default_rng(3).standard_normal((2, 3000)).astype(np.float32)
    y[:, 17] = 200.0
    assert_fused(ops, y, 10)
    assert_fused(ops, y.astype(np.float16) , 10)


@pytest.mark.parametrize("rows,n,k,dtype", [(2, 20000, 300, np.float32), (3, 70001, 1024, np.float32),
                                             (2, 32768, 500, np.float16)])
def test_fused_long_rows_large_k(ops, rows, n, k, dtype):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal((rows, n)) * 2).astype(np.float32)
    x[0, 100:9000] = np.round(x[0, 100:9000])   # equal logits -> equal probabilities
    assert_fused(ops, x.astype(dtype), k)


def test_fused_nan_rows(ops):
    x = np.random.default_rng(4).standard_normal((3, 900)).astype(np.float32)
    x[0, 400] = np.nan
    x[1, 2] = np.inf
    v, ix = ops.softmax_topk(dev(x), 6)
    v, ix = host(v), host(ix)
    assert np.isnan(v[0]).all() and np.isnan(v[1]).all()
    assert ix[0].tolist() == list(range(6)) and ix[1].tolist() == list(range(6))
    ov, oix = oracle.softmax_topk(x, 6)
    assert np.array_equal(ix, oix) and ulp_diff(v, ov).max() <= 2


def test_fused_headline_workload(ops):
    """[64,128256] float32, k=50: every row against the oracle."""
    x = synth.llm_logits(64, 128256, synth.SEEDS["C3"])
    v, ix = ops.softmax_topk(dev(x), 50)
    v, ix = host(v), host(ix)
    ov, oix = oracle.softmax_topk(x, 50)
    assert np.array_equal(ix, oix)
    assert ulp_diff(v, ov).max() <= 2
    # run to run: bit-identical
    v2, ix2 = ops.softmax_topk(dev(x), 50)
    assert np.array_equal(host(ix2), ix) and np.array_equal(host(v2).view(np.uint32), v.view(np.uint32))


def test_detection_style_chain(ops, golden):
    """softmax over the class axis -> per-anchor class max -> top-k anchors."""
    for x, k in ((golden["c5_in"], int(golden["c5_k"])), (synth.detection_scores(16, 80, 8400, synth.SEEDS["C5"]), 300)):
        p = ops.softmax(dev(x), 1)
        m = ops.reduce_max(p, 1)
        v, ix = ops.topk(m, k)
        p, m, v, ix = host(p), host(m), host(v), host(ix)
        assert np.array_equal(m.view(np.uint32), p.max(axis=1).view(np.uint32))
        ev, eix = oracle.topk(m, k)
        assert np.array_equal(ix, eix) and np.array_equal(v.view(np.uint32), ev.view(np.uint32))
        assert ulp_diff(m, oracle.reduce_max(oracle.softmax(x, 1), 1)).max() <= 2
    assert reference_float_tolerance_ok(host(ops.reduce_max(ops.softmax(dev(golden["c5_in"]), 1), 1)), golden["c5_max"])


@pytest.mark.parametrize("shape,axis,dtype", [((16, 80, 8400), 1, np.float32), ((3, 80, 1000), 1, np.float16),
                                              ((5, 7, 9), 0, np.float32), ((4, 300), 1, np.float32),
                                              ((2, 200, 33), 1, np.float32), ((6, 5000), -1, np.float32),
                                              ((2, 1000, 64), 1, np.float32), ((1, 4100, 130), 1, np.float16),
                                              ((300, 200, 64), 1, np.float32)])
def test_softmax_then_max_in_one_pass(ops, shape, axis, dtype):
    """The per-line maximum of the softmax equals, bit for bit, the max operator
    applied to the softmax operator's output; NaN and -inf lines included."""
    x = (np.random.default_rng(sum(shape)).standard_normal(shape) * 2 - 3).astype(np.float32)
    xm = np.moveaxis(x, axis, -1)
    xm[..., :] = xm  # (view)
    flat = xm.reshape(-1, xm.shape[-1])
    flat[0, 1] = np.nan
    flat[1, :] = -np.inf
    flat[2, 0] = np.inf
    x = x.astype(dtype)
    fused = host(ops.softmax_reduce_max(dev(x), axis))
    chain = host(ops.reduce_max(ops.softmax(dev(x), axis), axis))
    bits = np.uint16 if dtype == np.float16 else np.uint32
    assert fused.shape == chain.shape
    assert np.array_equal(np.isnan(fused), np.isnan(chain))
    ok = ~np.isnan(chain)
    assert np.array_equal(fused.view(bits)[ok], chain.view(bits)[ok])
    if dtype == np.float32:
        want = oracle.reduce_max(oracle.softmax(x, axis), axis)
        assert ulp_diff(fused[ok], want[ok]).max() <= 2


def test_workspace_too_small_is_an_error(ops):
    from vkop_amd import capi
    x = dev(synth.classifier_logits(4, 1000, 1))
    v = torch.empty((4, 5), device="cuda")
    ix = torch.empty((4, 5), dtype=torch.int32, device="cuda")
    with pytest.raises(capi.VkopHipError) as e:
        capi.softmax_topk(x.data_ptr(), 0, v.data_ptr(), ix.data_ptr(), capi.F32, (4, 1000), -1, 5, 1, 0, 0, 0)
    assert e.value.code == capi.ERR_WORKSPACE


# ------------------------------------------- recordings, streams, variants --

def _aligned_workspace(capi, nbytes, stream):
    buf = torch.empty(nbytes + 256, dtype=torch.uint8, device="cuda")
    ptr = buf.data_ptr() + (-buf.data_ptr()) % 256
    capi.workspace_init(ptr, nbytes // 4 * 4, stream)
    capi.stream_sync(stream)
    return buf, ptr


def test_recording_replayed_with_new_inputs(ops):
    """A recorded fused call is replayed several times; between replays the input
    buffer is rewritten by ordinary eager work.  Every replay must equal the
    eager result for the data then in the buffer."""
    from vkop_amd import capi
    rows, n, k = 16, 128256, 50
    shape = (rows, n)
    stream = capi.stream_create()
    x = torch.empty(shape, dtype=torch.float32, device="cuda")
    vals = torch.empty((rows, k), dtype=torch.float32, device="cuda")
    idx = torch.empty((rows, k), dtype=torch.int32, device="cuda")
    nb = capi.softmax_topk_workspace_bytes(capi.F32, shape, -1, k)
    ws, ptr = _aligned_workspace(capi, nb, stream)
    x.copy_(dev(synth.llm_logits(rows, n, 100)))
    torch.cuda.synchronize()
    capi.graph_begin(stream)
    capi.softmax_topk(x.data_ptr(), 0, vals.data_ptr(), idx.data_ptr(), capi.F32, shape, -1, k, 1, ptr, nb, stream)
    graph = capi.graph_end(stream)
    try:
        for rep in range(4):
            h = synth.llm_logits(rows, n, 100 + rep)
            x.copy_(dev(h))          # eager work between replays
            torch.cuda.synchronize()
            capi.graph_launch(graph, stream)
            capi.stream_sync(stream)
            ev, eix = ops.softmax_topk(x, k)   # eager call, its own workspace
            torch.cuda.synchronize()
            assert np.array_equal(host(idx), host(eix)), rep
            assert np.array_equal(host(vals).view(np.uint32), host(ev).view(np.uint32)), rep
            ov, oix = oracle.softmax_topk(h, k)
            assert np.array_equal(host(idx), oix) and ulp_diff(host(vals), ov).max() <= 2
    finally:
        capi.graph_destroy(graph)
        capi.stream_destroy(stream)


def test_calls_in_flight_on_separate_streams():
    """Four independent calls, each on its own stream with its own workspace and
    outputs, submitted without waiting in between (what bench.py times)."""
    from vkop_amd import capi
    rows, n, k = 64, 128256, 50
    shape = (rows, n)
    lanes = []
    for j in range(4):
        s = capi.stream_create()
        h = synth.llm_logits(rows, n, 200 + j)
        nb = capi.softmax_topk_workspace_bytes(capi.F32, shape, -1, k)
        ws, ptr = _aligned_workspace(capi, nb, s)
        lanes.append(dict(s=s, h=h, x=dev(h), ws=ws, ptr=ptr, nb=nb,
                          v=torch.empty((rows, k), dtype=torch.float32, device="cuda"),
                          i=torch.empty((rows, k), dtype=torch.int32, device="cuda")))
    torch.cuda.synchronize()
    for rep in range(3):
        for ln in lanes:
            capi.softmax_topk(ln["x"].data_ptr(), 0, ln["v"].data_ptr(), ln["i"].data_ptr(), capi.F32, shape, -1, k, 1,
                              ln["ptr"], ln["nb"], ln["s"])
    for ln in lanes:
        capi.stream_sync(ln["s"])
    for ln in lanes:
        ov, oix = oracle.softmax_topk(ln["h"], k)
        assert np.array_equal(host(ln["i"]), oix)
        assert ulp_diff(host(ln["v"]), ov).max() <= 2
        capi.stream_destroy(ln["s"])


@pytest.mark.parametrize("shape_knobs", [(1024, 4, 8), (512, 8, 8), (256, 4, 32)])
def test_streaming_variants_agree(ops, shape_knobs):
    """The one-kernel variant (arrival counters) and other launch shapes give the
    bits the default gives; the same workspace serves them in turn."""
    from vkop_amd import capi
    x = synth.llm_logits(64, 128256, synth.SEEDS["C3"])
    xd = dev(x)
    v0, i0 = ops.softmax_topk(xd, 50)
    t0, j0 = ops.topk(xd, 50)
    v0, i0, t0, j0 = host(v0), host(i0), host(t0), host(j0)
    try:
        for fused in (1, 0):
            capi.tune("rows.fused", fused)
            for knobs in (None, shape_knobs):
                for name, val in zip(("rows.threads", "rows.loads", "rows.chunks"), knobs or (0, 0, 0)):
                    capi.tune(name, val)
                for rep in range(2):
                    v, i = ops.softmax_topk(xd, 50)
                    assert np.array_equal(host(i), i0), (fused, knobs, rep)
                    assert ulp_diff(host(v), v0).max() <= 1   # another chunking sums in another order
                    t, j = ops.topk(xd, 50)
                    assert np.array_equal(host(j), j0) and np.array_equal(host(t).view(np.uint32), t0.view(np.uint32))
    finally:
        capi.tune("rows.fused", 0)
        for name in ("rows.threads", "rows.loads", "rows.chunks"):
            capi.tune(name, 0)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_fused_quantised_logits_tie_at_the_cut(ops, dtype):
    """Logits that went through bfloat16 (8 mantissa bits) repeat a lot: equal
    logits, hence equal probabilities, straddle the k-th place in most rows."""
    rng = np.random.default_rng(77)
    x = (rng.standard_normal((32, 128256)) * 1.25).astype(np.float32)
    x = (x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)   # truncate to bfloat16 precision
    x = np.ascontiguousarray(x.astype(dtype))
    k = 50
    sx = np.sort(x.astype(np.float32), axis=-1)[:, ::-1]
    assert (sx[:, k - 1] == sx[:, k]).mean() > 0.3      # the case is really there
    assert_fused(ops, x, k)
    # and a short-row shape, where one workgroup owns the row
    assert_fused(ops, np.ascontiguousarray(x[:, :1000]), 5)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_fused_ordered_and_clustered_rows(ops, dtype):
    """Rows whose large values sit side by side (sorted rows, one hot region):
    the lanes that hold them are few, so a bound taken from lane maxima lets far
    too many elements through and the chunk has to find its exact threshold."""
    rng = np.random.default_rng(123)
    n, k = 128256, 50
    base = (rng.standard_normal((6, n)) * 2).astype(np.float32)
    x = base.copy()
    x[0] = np.sort(base[0])                 # ascending: the top sits in the last chunk
    x[1] = np.sort(base[1])[::-1]           # descending
    x[2, 40000:43000] += 9.0                # a hot region inside one chunk
    x[3, 8000:8200] += 12.0                 # a narrow one: more than k, fewer than a list holds
    x[4] = np.sort(base[4])
    x[4, ::2] = x[4, ::2][::-1]             # interleaved ascending / descending
    x[5, 100000:100064] = 30.0              # equal values at the top, more than k of them
    x = np.ascontiguousarray(x.astype(dtype))
    assert_fused(ops, x, k)
    for largest in (True, False):
        v, ix = ops.topk(dev(x), k, -1, largest)
        ev, eix = oracle.topk(x, k, -1, largest)
        bits = np.uint16 if dtype == np.float16 else np.uint32
        assert np.array_equal(host(ix), eix) and np.array_equal(host(v).view(bits), ev.view(bits))
    # ragged chunks (row length not a multiple of the vector width) take the other code path
    y = np.ascontiguousarray(np.sort(base[:2, :70001], axis=-1).astype(dtype))
    assert_fused(ops, y, 64)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_masked_and_underflowed_rows(ops, dtype):
    """Rows where the k-th place falls among probabilities that are exactly 0
    (masked logits at -inf, a tail that underflows) or among -inf elements: the
    places behind the positive probabilities go to the lowest indices."""
    rng = np.random.default_rng(321)
    n, k = 128256, 50
    x = (rng.standard_normal((8, n)) * 2).astype(np.float32)
    allowed = rng.choice(n, 20, replace=False)
    x[0] = -np.inf
    x[0, allowed] = rng.standard_normal(20).astype(np.float32)       # 20 allowed tokens, k = 50
    x[1] = -np.inf
    x[1, 77777] = 1.5                                                # a single allowed token
    x[2, 5000] = 150.0 if dtype == np.float32 else 60.0              # everything else underflows (or nearly)
    x[3, :] = -np.inf
    x[3, 100:100 + k] = 0.25                                         # exactly k finite elements, all equal
    x[4, ::3] = -np.inf                                              # a third masked: plenty left
    x[5] = -np.inf                                                   # nothing left: NaN row
    x[6, 1000] = np.inf                                              # NaN row
    x[7, 64000:64100] = 120.0 if dtype == np.float32 else 50.0      # a plateau far above a tail that underflows
    x = np.ascontiguousarray(x.astype(dtype))
    v, ix = ops.softmax_topk(dev(x), k)
    v, ix = host(v), host(ix)
    ov, oix = oracle.softmax_topk(x, k)
    assert np.array_equal(ix, oix)
    if dtype == np.float16:
        assert half_ulp_diff(v, ov).max() <= 1
    else:
        assert ulp_diff(v, ov).max() <= 2
    # the same through the softmax tensor route
    assert_fused(ops, x[[0, 1, 2, 3, 4, 7]], k)
    # plain top-k: -inf elements tie by index behind the finite ones
    for largest in (True, False):
        y = x if largest else -x
        y = np.ascontiguousarray(y[[0, 1, 3, 4, 5]])
        t, j = ops.topk(dev(y), k, -1, largest)
        et, ej = oracle.topk(y, k, -1, largest)
        bits = np.uint16 if dtype == np.float16 else np.uint32
        assert np.array_equal(host(j), ej) and np.array_equal(host(t).view(bits), et.view(bits))
    # short rows, one workgroup per row
    short = np.ascontiguousarray(x[:5, :1000])
    short[0, allowed[:3] % 1000] = np.array([0.5, -1.0, 2.0], dtype)   # 3 allowed tokens, k = 5
    short[1, 777] = 1.5
    short[2, 500] = 150.0 if dtype == np.float32 else 60.0
    assert_fused(ops, short, 5)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("levels", [17, 256, 3])
def test_heavily_quantised_rows(ops, dtype, levels):
    """Logits on a coarse grid: hundreds or thousands of elements equal the value
    at the k-th place, in every chunk of the row; the lowest indices win."""
    rng = np.random.default_rng(levels)
    n, k = 128256, 50
    if levels == 256:    # int8-like: a bell shape over 256 levels
        x = np.clip(np.round(rng.standard_normal((6, n)) * 40), -128, 127).astype(np.float32) * np.float32(0.125)
    else:
        x = rng.integers(0, levels, size=(6, n)).astype(np.float32) * np.float32(0.5) - np.float32(2.0)
    x[1, :20000] = x[1].min()        # the first chunks of the row hold nothing of interest
    x[2] = np.sort(x[2])             # equal values side by side
    x = np.ascontiguousarray(x.astype(dtype))
    assert_fused(ops, x, k)
    assert_fused(ops, np.ascontiguousarray(x[:, :70001]), 200)
    for largest in (True, False):
        t, j = ops.topk(dev(x), k, -1, largest)
        et, ej = oracle.topk(x, k, -1, largest)
        bits = np.uint16 if dtype == np.float16 else np.uint32
        assert np.array_equal(host(j), ej) and np.array_equal(host(t).view(bits), et.view(bits))


def _awkward_rows(rng, rows, n):
    """Rows mixing the shapes that strain a streaming select: coarse grids, sorted
    runs, plateaus, masks, wide spreads, repeated blocks."""
    x = (rng.standard_normal((rows, n)) * rng.choice([0.3, 2.0, 8.0])).astype(np.float32)
    for r in range(rows):
        kind = rng.integers(0, 9)
        if kind == 0:
            x[r] = np.round(x[r] * rng.choice([0.5, 2.0, 16.0])) / np.float32(4.0)
        elif kind == 1:
            a, b = sorted(rng.integers(0, n, 2))
            x[r, a:b] = np.sort(x[r, a:b])[::rng.choice([-1, 1])]
        elif kind == 2:
            a = rng.integers(0, n - 1)
            x[r, a:a + rng.integers(1, 5000)] = np.float32(rng.choice([5.0, 30.0, 100.0]))
        elif kind == 3:
            x[r, rng.random(n) < rng.choice([0.5, 0.99, 0.9999])] = -np.inf
        elif kind == 4:
            x[r, rng.integers(0, n)] = np.float32(rng.choice([90.0, 200.0, 1e4]))
        elif kind == 5:
            x[r] = np.tile(x[r, :257], n // 257 + 1)[:n]
        elif kind == 6:
            x[r] = np.float32(rng.choice([0.0, -3.5, 1e-30]))
        elif kind == 7:
            x[r, :: int(rng.integers(1, 50))] = np.float32(7.25)
    return x


@pytest.mark.parametrize("n,k", [(128256, 50), (128256, 255), (40000, 1), (8200, 5), (65536, 64), (1000, 5)])
def test_awkward_rows_against_the_oracle(ops, n, k):
    rng = np.random.default_rng(n + k)
    for dtype in (np.float32, np.float16):
        x = np.ascontiguousarray(_awkward_rows(rng, 24, n).astype(dtype))
        v, ix = ops.softmax_topk(dev(x), k)
        v, ix = host(v), host(ix)
        p = host(ops.softmax(dev(x)))
        ev, eix = oracle.topk(p, k)                       # top-k of the softmax tensor the library writes
        ov, oix = oracle.softmax_topk(x, k)               # and the oracle's own
        rows_equal = (ix == eix).all(axis=1)
        if dtype == np.float16:
            assert half_ulp_diff(v, ov).max() <= 1
        else:
            assert ulp_diff(v, ov).max() <= 2
        # a row may differ from the tensor route only where a 1-ulp difference in the
        # row sum opens or closes a probability tie: the values must still agree
        for r in np.nonzero(~rows_equal)[0]:
            d = half_ulp_diff(v[r], ev[r]) if dtype == np.float16 else ulp_diff(v[r], ev[r])
            assert d.max() <= 1, (r, n, k)
            assert len(set(ix[r].tolist())) == k
        # (how many: 0 of 24 on every case here; the ceiling is that measurement, so that a change which moves it shows)
        assert int((~rows_equal).sum()) <= 0, "n=%d k=%d %s: %d of %d rows differ from the tensor route by a tie the row sum opened or closed" % (
            n, k, np.dtype(dtype).name, int((~rows_equal).sum()), len(rows_equal))
        # every row, tolerant branch or not: ranked by (probability, then lower index) of a
        # monotone function of the logits; and exactly the oracle's indices wherever its
        # probabilities around the cut are well apart (or tie through equal logits)
        op_full = oracle.softmax(x)
        xf = x.astype(np.float32)
        exact_rows = 0
        for r in range(x.shape[0]):
            vr = v[r].astype(np.float32)
            if np.isfinite(vr).all():
                check_fused_invariants(xf[r], vr, ix[r])
            if well_separated_cut(op_full[r].astype(np.float32), xf[r], k, 4 if dtype == np.float32 else 1 << 14):
                exact_rows += 1
                assert np.array_equal(ix[r], oix[r]), (r, n, k)
        print("   ... %d rows with a well separated cut match the oracle's indices exactly" % exact_rows)
        for largest in (True, False):
            t, j = ops.topk(dev(x), k, -1, largest)
            et, ej = oracle.topk(x, k, -1, largest)
            bits = np.uint16 if dtype == np.float16 else np.uint32
            assert np.array_equal(host(j), ej) and np.array_equal(host(t).view(bits), et.view(bits)), (n, k, largest)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("n,k", [(8400, 300), (8400, 255), (8400, 256), (8400, 408), (8400, 409), (32768, 400), (1200, 100),
                                 (300, 299)])
def test_large_k_on_rows_one_workgroup_holds(ops, dtype, n, k):
    """k beyond the merge kernel's 255 ranks (and large k in general) on rows short
    enough for one workgroup: [16,8400] k = 300 is the detection workload's select."""
    rng = np.random.default_rng(n * 7 + k)
    x = rng.random((16, n)).astype(np.float32)
    x[1] = np.round(x[1] * 50) / 50            # heavy ties
    x[2] = np.sort(x[2])
    x[3, : n // 2] = -np.inf
    x[4] = 0.5
    x = np.ascontiguousarray(x.astype(dtype))
    bits = np.uint16 if dtype == np.float16 else np.uint32
    for largest in (True, False):
        t, j = ops.topk(dev(x), k, -1, largest)
        et, ej = oracle.topk(x, k, -1, largest)
        assert np.array_equal(host(j), ej) and np.array_equal(host(t).view(bits), et.view(bits)), (n, k, largest)
    assert_fused(ops, x * 8, k)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("rows,n,k", [(16, 8400, 300), (48, 8192, 100), (40, 4096, 64), (24, 8190, 100), (12, 20000, 120)])
@pytest.mark.parametrize("kind", ["runs", "levels", "ascending", "descending", "two_values"])
def test_rows_in_order_and_rows_of_levels_on_the_one_workgroup_route(ops, kind, rows, n, k, dtype):
    """Rows one workgroup holds whose first list of candidates overflows: values in order (the bound
    from the lane maxima is far too low; the vector minima give a second one, and the list is made
    straight from the registers) and values equal en masse (the cut is looked for among the next few
    distinct values before any radix pass).  Shapes with vectors no thread holds (8400 elements in a
    workgroup shaped for 32768), a row of an odd length, and one of 20000 elements."""
    x = np.ascontiguousarray(synth.awkward_rows(kind, rows, n, seed=n + k).astype(dtype))
    bits = np.uint16 if dtype == np.float16 else np.uint32
    t, j = ops.topk(dev(x), k)
    et, ej = oracle.topk(x, k)
    assert np.array_equal(host(j), ej) and np.array_equal(host(t).view(bits), et.view(bits)), (kind, rows, n, k)
    assert_fused(ops, x, k)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
def test_topk_without_an_order(ops, dtype):
    """sorted = 0 (the reference parses the attribute and ignores it, ops/Topk.hpp:73-75): the same k
    elements in an order of the library's choosing, the same on every call.  On the multi-pass radix
    select -- smallest first on long rows -- that is the order the select lists them in (its ranking
    step is left out); on the other routes the sorted result."""
    rng = np.random.default_rng(21)
    bits = np.uint16 if dtype == np.float16 else np.uint32
    cases = [((6, 100000), 300, False), ((3, 70000), 2048, False), ((5, 40000), 64, False), ((64, 9000), 7, True), ((8, 1000), 5, True),
             ((4, 60000), 100, True)]
    took_the_select = 0
    for shape, k, largest in cases:
        x = (np.round(rng.standard_normal(shape) * 64) / 64).astype(np.float32)     # ties at the cut in most rows
        x[0, :5] = np.nan
        x = np.ascontiguousarray(x.astype(dtype))
        et, ej = oracle.topk(x, k, -1, largest)
        t, j = ops.topk(dev(x), k, -1, largest, sorted=False)
        t, j = host(t), host(j)
        t2, j2 = ops.topk(dev(x), k, -1, largest, sorted=False)
        assert np.array_equal(j, host(j2)) and np.array_equal(t.view(bits), host(t2).view(bits)), (shape, k, largest)
        for r in range(shape[0]):
            order = np.argsort(j[r], kind="stable")
            want = np.argsort(ej[r], kind="stable")
            assert np.array_equal(j[r][order], ej[r][want]), (shape, k, largest, r)          # the same elements (ties: lowest indices)
            assert np.array_equal(t[r][order].view(bits), et[r][want].view(bits)), (shape, k, largest, r)
        if not np.array_equal(j, ej):
            took_the_select += 1
            assert not largest, (shape, k)          # (largest first, these shapes take routes whose result is in order anyway)
    assert took_the_select >= 2        # (the long smallest-first rows: their unordered result differs from the ordered one)


# ---- non-maximum suppression ------------------------------------------------------------------------

def _nms_boxes(rng, B, N, spread=1.3):
    c = rng.random((B, N, 2)).astype(np.float32)
    s = (rng.random((B, N, 2)) * spread).astype(np.float32)
    return np.concatenate([np.clip(c - s / 2, 0, 1), np.clip(c + s / 2, 0, 1)], axis=-1).astype(np.float32)


@pytest.mark.parametrize("B,C,N,max_per_class,iou_thr,score_thr", [
    (1, 2, 10, 0, 0.5, 0.5), (1, 1, 200, 50, 0.7, 0.4), (1, 7, 50, 0, 0.3, 0.2),      # tests/NmsTest.cpp:165-169
    (3, 5, 300, 0, 0.45, 0.25), (2, 3, 3000, 100, 0.5, 0.3), (16, 4, 8400, 0, 0.6, 0.9), (1, 1, 1, 0, 0.5, 0.1),
    (2, 2, 1500, 0, 0.5, -1.0),
    (1, 2, 30000, 0, 0.5, 0.95), (1, 1, 40000, 50, 0.5, 0.9), (2, 1, 12289, 0, 0.4, 0.9)])   # several rounds of the scan
def test_nms_matches_the_oracle(ops, B, C, N, max_per_class, iou_thr, score_thr):
    rng = np.random.default_rng(B * 1000 + N)
    boxes = _nms_boxes(rng, B, N, 1.3 if N <= 300 else 0.2)
    scores = rng.random((B, C, N)).astype(np.float32)
    if N >= 300:
        scores[0, 0, 5:40] = scores[0, 0, 5]              # equal scores: lower box index first
    got, over = ops.nms(dev(boxes), dev(scores), iou_thr, score_thr, max_per_class)
    want = oracle.nms(boxes, scores, iou_thr, score_thr, max_per_class, max_candidates=2048)
    assert np.array_equal(host(got), want)
    assert over == bool(((scores > score_thr).sum(axis=-1) > 2048).any())
    # centre format, and half precision inputs (the same numbers after widening)
    centre = np.stack([(boxes[..., 0] + boxes[..., 2]) / 2, (boxes[..., 1] + boxes[..., 3]) / 2,
                       boxes[..., 2] - boxes[..., 0], boxes[..., 3] - boxes[..., 1]], -1).astype(np.float32)
    got_c, _ = ops.nms(dev(centre), dev(scores), iou_thr, score_thr, max_per_class, center_point_box=1)
    assert np.array_equal(host(got_c), oracle.nms(centre, scores, iou_thr, score_thr, max_per_class, 1, max_candidates=2048))
    bh, sh = boxes.astype(np.float16), scores.astype(np.float16)
    got_h, _ = ops.nms(dev(bh), dev(sh), iou_thr, score_thr, max_per_class)
    want_h = oracle.nms(bh.astype(np.float32), sh.astype(np.float32), iou_thr, score_thr, max_per_class, max_candidates=2048)
    assert np.array_equal(host(got_h), want_h)
    # a small output buffer keeps the first records; the count still says how many there are
    if len(want) > 3:
        few, _ = ops.nms(dev(boxes), dev(scores), iou_thr, score_thr, max_per_class, out_capacity=3)
        assert np.array_equal(host(few), want[:3])


@pytest.mark.parametrize("threads", [256, 1024])
def test_nms_either_workgroup_size(ops, threads):
    """The kernel has a 256-thread and a 1024-thread form, picked by the number of pairs: each on sparse, dense,
    multi-block and overflowing candidate sets."""
    from vkop_amd import capi
    capi.tune("nms.threads", threads)
    try:
        for B, C, N, per_class, iou_thr, score_thr in [(1, 3, 50, 0, 0.3, 0.2), (2, 3, 3000, 100, 0.5, 0.3), (1, 2, 2048, 0, 0.6, -1.0),
                                                       (1, 1, 600, 0, 0.5, 0.1), (1, 2, 30000, 0, 0.5, 0.95), (3, 2, 700, 7, 0.4, 0.5)]:
            rng = np.random.default_rng(N + threads)
            boxes = _nms_boxes(rng, B, N, 1.3 if N <= 300 else 0.2)
            scores = rng.random((B, C, N)).astype(np.float32)
            got, over = ops.nms(dev(boxes), dev(scores), iou_thr, score_thr, per_class)
            want = oracle.nms(boxes, scores, iou_thr, score_thr, per_class, max_candidates=2048)
            assert np.array_equal(host(got), want), (threads, B, C, N)
            assert over == bool(((scores > score_thr).sum(axis=-1) > 2048).any())
    finally:
        capi.tune("nms.threads", 0)


def test_nms_pairs_without_candidates_and_tiny_rows(ops):
    rng = np.random.default_rng(4)
    for B, C, N in [(2, 3, 4), (1, 5, 3), (2, 2, 64), (1, 1, 2), (3, 1, 8)]:
        boxes = _nms_boxes(rng, B, N)
        scores = rng.random((B, C, N)).astype(np.float32)
        got, over = ops.nms(dev(boxes), dev(scores), 0.5, 2.0)                  # nothing passes the score threshold
        assert host(got).shape == (0, 3) and not over
        scores[:, 0] = -1.0                                                     # class 0 has no candidate, the others do
        got, _ = ops.nms(dev(boxes), dev(scores), 0.5, 0.0)
        want = oracle.nms(boxes, scores, 0.5, 0.0, 0, max_candidates=2048)
        assert np.array_equal(host(got), want) and not (want[:, 1] == 0).any()
        for dt in (np.float16,):
            got16, _ = ops.nms(dev(boxes.astype(dt)), dev(scores.astype(dt)), 0.5, 0.0)
            want16 = oracle.nms(boxes.astype(dt).astype(np.float32), scores.astype(dt).astype(np.float32), 0.5, 0.0, 0,
                                max_candidates=2048)
            assert np.array_equal(host(got16), want16)


def test_nms_random_configurations(ops):
    """Seeded sweep over sizes around the kernel's tile, block and capacity boundaries, quantised scores and boxes
    (ties, identical and empty boxes), thresholds including negative ones, limits, both box formats and types."""
    from vkop_amd import capi
    rng = np.random.default_rng(2026)
    try:
        for it in range(80):
            B, C = int(rng.integers(1, 4)), int(rng.integers(1, 6))
            N = int(rng.choice([1, 3, 4, 63, 64, 65, 255, 256, 257, 512, 513, 1000, 2047, 2048, 2049, 4096, 9216, 9217, 12289]))
            ctr = rng.random((B, N, 2)).astype(np.float32)
            size = (rng.random((B, N, 2)) * float(rng.choice([0.05, 0.2, 0.6, 1.3]))).astype(np.float32)
            boxes = np.concatenate([ctr - size / 2, ctr + size / 2], -1).astype(np.float32)
            scores = rng.random((B, C, N)).astype(np.float32)
            mode = int(rng.integers(0, 4))
            if mode == 1:
                scores = np.round(scores * 8) / 8
            elif mode == 2:
                boxes = np.round(boxes * 4) / 4
            elif mode == 3:
                scores[..., ::3] = scores[..., :1]
            thr, iou = float(rng.choice([-1.0, 0.0, 0.1, 0.5, 0.9, 0.99])), float(rng.choice([-0.5, 0.0, 0.1, 0.45, 0.7, 1.0]))
            per, centre = int(rng.choice([0, 0, 1, 7, 100, 3000])), int(rng.integers(0, 2))
            capi.tune("nms.threads", int(rng.choice([0, 256, 1024])))
            if centre:
                boxes = np.stack([(boxes[..., 0] + boxes[..., 2]) / 2, (boxes[..., 1] + boxes[..., 3]) / 2,
                                  boxes[..., 2] - boxes[..., 0], boxes[..., 3] - boxes[..., 1]], -1).astype(np.float32)
            if rng.integers(0, 2):
                boxes, scores = boxes.astype(np.float16), scores.astype(np.float16)
            got, over = ops.nms(dev(boxes), dev(scores), iou, thr, per, centre)
            b32, s32 = boxes.astype(np.float32), scores.astype(np.float32)
            want = oracle.nms(b32, s32, iou, thr, per, centre, max_candidates=2048)
            assert np.array_equal(host(got), want), (it, B, C, N, mode, thr, iou, per, centre, boxes.dtype)
            assert over == bool(((s32 > thr).sum(-1) > 2048).any()), it
    finally:
        capi.tune("nms.threads", 0)


def test_nms_detection_workload_full_size(ops):
    """The detection-shaped case of the operator benchmark, and a dense one with a per-class limit, against the oracle."""
    c5 = synth.detection_scores(16, 80, 8400, synth.SEEDS["C5"])
    e = np.exp(c5 - c5.max(axis=1, keepdims=True))
    scores = np.ascontiguousarray((e / e.sum(axis=1, keepdims=True)).astype(np.float32))
    rng = np.random.default_rng(synth.SEEDS["C5"] + 1)
    boxes = _nms_boxes(rng, 16, 8400, 0.2)
    got, over = ops.nms(dev(boxes), dev(scores), 0.45, 0.25, 100)
    want = oracle.nms(boxes, scores, 0.45, 0.25, 100, max_candidates=2048)
    assert not over and len(want) > 10000 and np.array_equal(host(got), want)
    # keeping is idempotent: the kept boxes of a pair suppress nothing among themselves
    first = want[(want[:, 0] == 3) & (want[:, 1] == 7)][:, 2]
    again, _ = ops.nms(dev(boxes[3:4, first]), dev(scores[3:4, 7:8, first]), 0.45, 0.25, 100)
    assert len(host(again)) == len(first)
    dense_scores = rng.random((4, 20, 2048)).astype(np.float32)
    got, over = ops.nms(dev(boxes[:4, :2048]), dev(dense_scores), 0.5, 0.0, 200)
    want = oracle.nms(boxes[:4, :2048], dense_scores, 0.5, 0.0, 200, max_candidates=2048)
    assert not over and np.array_equal(host(got), want) and len(want) == 4 * 20 * 200


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_topp_count_on_fused_output(ops, dtype):
    x = np.ascontiguousarray(synth.llm_logits(64, 128256, synth.SEEDS["C3"])[:, :32000].astype(dtype))
    for k in (1, 50, 200, 255):
        v, _ = ops.softmax_topk(dev(x), k)
        for p in (0.0, 0.3, 0.9, 0.999, 2.0):
            assert np.array_equal(host(ops.topp_count(v, p)), oracle.topp_count(host(v), p)), (k, p)
    wide = np.sort(np.random.default_rng(1).random((3, 5, 2048)).astype(dtype) / 1024, axis=-1)[..., ::-1].copy()
    got = host(ops.topp_count(dev(wide), 0.75))
    assert got.shape == (3, 5) and np.array_equal(got, oracle.topp_count(wide, 0.75))


# ---- models from .vkopbin files ---------------------------------------------------------------------

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_model_files_drive_the_operators(ops, dtype):
    from vkop_amd import runtime, vkopbin
    # classifier head, fused and not: the same ranking; values to the fused operator's bar
    head = vkopbin.read_model(os.path.join(GOLDEN_DIR, "classifier_head.vkopbin"))
    x = np.ascontiguousarray(synth.classifier_logits(8, 1000, 77).astype(dtype))
    fused = runtime.run_model(head, {"logits": dev(x)})
    plain = runtime.run_model(head, {"logits": dev(x)}, fuse=False)
    p = oracle.softmax(x, -1)
    ev, ei = oracle.topk(p, 5, -1)
    assert np.array_equal(host(plain["indices"]), ei)
    bits = np.uint16 if dtype == np.float16 else np.uint32
    close = half_ulp_diff if dtype == np.float16 else ulp_diff
    assert close(host(plain["values"]), ev).max() <= 2
    assert close(host(fused["values"]), host(plain["values"])).max() <= 2
    if not np.array_equal(host(fused["indices"]), ei):       # only equal probabilities may trade places
        assert np.array_equal(np.take_along_axis(p, host(fused["indices"]).astype(np.int64), -1).view(bits), ev.view(bits))
    # K from the second input; the probabilities are an output as well
    shared = vkopbin.read_model(os.path.join(GOLDEN_DIR, "classifier_head_k_input.vkopbin"))
    out = runtime.run_model(shared, {"logits": dev(x[:4])})
    assert host(out["values"]).shape == (4, 7)
    ev7, ei7 = oracle.topk(host(out["probs"]), 7, -1)
    assert np.array_equal(host(out["indices"]), ei7) and np.array_equal(host(out["values"]).view(bits), ev7.view(bits))
    # detection chain: softmax over classes, class maximum (one operator when fused), top anchors
    chain = vkopbin.read_model(os.path.join(GOLDEN_DIR, "detection_chain.vkopbin"))
    sc = np.ascontiguousarray(synth.detection_scores(2, 80, 840, 5).astype(dtype))
    probs = oracle.softmax(sc, 1)
    best = oracle.reduce_max(probs, 1) if dtype == np.float32 else probs.max(axis=1)   # (a maximum has no rounding)
    bv, bi = oracle.topk(best, 30, -1)
    for fuse in (True, False):
        out = runtime.run_model(chain, {"scores": dev(sc)}, fuse=fuse)
        assert np.array_equal(host(out["anchors"]), bi) and np.array_equal(host(out["values"]).view(bits), bv.view(bits)), fuse
    # two heads in one model
    two = vkopbin.read_model(os.path.join(GOLDEN_DIR, "two_heads.vkopbin"))
    rng2 = np.random.default_rng(12)
    tb, tsc = _nms_boxes(rng2, 1, 200, 0.4).astype(dtype), rng2.random((1, 4, 200)).astype(dtype)
    out = runtime.run_model(two, {"logits": dev(x[:4]), "boxes": dev(tb), "scores": dev(tsc)})
    ev7, ei7 = oracle.topk(host(out["probs"]), 7, -1)
    assert np.array_equal(host(out["indices"]), ei7) and np.array_equal(host(out["values"]).view(bits), ev7.view(bits))
    assert np.array_equal(host(out["selected"]), oracle.nms(tb.astype(np.float32), tsc.astype(np.float32), 0.4, 0.5, 0,
                                                             max_candidates=2048))
    # detection tail
    tail = vkopbin.read_model(os.path.join(GOLDEN_DIR, "detection_tail.vkopbin"))
    rng = np.random.default_rng(9)
    boxes = _nms_boxes(rng, 2, 300, 0.3).astype(dtype)
    scores = rng.random((2, 3, 300)).astype(dtype)
    got = runtime.run_model(tail, {"boxes": dev(boxes), "scores": dev(scores)})["selected"]
    want = oracle.nms(boxes.astype(np.float32), scores.astype(np.float32), 0.5, 0.25, 0, max_candidates=2048)
    assert np.array_equal(host(got), want) and len(want) > 0
