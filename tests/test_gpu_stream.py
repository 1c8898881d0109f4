"""The scan + pick kernel pair (long last-axis rows) and the sampling-style entry
point, on the GPU, through the C ABI.

* The pair against the chunk + merge kernels it stands in for (vkop_hip_tune
  "rows.path"): bit-identical results -- both implement "top-k by (probability, then
  lower index) of the row's softmax" and sum the row's terms in orders of their own,
  so a value may differ by an ulp where the sums round apart; indices, and values
  where the sums agree, are compared exactly, values otherwise to one ulp -- and
  against the oracle: the monotone-ranking invariants on every row, exact indices
  wherever the oracle's probabilities around the cut are well apart.
* vkop_hip_softmax_topk_sampling against the oracle's sampling variant and against
  the plain entry point on a tensor scaled on the host.
* The NaN replacement option of the softmax on axes other than the last.
"""
import numpy as np
import pytest

import oracle
from helpers import check_fused_invariants, check_topk_invariants, half_ulp_diff, ulp_diff, well_separated_cut
from vkop_amd import synth

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def ops():
    from vkop_amd import capi, ops as _ops
    capi.lib()              # raises if the HIP library is not built: no fallback
    capi.init(0)
    yield _ops
    capi.tune("rows.path", 0)


def dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        a = a.view(np.float16)
    return torch.from_numpy(a).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def _rows(kind, rows, n, rng):
    if kind == "llm":
        return synth.llm_logits(rows, n, seed=int(rng.integers(1, 1 << 30)))
    if kind == "grid":        # 513 levels, hundreds of elements on each
        return synth.grid_values(rows, n, seed=int(rng.integers(1, 1 << 30)))
    x = (rng.standard_normal((rows, n)) * 1.5).astype(np.float32)
    if kind == "bf16":        # what a bf16 head hands over: equal logits straddle the cut
        return np.ascontiguousarray((x.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32))
    if kind == "levels":      # 64 levels: massive ties
        return (np.round(x * 8) / 8).astype(np.float32)
    if kind == "sorted":
        x = np.sort(x, axis=1)
        x[1::2] = x[1::2, ::-1]
        return np.ascontiguousarray(x)
    if kind == "masked":      # a few allowed tokens per row, the rest -inf
        m = rng.random((rows, n)) < (40.0 / n)
        x[~m] = -np.inf
        x[0, :] = -np.inf
        x[0, min(5, n - 1)] = 1.0
        return x
    if kind == "constant":
        x[:] = np.float32(-2.5)
        x[1, n // 2:] = np.float32(3.0)
        return x
    if kind == "spikes":      # elements far above their wave's first vectors, and a dominant one
        x[:, n // 3] += 40.0
        x[2, 17::4099] += 25.0
        return x
    if kind == "tenth":       # one value everywhere, not a round one (its key has low bits set)
        x[:] = np.float32(0.1)
        x[rows - 1, :] = np.float32(-7.3)
        return x
    if kind == "two_values":
        return np.where(rng.random((rows, n)) < 0.5, np.float32(1.7), np.float32(1.7000002)).astype(np.float32)
    if kind == "sorted_desc":
        return np.ascontiguousarray(np.sort(x, axis=1)[:, ::-1])
    if kind == "flat_with_peaks":   # one value, and a few larger ones scattered over the row
        x[:] = np.float32(-0.3)
        for r in range(rows):
            at = rng.choice(n, size=min(n, 3 + 2 * r), replace=False)
            x[r, at] = np.float32(2.0) + rng.random(at.size).astype(np.float32)
        return x
    if kind == "runs":        # sorted inside runs of 4096: clustered, not sorted as a whole
        x = x.copy()
        for s0 in range(0, n, 4096):
            x[:, s0:s0 + 4096] = np.sort(x[:, s0:s0 + 4096], axis=1)
        return x
    if kind == "half_half":   # two values, either one in half of the places: the threshold's value is everywhere
        return np.where(rng.random((rows, n)) < 0.5, np.float32(1.0), np.float32(-1.0)).astype(np.float32)
    if kind == "three_allowed":   # three finite elements a row: the rest of the result is -inf, in index order
        x[:] = -np.inf
        x[:, [n // 7, n // 2, n - 3]] = np.float32(0.5)
        return x
    if kind == "nan_and_inf":  # rows of NaN probabilities (NaN ranks first in the plain top-k)
        x[0, n // 2] = np.nan
        x[1, n // 3] = np.inf
        x[2, 5] = np.nan
        x[2, n - 1] = np.nan
        return x
    if kind == "huge":        # differences of thousands: all but a few probabilities are 0 and tie
        return (x * np.float32(1e4)).astype(np.float32)
    if kind == "masked90":    # nine in ten -inf: block maxima of both signs (coarse histogram bins)
        x[rng.random((rows, n)) < 0.9] = -np.inf
        return x
    if kind == "coarse_levels":   # a dozen levels, thousands of elements on the one at the cut
        return (np.round(x) / 2).astype(np.float32)
    if kind == "signed_zeros":    # -0 == +0: one rank group, in index order
        x = np.where(rng.random((rows, n)) < 0.5, np.float32(0.0), np.float32(-0.0)).astype(np.float32)
        x[:, ::1000] = np.float32(1.0)
        return x
    raise ValueError(kind)


KINDS = ["llm", "bf16", "levels", "sorted", "masked", "constant", "spikes"]
TIE_KINDS = ["tenth", "two_values", "sorted_desc", "flat_with_peaks", "runs"]
WALK_KINDS = ["half_half", "three_allowed", "nan_and_inf", "huge", "masked90", "coarse_levels", "signed_zeros", "sorted", "runs",
              "flat_with_peaks"]


def _compare_paths(ops, n, k, dtype, rows, kinds, path):
    """The library's choice of kernels (which has to be `path`) against the kernels
    rows.path = 1 selects, and both against the oracle."""
    from vkop_amd import capi
    rng = np.random.default_rng(n * 31 + k)
    dt = capi.F32 if dtype == np.float32 else capi.F16
    capi.tune("rows.path", 0)
    if capi.measure_path(dt, (rows, n), -1, k) != path:
        pytest.skip("not a shape these kernels take in this element type")
    for kind in kinds:
        x = np.ascontiguousarray(_rows(kind, rows, n, rng).astype(dtype))
        xd = dev(x)
        capi.tune("rows.path", 0)
        v, ix = ops.softmax_topk(xd, k)
        t, tj = ops.topk(xd, k)
        v, ix, t, tj = host(v), host(ix), host(t), host(tj)
        capi.tune("rows.path", 1)
        v1, ix1 = ops.softmax_topk(xd, k)
        t1, tj1 = ops.topk(xd, k)
        v1, ix1, t1, tj1 = host(v1), host(ix1), host(t1), host(tj1)
        capi.tune("rows.path", 0)
        bits = np.uint16 if dtype == np.float16 else np.uint32
        what = (kind, n, k, np.dtype(dtype).name)
        # plain top-k: no arithmetic, everything exact, both pairs and the oracle
        et, ej = oracle.topk(x, k)
        assert np.array_equal(tj, ej) and np.array_equal(t.view(bits), et.view(bits)), what
        assert np.array_equal(tj1, ej) and np.array_equal(t1.view(bits), et.view(bits)), what
        # fused: values within an ulp of the other pair's, to the bar against the oracle
        ov, oix, op = oracle.softmax_topk(x, k, return_probs=True)
        if dtype == np.float16:
            assert half_ulp_diff(v, v1).max() <= 1 and half_ulp_diff(v, ov).max() <= 1, what
        else:
            # (the bar is the distance to the oracle; the radix select behind rows.path = 1 at
            # large k sums accurate terms only, the scan sums fast ones: on rows of few distinct
            # values the two row sums may lie an ulp from the oracle's on either side)
            assert ulp_diff(v, ov).max() <= 2 and ulp_diff(v1, ov).max() <= 2 and ulp_diff(v, v1).max() <= 2, what
        differ = 0
        xf = x.astype(np.float32)
        for r in range(rows):
            vr = v[r].astype(np.float32)
            if not np.array_equal(ix[r], ix1[r]):
                differ += 1      # only where the two row sums round a tie open or closed
                assert not np.array_equal(v[r].view(bits), v1[r].view(bits)) or \
                    sorted(ix[r].tolist()) != sorted(ix1[r].tolist()), what
            if np.isfinite(vr).all():
                check_fused_invariants(xf[r], vr, ix[r])
            else:
                assert np.array_equal(ix[r], np.arange(k)), what       # all-NaN row: lowest indices
            if well_separated_cut(op[r].astype(np.float32), xf[r], k, 4 if dtype == np.float32 else 1 << 14):
                assert np.array_equal(ix[r], oix[r]), (what, r)
        assert differ <= 2, (what, differ)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("n,k", [(128256, 50), (128256, 1), (128256, 255), (40000, 7), (16385, 20), (13057, 50),
                                 (262144, 64), (100003, 33), (500000, 100), (300000, 511), (50257, 300)])
def test_scan_pick_pair_equals_chunk_merge_and_oracle(ops, n, k, dtype):
    """(From k = 256 on the pair is the library's choice on more than 16 rows only, there also
    with fewer than two blocks per wanted place.)"""
    _compare_paths(ops, n, k, dtype, 20 if k >= 256 else 6, KINDS, 2)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("n,k", [(262144, 1024), (262144, 600), (524288, 2048), (200003, 700), (131072, 512),
                                 (300000, 1500), (200000, 300), (50257, 200), (100000, 400)])
def test_scan_with_spread_out_pick_for_large_k_equals_radix_select_and_oracle(ops, n, k, dtype):
    """k beyond one workgroup's candidate list (and, on a few rows, from k = 256 on, or from
    k = 160 where the row has too few blocks for the pick kernel): scan, then the gather and rank kernels
    that spread a row's candidates over many workgroups, against the multi-pass radix
    select (rows.path = 1) and the oracle -- the regular rows, and the ones the pair hands
    to its exact fallback (constant and masked rows, levels with thousands of equals)."""
    _compare_paths(ops, n, k, dtype, 4, KINDS + ["grid"], 3)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("n,k", [(1000, 5), (1000, 16), (33, 5), (5, 5), (1024, 1), (2048, 7), (777, 10), (256, 3), (64, 16),
                                 (1001, 5), (130, 2), (1000, 32), (2048, 24), (1500, 20), (40, 32)])
def test_one_wave_kernel_for_short_rows_equals_chunk_kernel_and_oracle(ops, n, k, dtype):
    """Short rows, small k (a classifier head): the one-wave-per-row kernel against the
    chunk kernel (rows.path = 1) and the oracle, on regular rows and on the ones it hands
    to its exact fallback (ties en masse, masked rows, constant rows), and on rows whose
    probabilities underflow to 0 for all but a few elements (a tie at 0 that runs to the row's end)."""
    _compare_paths(ops, n, k, dtype, 6, KINDS + ["huge", "masked90"], 4)


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("n,k,path", [(128256, 50, 2), (40000, 255, 2), (262144, 200, 2), (1048576, 100, 2), (262144, 1024, 3), (300000, 600, 3), (131072, 800, 3), (1000, 5, 4),
                                      (2048, 16, 4), (2048, 32, 4)])
def test_rows_of_equal_and_clustered_values_on_every_route(ops, n, k, path, dtype):
    """Rows that defeat a threshold taken from block or lane maxima -- one value everywhere
    (with a key that is not a round number), two values a float apart, rows sorted
    downwards, a flat row with a few peaks, rows sorted in runs -- settled by each route's
    own means (a second threshold, the first elements equal to the tie value, block
    minima), against the other kernels and the oracle."""
    _compare_paths(ops, n, k, dtype, 4, TIE_KINDS, path)


@pytest.mark.parametrize("n,k", [(262144, 1024), (262144, 2000), (524288, 2048), (300000, 600), (300001, 700), (65536, 512),
                                 (100000, 1200)])
def test_large_k_rows_whose_cut_falls_into_a_crowd(ops, n, k):
    """The large-k kernels on rows where the threshold's own rank group is too large for the
    candidate lists (one value in half of the places, -inf nearly everywhere, probabilities
    that underflow to 0, -0 and +0, a dozen levels) -- its first members come from a walk over
    the row in index order, also on rows that do not start on 16 bytes -- on rows of NaN
    probabilities, on block maxima of both signs and on sorted rows at a k close to the
    lists' capacity, and on rows with hardly more blocks than wanted places (1.3 a place:
    most of the row is a candidate); against the radix select and the oracle."""
    _compare_paths(ops, n, k, np.float32, 4, WALK_KINDS, 3)


@pytest.mark.parametrize("rows,n,k", [(16, 131072, 1), (32, 50000, 3), (4, 262144, 1024), (8, 100000, 600), (64, 8192, 3),
                                      (256, 1000, 5), (7, 128255, 50)])
def test_rows_of_one_repeated_value_and_a_few_peaks(ops, rows, n, k):
    """One value everywhere but in three places: the row's sum is that value's term times its
    count, and the term is, by definition, the correctly rounded float exponential of the
    ROUNDED difference to the maximum -- off the exact exponential of the exact difference by up
    to 3e-7, the same for every copy.  A streaming pass that sums against a reference of its
    own has to say so exactly (the scan kernel records a wave of equal elements as a count and
    the value), or the probabilities drift by several ulp; every route, the plain softmax too."""
    rng = np.random.default_rng(rows + n + k)
    for rep in range(2):
        x = np.zeros((rows, n), np.float32) + (rng.standard_normal((rows, 1)) * 2).astype(np.float32)
        for r in range(rows):
            x[r, rng.choice(n, 3, replace=False)] = x[r, 0] + (rng.random(3) * 8 + 1).astype(np.float32)
        v, ix = ops.softmax_topk(dev(x), k)
        v, ix = host(v), host(ix)
        ov, oix = oracle.softmax_topk(x, k)
        assert ulp_diff(v, ov).max() <= 2, (rows, n, k, int(ulp_diff(v, ov).max()))
        assert np.array_equal(ix, oix), (rows, n, k)
        y = host(ops.softmax(dev(x)))
        assert ulp_diff(y, oracle.softmax(x)).max() <= 2, (rows, n, k)


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_shapes_k_and_row_kinds_on_whatever_route_they_take(ops, seed):
    """A dozen draws a seed of (rows, n, k, element type, three kinds of rows) through the
    comparison of the library's own choice of kernels with the kernels rows.path = 1 selects and
    with the oracle: the shapes between the ones the other tests name (this is how the rows of
    one repeated value and three peaks, and a row that overflowed a wave's stage twice, were found).
    A flat row with dozens of peaks per thousand copies ([n = 20001, k = 16] under seed 23) measured
    3 ulp on every streaming route until their waves counted the copies of a value that fills them
    apart (a record word of its own: the scan kernel's, then the chunk kernel's): the kind
    "flat_with_peaks" is drawn like any other."""
    from vkop_amd import capi
    rng = np.random.default_rng(seed)
    kinds_all = list(dict.fromkeys(KINDS + TIE_KINDS + WALK_KINDS))
    ns = [33, 64, 100, 255, 256, 257, 777, 1000, 1024, 2047, 2048, 4096, 5000, 8191, 8192, 8400, 12000, 16384, 20001, 32768, 40000,
          50257, 65536, 100000, 128256, 200003]
    ks = [1, 2, 5, 8, 16, 31, 32, 33, 50, 64, 65, 100, 128, 159, 160, 200, 255, 256, 257, 300, 408, 409, 500, 511, 512, 600, 1024, 2000, 2048]
    for _ in range(12):
        n = int(rng.choice(ns))
        k = int(min(n, rng.choice(ks)))
        rows = int(rng.choice([3, 4, 5, 8, 16, 17, 24, 40])) if n <= 65536 else int(rng.choice([3, 4, 8, 16, 17, 20]))
        dtype = np.float32 if rng.random() < 0.6 else np.float16
        kinds = [str(t) for t in rng.choice(kinds_all, size=3, replace=False)]
        capi.tune("rows.path", 0)
        path = capi.measure_path(capi.F32 if dtype == np.float32 else capi.F16, (rows, n), -1, k)
        _compare_paths(ops, n, k, dtype, rows, kinds, path)


@pytest.mark.parametrize("rows,n,k", [(17, 20001, 16), (8, 20001, 16), (24, 50000, 40), (5, 131072, 64), (16, 16385, 5)])
def test_flat_rows_with_dozens_of_peaks_on_the_chunk_and_merge_kernels(ops, rows, n, k):
    """The chunk + merge kernels over several chunks (rows.path = 1: no shape takes them by itself any
    more) on rows that are one value and dozens of peaks: most waves hold a larger element beside the
    copies, all of them sum against references of their own, and the copies' common term error came to
    3 ulp of the probabilities (n = 20001, k = 16) until the chunk kernel's waves counted the copies
    apart, in a record word of their own, for the merge to add them as the sum is defined."""
    from vkop_amd import capi
    rng = np.random.default_rng(rows * 1000 + k)
    x = np.full((rows, n), np.float32(-0.3))
    for r in range(rows):
        at = rng.choice(n, size=20 + 13 * r, replace=False)
        x[r, at] = np.float32(2.0) + rng.random(at.size).astype(np.float32)
    ov, oix = oracle.softmax_topk(x, k)
    try:
        capi.tune("rows.path", 1)
        assert capi.measure_path(capi.F32, (rows, n), -1, k) == 1 and capi.rows_plan(capi.F32, (rows, n), -1, k)[2] > 1
        v, ix = ops.softmax_topk(dev(x), k)
        v, ix = host(v), host(ix)
    finally:
        capi.tune("rows.path", 0)
    assert np.array_equal(ix, oix), (rows, n, k)
    assert ulp_diff(v, ov).max() <= 2, (rows, n, k, int(ulp_diff(v, ov).max()))
    v0, ix0 = ops.softmax_topk(dev(x), k)
    assert np.array_equal(host(ix0), oix) and ulp_diff(host(v0), ov).max() <= 2, (rows, n, k)


@pytest.mark.parametrize("n", [16388, 40002, 128255])
def test_scan_pick_pair_on_rows_that_do_not_start_on_16_bytes(ops, n):
    """n not a multiple of the vector width (rows after the first are unaligned), and a
    tensor that starts two elements into an allocation: the element-wise load variants."""
    rng = np.random.default_rng(n)
    for dtype in (np.float32, np.float16):
        x = np.ascontiguousarray((rng.standard_normal((5, n)) * 2).astype(dtype))
        x[3, ::5] = x[3, 1]
        big = torch.empty(5 * n + 8, dtype=torch.float32 if dtype == np.float32 else torch.float16, device="cuda")
        xd = big[2:2 + 5 * n].view(5, n)
        xd.copy_(dev(x))
        for k in (5, 60):
            v, ix = ops.softmax_topk(xd, k)
            t, tj = ops.topk(xd, k)
            v, ix, t, tj = host(v), host(ix), host(t), host(tj)
            et, ej = oracle.topk(x, k)
            bits = np.uint16 if dtype == np.float16 else np.uint32
            assert np.array_equal(tj, ej) and np.array_equal(t.view(bits), et.view(bits)), (n, k)
            ov, oix, op = oracle.softmax_topk(x, k, return_probs=True)
            if dtype == np.float16:
                assert half_ulp_diff(v, ov).max() <= 1
            else:
                assert ulp_diff(v, ov).max() <= 2
            for r in range(5):
                check_fused_invariants(x[r].astype(np.float32), v[r].astype(np.float32), ix[r])
                if well_separated_cut(op[r].astype(np.float32), x[r].astype(np.float32), k, 4 if dtype == np.float32 else 1 << 14):
                    assert np.array_equal(ix[r], oix[r]), (n, k, r)


def test_plain_topk_nan_ranks_first_through_the_scan_pick_pair(ops):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 70000)).astype(np.float32)
    x[0, [5, 69999, 30000]] = np.nan
    x[1, ::3] = np.nan                       # more NaN than k
    x[2, 1000] = np.inf
    x[2, 2000] = -np.inf
    x[3, :] = np.nan
    for k in (1, 4, 100):
        t, tj = ops.topk(dev(x), k)
        et, ej = oracle.topk(x, k)
        assert np.array_equal(host(tj), ej) and np.array_equal(host(t).view(np.uint32), et.view(np.uint32)), k


# ------------------------------------------------------------ sampling variant --

@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape,k", [((16, 128256), 50), ((3, 40000), 7), ((256, 1000), 5), ((2, 33), 33), ((5, 2, 4097), 9),
                                     ((64, 8192), 40), ((16, 8400), 300), ((40, 4096), 64), ((300, 257), 8), ((7, 20000), 100),
                                     ((4, 262144), 1024)])
def test_sampling_variant_against_the_oracle(ops, shape, k, dtype):
    rng = np.random.default_rng(shape[-1] + k)
    x = synth.llm_logits(int(np.prod(shape[:-1])), shape[-1], seed=shape[-1], temperature=1.0).reshape(shape)
    x = np.ascontiguousarray(x.astype(dtype))
    bits = np.uint16 if dtype == np.float16 else np.uint32
    for scale, top_p in ((1.25, 0.9), (1.0, 0.5), (0.5, 0.999), (3.0, 0.2)):
        v, ix, c = ops.softmax_topk_sampling(dev(x), k, scale, top_p)
        v, ix, c = host(v), host(ix), host(c)
        ov, oix, oc = oracle.softmax_topk_sampling(x, k, scale, top_p)
        what = (shape, k, scale, top_p)
        if dtype == np.float16:
            assert half_ulp_diff(v, ov).max() <= 1, what
        else:
            assert ulp_diff(v, ov).max() <= 2, what
        # the count is a function of the stored values: exact against the pinned CPU rule on them,
        # and equal to the separate entry point's
        vf = v.astype(np.float32).reshape(-1, k)
        assert np.array_equal(c.reshape(-1), oracle.topp_count(vf, top_p)), what
        same_values = np.array_equal(v.view(bits), ov.view(bits))
        if same_values:
            assert np.array_equal(c, oc), what
        # bit for bit the plain entry point on a tensor scaled on the host (one float32 product per element)
        xs = (x.astype(np.float32) * np.float32(scale)).astype(np.float32)
        # (bit for bit where both run the scan + pick kernels; other shapes take the line kernels here and the
        # one-workgroup streaming kernels there, which add up the row in different orders: both within the 2-ulp bar of the oracle)
        if dtype == np.float32:
            from vkop_amd import capi
            pv, pix = ops.softmax_topk(dev(xs), k)
            pv, pix = host(pv), host(pix)
            if capi.measure_path(capi.F32, shape, -1, k) == 2:
                assert np.array_equal(pix, ix) and np.array_equal(pv.view(np.uint32), v.view(np.uint32)), what
            else:
                assert ulp_diff(pv, v).max() <= 2, what
        xf = (x.astype(np.float32) * np.float32(scale)).reshape(-1, shape[-1])
        op = oracle.softmax(xf)
        for r in range(xf.shape[0]):
            check_fused_invariants(xf[r], vf[r], ix.reshape(-1, k)[r])
            if dtype == np.float32 and well_separated_cut(op[r], xf[r], k):
                assert np.array_equal(ix.reshape(-1, k)[r], oix.reshape(-1, k)[r]), (what, r)


@pytest.mark.parametrize("n", [50000, 8192, 1000, 8400])
def test_sampling_variant_ties_special_rows_and_errors(ops, n):
    """(n = 50000: the scan + pick kernels; the shorter rows: one workgroup, or one wave, per row)"""
    from vkop_amd import capi
    rng = np.random.default_rng(9)
    x = (np.round(rng.standard_normal((6, n)) * 4) / 4).astype(np.float32)   # ties across the cut
    x[1, 10:] = -np.inf                     # fewer elements above -inf than k
    x[2, 77] = np.nan                       # an all-NaN result
    x[3] = 1.5                              # a constant row
    k = 40
    v, ix, c = ops.softmax_topk_sampling(dev(x), k, 0.75, 0.8)
    v, ix, c = host(v), host(ix), host(c)
    with np.errstate(invalid="ignore"):
        ov, oix, oc = oracle.softmax_topk_sampling(x, k, 0.75, 0.8)
    assert np.array_equal(np.isnan(v), np.isnan(ov))
    assert ulp_diff(v, ov).max() <= 2
    assert np.array_equal(ix[2], np.arange(k)) and c[2] == k
    assert np.array_equal(ix[3], np.arange(k)) and np.array_equal(ix[1][:10], oix[1][:10])
    ok = ~np.isnan(v).any(axis=1)
    assert np.array_equal(c[ok], oracle.topp_count(v[ok], 0.8))
    xs = (x * np.float32(0.75)).astype(np.float32)
    for r in np.nonzero(ok)[0]:
        check_fused_invariants(xs[r], v[r], ix[r])
    xd = dev(x)
    out = torch.empty((6, k), dtype=torch.float32, device="cuda")
    oi = torch.empty((6, k), dtype=torch.int32, device="cuda")
    ws = torch.zeros(1 << 22, dtype=torch.uint8, device="cuda")
    ptr = (ws.data_ptr() + 255) // 256 * 256
    for bad in (0.0, -1.0, float("inf"), float("nan")):
        with pytest.raises(capi.VkopHipError) as e:
            capi.softmax_topk_sampling(xd.data_ptr(), out.data_ptr(), oi.data_ptr(), 0, capi.F32, x.shape, -1, k, bad, 0.5, ptr,
                                       1 << 21, 0)
        assert e.value.code == capi.ERR_INVALID
    with pytest.raises(capi.VkopHipError) as e:   # the count along an axis that is not the last
        capi.softmax_topk_sampling(xd.data_ptr(), out.data_ptr(), oi.data_ptr(), oi.data_ptr(), capi.F32, x.shape, 0, 3, 1.0, 0.5,
                                   ptr, 1 << 21, 0)
    assert e.value.code == capi.ERR_UNSUPPORTED


# ------------------------------------------ softmax: NaN option on the other axes --

@pytest.mark.parametrize("shape,axis", [((130, 70), 0), ((5, 130, 70), 1), ((2, 3, 40, 9), 2), ((80, 8400), 0), ((3, 4, 5, 6), 0),
                                        ((4, 3000, 3), 1)])
def test_nan_replacement_on_axes_other_than_the_last(ops, shape, axis):
    """shaders/softmax2.comp:177-181 implements the option for axis 0 of a matrix; here every axis."""
    rng = np.random.default_rng(sum(shape) + axis)
    for dtype in (np.float32, np.float16):
        x = rng.standard_normal(shape).astype(np.float32)
        idx = tuple(rng.integers(0, s, size=6) for s in shape)
        x[idx] = np.nan                                     # lines holding a NaN: all of the line's outputs are NaN
        line = [0] * len(shape)
        line[axis] = slice(None)
        x[tuple(line)] = -np.inf                            # a line of -inf: NaN too
        x = np.ascontiguousarray(x.astype(dtype))
        with np.errstate(invalid="ignore"):
            exp = oracle.softmax(x, axis)
            expn = oracle.softmax(x, axis, nan_where=1, nan_value=0.25)
        assert np.isnan(exp.astype(np.float32)).any()
        got = host(ops.softmax(dev(x), axis))
        gotn = host(ops.softmax(dev(x), axis, nan_where=True, nan_value=0.25))
        assert np.array_equal(np.isnan(got.astype(np.float32)), np.isnan(exp.astype(np.float32)))
        assert not np.isnan(gotn.astype(np.float32)).any()
        assert np.array_equal(gotn.astype(np.float32) == 0.25, (expn.astype(np.float32) == 0.25))
        if dtype == np.float16:
            assert half_ulp_diff(gotn, expn).max() <= 1
        else:
            assert ulp_diff(gotn, expn).max() <= 2


# ------------------------------------------------------------ the benchmark's timeline leg --

def test_bench_timeline_leg_sees_every_lane(ops):
    """bench.py --timeline (a child process on libvkop_hip_timeline.so, whose scan and pick kernels log their own
    device timestamps): the summary names as many lanes as calls were in flight, and its per-call time from the
    log agrees with the HIP-event figure of the same pass."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if not os.path.exists(os.path.join(root, "vkop_amd", "libvkop_hip_timeline.so")):
        pytest.skip("libvkop_hip_timeline.so is not built (make -C vkop_amd/csrc timeline)")
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--timeline", "--hw-queues", "8", "--inflight", "3",
                        "--steps", "120", "--warmup", "12"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-500:]
    out = json.loads([line for line in r.stdout.splitlines() if line.startswith("{")][-1])
    assert out.get("lanes_seen") == 3, out
    assert 0.7 < out["us_per_call_from_the_log"] / out["us_per_step_by_hip_events_same_run"] < 1.3, out
    assert 1.0 < out["mean_kernels_running"] <= 3.2, out
