"""The fused entry point that allocates nothing (vkop_hip_softmax_topk_static)
against the workspace-taking one it is a variant of: bit-identical values and
indices, on two calls in a row (the second on a smaller tensor, so that what the
first left in the library's static scratch is still there), in float32 and
float16, on every route a fused call can take; a tensor beyond the static
scratch is refused with a clear error; and the call records into a HIP graph
(which an allocating call could not) and replays to the same result.

Collected last (the file name sorts after every other test file).
"""
import numpy as np
import pytest

from vkop_amd import synth

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def capi():
    from vkop_amd import capi as _capi
    _capi.lib()   # raises if the HIP library is not built: no fallback
    _capi.init(0)
    return _capi


def _dev(a):
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        a = a.view(np.float16)
    return torch.from_numpy(a).cuda()


def _out_shape(shape, axis, k):
    out = list(shape)
    out[axis] = k
    return out


def _with_workspace(capi, xd, k, axis=-1, largest=1):
    dt = capi.F32 if xd.dtype == torch.float32 else capi.F16
    shape = list(xd.shape)
    need = capi.softmax_topk_workspace_bytes(dt, shape, axis, k)
    ws = torch.zeros(max(need, 4) // 4 + 64, dtype=torch.int32, device="cuda")
    ptr = (ws.data_ptr() + 255) // 256 * 256
    vals = torch.empty(_out_shape(shape, axis, k), dtype=xd.dtype, device="cuda")
    idx = torch.empty(_out_shape(shape, axis, k), dtype=torch.int32, device="cuda")
    capi.softmax_topk(xd.data_ptr(), 0, vals.data_ptr(), idx.data_ptr(), dt, shape, axis, k, largest, ptr, need, 0)
    torch.cuda.synchronize()
    return vals.cpu().numpy(), idx.cpu().numpy(), need


def _static(capi, xd, k, axis=-1, largest=1):
    dt = capi.F32 if xd.dtype == torch.float32 else capi.F16
    shape = list(xd.shape)
    vals = torch.full(_out_shape(shape, axis, k), -1.0, dtype=xd.dtype, device="cuda")
    idx = torch.full(_out_shape(shape, axis, k), -1, dtype=torch.int32, device="cuda")
    capi.softmax_topk_static(xd.data_ptr(), vals.data_ptr(), idx.data_ptr(), dt, shape, axis, k, largest, 0)
    torch.cuda.synchronize()
    return vals.cpu().numpy(), idx.cpu().numpy()


def _bits(a):
    return a.view(np.uint32) if a.dtype == np.float32 else a.view(np.uint16)


def _same(capi, x, k, what, axis=-1, largest=1):
    xd = _dev(x)
    ev, ei, need = _with_workspace(capi, xd, k, axis, largest)
    assert need <= capi.STATIC_SCRATCH_BYTES, what
    gv, gi = _static(capi, xd, k, axis, largest)
    assert np.array_equal(gi, ei), what + ": indices differ"
    assert np.array_equal(_bits(gv), _bits(ev)), what + ": values differ"


@pytest.mark.parametrize("half", [False, True], ids=["f32", "f16"])
def test_static_scratch_matches_the_workspace_entry_point_twice_in_a_row(capi, half):
    def cast(x):
        return x.astype(np.float16) if half else x
    # several chunks per row (the streaming kernels with a workspace hand-over) ...
    _same(capi, cast(synth.llm_logits(16, 128256, seed=41)), 50, "first call [16,128256]")
    # ... then a smaller tensor of another shape on what that call left behind
    _same(capi, cast(synth.llm_logits(5, 40000, seed=42)), 7, "second call [5,40000]")
    # rows that one workgroup holds, and the same shapes once more
    _same(capi, cast(synth.classifier_logits(256, 1000, seed=43)), 5, "third call [256,1000]")
    _same(capi, cast(synth.llm_logits(16, 128256, seed=44)), 50, "fourth call [16,128256]")


def test_static_scratch_large_k_route_and_ties(capi):
    # k above the streaming kernels' limit on long rows: the multi-workgroup select
    x = synth.grid_values(2, 65536, seed=45)
    _same(capi, x, 600, "grid [2,65536] k=600")
    _same(capi, x[:1, :20000], 300, "grid [1,20000] k=300")


def test_static_scratch_on_the_other_routes_each_after_a_call_of_a_different_one(capi):
    """The array is never cleared between calls: every route has to cope with what another one left.
    The multi-pass radix select (its histograms, state and counts), the chunk + merge kernels over
    several chunks (rows.path = 1), lines along a non-last axis (the general kernels' line statistics)
    and the smallest-first direction, each right after a call that used the same bytes otherwise."""
    rng = np.random.default_rng(47)
    scan = synth.llm_logits(8, 65536, seed=48)
    _same(capi, scan, 40, "scan + pick first")
    # half-precision rows with too few blocks for the scan kernels at this k: the radix select
    x = (rng.standard_normal((64, 60000)) * 2).astype(np.float16)
    assert capi.measure_path(capi.F16, [64, 60000], -1, 300) == 0
    _same(capi, x, 300, "radix select after scan + pick")
    _same(capi, scan, 40, "scan + pick after the radix select")
    try:
        capi.tune("rows.path", 1)
        assert capi.measure_path(capi.F32, [6, 40000], -1, 16) == 1 and capi.rows_plan(capi.F32, [6, 40000], -1, 16)[2] > 1
        _same(capi, synth.llm_logits(6, 40000, seed=49), 16, "chunk + merge over several chunks after scan + pick")
    finally:
        capi.tune("rows.path", 0)
    y = (rng.standard_normal((3, 700, 40)) * 2).astype(np.float32)
    _same(capi, y, 9, "lines along axis 1 after chunk + merge", axis=1)
    _same(capi, scan, 25, "smallest first after the line kernels", largest=0)
    _same(capi, x, 100, "half precision, smallest first", largest=0)
    _same(capi, scan, 40, "and scan + pick once more")


def test_static_scratch_refuses_what_it_cannot_hold(capi):
    shape = [4096, 128256]
    need = capi.softmax_topk_workspace_bytes(capi.F32, shape, -1, 50)
    assert need > capi.STATIC_SCRATCH_BYTES
    x = torch.zeros(8, device="cuda")
    with pytest.raises(capi.VkopHipError) as e:   # refused before anything is launched: the pointers are never used
        capi.softmax_topk_static(x.data_ptr(), x.data_ptr(), x.data_ptr(), capi.F32, shape, -1, 50, 1, 0)
    assert e.value.code == capi.ERR_WORKSPACE
    assert "static" in str(e.value)


def test_static_scratch_call_records_into_a_graph(capi):
    x = synth.llm_logits(8, 50000, seed=46)
    xd = _dev(x)
    k = 20
    ev, ei, _ = _with_workspace(capi, xd, k)
    vals = torch.zeros(8, k, dtype=torch.float32, device="cuda")
    idx = torch.zeros(8, k, dtype=torch.int32, device="cuda")
    st = capi.stream_create()
    try:
        capi.graph_begin(st)
        capi.softmax_topk_static(xd.data_ptr(), vals.data_ptr(), idx.data_ptr(), capi.F32, [8, 50000], -1, k, 1, st)
        g = capi.graph_end(st)
        try:
            for _ in range(3):
                vals.zero_()
                idx.zero_()
                torch.cuda.synchronize()
                capi.graph_launch(g, st)
                capi.stream_sync(st)
                assert np.array_equal(idx.cpu().numpy(), ei)
                assert np.array_equal(vals.cpu().numpy().view(np.uint32), ev.view(np.uint32))
        finally:
            capi.graph_destroy(g)
    finally:
        capi.stream_destroy(st)
