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


def _with_workspace(capi, xd, k):
    dt = capi.F32 if xd.dtype == torch.float32 else capi.F16
    shape = list(xd.shape)
    need = capi.softmax_topk_workspace_bytes(dt, shape, -1, k)
    ws = torch.zeros(max(need, 4) // 4 + 64, dtype=torch.int32, device="cuda")
    ptr = (ws.data_ptr() + 255) // 256 * 256
    vals = torch.empty(shape[:-1] + [k], dtype=xd.dtype, device="cuda")
    idx = torch.empty(shape[:-1] + [k], dtype=torch.int32, device="cuda")
    capi.softmax_topk(xd.data_ptr(), 0, vals.data_ptr(), idx.data_ptr(), dt, shape, -1, k, 1, ptr, need, 0)
    torch.cuda.synchronize()
    return vals.cpu().numpy(), idx.cpu().numpy(), need


def _static(capi, xd, k):
    dt = capi.F32 if xd.dtype == torch.float32 else capi.F16
    shape = list(xd.shape)
    vals = torch.full(shape[:-1] + [k], -1.0, dtype=xd.dtype, device="cuda")
    idx = torch.full(shape[:-1] + [k], -1, dtype=torch.int32, device="cuda")
    capi.softmax_topk_static(xd.data_ptr(), vals.data_ptr(), idx.data_ptr(), dt, shape, -1, k, 1, 0)
    torch.cuda.synchronize()
    return vals.cpu().numpy(), idx.cpu().numpy()


def _bits(a):
    return a.view(np.uint32) if a.dtype == np.float32 else a.view(np.uint16)


def _same(capi, x, k, what):
    xd = _dev(x)
    ev, ei, need = _with_workspace(capi, xd, k)
    assert need <= capi.STATIC_SCRATCH_BYTES, what
    gv, gi = _static(capi, xd, k)
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
