"""ctypes binding of the C ABI in include/vkop_hip.h (vkop_amd/libvkop_hip.so).

There is no fallback: if the library is not built, or a call fails, this module
raises.  Pointers are plain integers (device addresses), streams are
hipStream_t values as integers (0 = default stream).
"""
import ctypes
import os
import re
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(_HERE)
LIB_PATH = os.path.join(_HERE, "libvkop_hip.so")
# the same library built with the benchmark's hook (vkop_hip_measure_stages): bench.py's per-kernel legs load
# this one instead, in a process of their own (use_bench_library() before the first lib())
BENCH_LIB_PATH = os.path.join(_HERE, "libvkop_hip_bench.so")
BENCH_ONLY = ("vkop_hip_measure_stages",)
HEADER_PATH = os.path.join(ROOT, "include", "vkop_hip.h")

OK, ERR_INVALID, ERR_DEVICE, ERR_WORKSPACE, ERR_UNSUPPORTED = 0, 1, 2, 3, 4
F32, F16 = 0, 1
MAX_K = 2048


class VkopHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("vkop_hip error %d: %s" % (code, message))
        self.code = code


def build():
    """Compile vkop_amd/libvkop_hip.so for gfx950 with hipcc (no GPU needed), its benchmark build
    (libvkop_hip_bench.so) and the build whose headline kernels log a timeline (libvkop_hip_timeline.so)."""
    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), "-B"])
    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), "timeline"])
    return LIB_PATH


def declared_symbols():
    """Names of every function include/vkop_hip.h declares."""
    text = open(HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vkop_hip_[a-z0-9_]+)\s*\(", text)))


TIMELINE_LIB_PATH = os.path.join(_HERE, "libvkop_hip_timeline.so")


def use_timeline_library():
    """Load libvkop_hip_timeline.so (`make -C vkop_amd/csrc timeline`: the float softmax scan / pick kernels log
    device timestamps per workgroup) instead of libvkop_hip.so (only before the first lib())."""
    global LIB_PATH
    if _lib is not None:
        raise RuntimeError("the library is loaded already")
    if not os.path.exists(TIMELINE_LIB_PATH):
        raise RuntimeError("%s is not built: run `make -C vkop_amd/csrc timeline`" % TIMELINE_LIB_PATH)
    LIB_PATH = TIMELINE_LIB_PATH


def timeline_records(cap=1 << 20):
    """The timeline library's log since the last call: an array [n, 3] of uint64 (tag, entry, exit); tag = kernel
    (bit 63: 0 scan, 1 pick) | workgroup << 40 | bits of the call's workspace address; clocks in 10 ns."""
    import numpy as np
    fn = lib().vkop_hip_dbg_timeline
    fn.argtypes = [ctypes.c_void_p, ctypes.c_uint]
    fn.restype = ctypes.c_int
    arr = np.zeros((cap, 3), dtype=np.uint64)
    n = fn(arr.ctypes.data, cap)
    if n < 0:
        raise RuntimeError("reading the timeline failed")
    return arr[:n]


def use_bench_library():
    """Load libvkop_hip_bench.so instead of libvkop_hip.so (only before the first lib())."""
    global LIB_PATH
    if _lib is not None:
        raise RuntimeError("the library is loaded already")
    LIB_PATH = BENCH_LIB_PATH


def internal_symbols():
    """Names of the measurement hooks vkop_amd/csrc/vkop_hip_internal.h declares (not part of the public interface;
    those in BENCH_ONLY exist in libvkop_hip_bench.so alone)."""
    text = open(os.path.join(_HERE, "csrc", "vkop_hip_internal.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vkop_hip_[a-z0-9_]+)\s*\(", text)))


_lib = None


def lib():
    """The loaded library with argument types set.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            "%s is not built; run `python -c 'import __graft_entry__ as g; g.build()'` or "
            "`make -C vkop_amd/csrc`" % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    i, f, vp, sz = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
    ip = ctypes.POINTER(ctypes.c_int)
    sig = {
        "vkop_hip_nms_workspace_bytes": (sz, [i, i, i, i]),
        "vkop_hip_nms": (i, [vp, vp, vp, i, vp, i, i, i, i, i, i, f, f, vp, sz, vp]),
        "vkop_hip_topp_count": (i, [vp, vp, i, i, i, i, f, vp]),
        "vkop_hip_init": (i, [i]),
        "vkop_hip_shutdown": (i, []),
        "vkop_hip_last_error": (ctypes.c_char_p, []),
        "vkop_hip_device_info": (i, [ctypes.c_char_p, sz, ip, ctypes.POINTER(sz)]),
        "vkop_hip_malloc": (i, [ctypes.POINTER(vp), sz]),
        "vkop_hip_free": (i, [vp]),
        "vkop_hip_memcpy_h2d": (i, [vp, vp, sz, vp]),
        "vkop_hip_memcpy_d2h": (i, [vp, vp, sz, vp]),
        "vkop_hip_memcpy_d2d": (i, [vp, vp, sz, vp]),
        "vkop_hip_stream_create": (i, [ctypes.POINTER(vp)]),
        "vkop_hip_stream_destroy": (i, [vp]),
        "vkop_hip_stream_sync": (i, [vp]),
        "vkop_hip_event_create": (i, [ctypes.POINTER(vp)]),
        "vkop_hip_event_destroy": (i, [vp]),
        "vkop_hip_event_record": (i, [vp, vp]),
        "vkop_hip_event_sync": (i, [vp]),
        "vkop_hip_stream_wait_event": (i, [vp, vp]),
        "vkop_hip_event_elapsed_ms": (i, [vp, vp, ctypes.POINTER(f)]),
        "vkop_hip_graph_begin": (i, [vp]),
        "vkop_hip_graph_end": (i, [vp, ctypes.POINTER(vp)]),
        "vkop_hip_graph_launch": (i, [vp, vp]),
        "vkop_hip_graph_destroy": (i, [vp]),
        "vkop_hip_workspace_init": (i, [vp, sz, vp]),
        "vkop_hip_softmax_workspace_bytes": (sz, [i, ip, i, i]),
        "vkop_hip_softmax": (i, [vp, vp, i, ip, i, i, i, f, vp, sz, vp]),
        "vkop_hip_topk_workspace_bytes": (sz, [i, ip, i, i, i]),
        "vkop_hip_topk": (i, [vp, vp, vp, i, ip, i, i, i, i, i, vp, sz, vp]),
        "vkop_hip_softmax_topk_workspace_bytes": (sz, [i, ip, i, i, i]),
        "vkop_hip_softmax_topk": (i, [vp, vp, vp, vp, i, ip, i, i, i, i, vp, sz, vp]),
        "vkop_hip_softmax_topk_static": (i, [vp, vp, vp, i, ip, i, i, i, i, vp]),
        "vkop_hip_softmax_topk_sampling": (i, [vp, vp, vp, vp, i, ip, i, i, i, f, f, vp, sz, vp]),
        "vkop_hip_reduce_max": (i, [vp, vp, i, ip, i, i, vp]),
        "vkop_hip_softmax_reduce_max_workspace_bytes": (sz, [i, ip, i, i]),
        "vkop_hip_softmax_reduce_max": (i, [vp, vp, i, ip, i, i, vp, sz, vp]),
        "vkop_hip_tune": (i, [ctypes.c_char_p, i]),
        "vkop_hip_measure_stages": (i, [i]),
        "vkop_hip_measure_path": (i, [i, ip, i, i, i]),
        "vkop_hip_rows_plan": (i, [i, ip, i, i, i, ip, ip, ip]),
    }
    for name in BENCH_ONLY:
        if not hasattr(L, name):
            del sig[name]
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    L._signatures = sig
    _lib = L
    return L


def last_error():
    return lib().vkop_hip_last_error().decode("utf-8", "replace")


def check(code):
    if code != OK:
        raise VkopHipError(code, last_error())


def _shape(shape):
    arr = (ctypes.c_int * max(len(shape), 1))(*[int(s) for s in shape])
    return arr, len(shape)


def init(device=0):
    check(lib().vkop_hip_init(int(device)))


def device_info():
    name = ctypes.create_string_buffer(256)
    cus = ctypes.c_int(0)
    mem = ctypes.c_size_t(0)
    check(lib().vkop_hip_device_info(name, 256, ctypes.byref(cus), ctypes.byref(mem)))
    return name.value.decode(), cus.value, mem.value


def malloc(nbytes):
    p = ctypes.c_void_p(0)
    check(lib().vkop_hip_malloc(ctypes.byref(p), int(nbytes)))
    return p.value or 0


def free(ptr):
    check(lib().vkop_hip_free(ptr))


def stream_create():
    s = ctypes.c_void_p(0)
    check(lib().vkop_hip_stream_create(ctypes.byref(s)))
    return s.value or 0


def stream_destroy(s):
    check(lib().vkop_hip_stream_destroy(s))


def stream_sync(s=0):
    check(lib().vkop_hip_stream_sync(s))


def event_create():
    e = ctypes.c_void_p(0)
    check(lib().vkop_hip_event_create(ctypes.byref(e)))
    return e.value


def event_destroy(e):
    check(lib().vkop_hip_event_destroy(e))


def event_record(e, stream=0):
    check(lib().vkop_hip_event_record(e, stream))


def event_sync(e):
    check(lib().vkop_hip_event_sync(e))


def event_elapsed_ms(start, stop):
    ms = ctypes.c_float(0)
    check(lib().vkop_hip_event_elapsed_ms(start, stop, ctypes.byref(ms)))
    return ms.value


def graph_begin(stream):
    check(lib().vkop_hip_graph_begin(stream))


def graph_end(stream):
    g = ctypes.c_void_p(0)
    check(lib().vkop_hip_graph_end(stream, ctypes.byref(g)))
    return g.value


def graph_launch(graph, stream):
    check(lib().vkop_hip_graph_launch(graph, stream))


def graph_destroy(graph):
    check(lib().vkop_hip_graph_destroy(graph))


def workspace_init(ptr, nbytes, stream=0):
    check(lib().vkop_hip_workspace_init(ptr, int(nbytes), stream))


def softmax_workspace_bytes(dtype, shape, axis):
    arr, nd = _shape(shape)
    return lib().vkop_hip_softmax_workspace_bytes(dtype, arr, nd, axis)


def softmax(inp, out, dtype, shape, axis, nan_where=0, nan_value=0.0, workspace=0, workspace_bytes=0, stream=0):
    arr, nd = _shape(shape)
    check(lib().vkop_hip_softmax(inp, out, dtype, arr, nd, axis, int(nan_where), float(nan_value), workspace,
                                 workspace_bytes, stream))


def topk_workspace_bytes(dtype, shape, axis, k):
    arr, nd = _shape(shape)
    return lib().vkop_hip_topk_workspace_bytes(dtype, arr, nd, axis, k)


def topk(inp, values, indices, dtype, shape, axis, k, largest=1, sorted_=1, workspace=0, workspace_bytes=0, stream=0):
    arr, nd = _shape(shape)
    check(lib().vkop_hip_topk(inp, values, indices, dtype, arr, nd, axis, int(k), int(largest), int(sorted_),
                              workspace, workspace_bytes, stream))


def softmax_topk_workspace_bytes(dtype, shape, axis, k):
    arr, nd = _shape(shape)
    return lib().vkop_hip_softmax_topk_workspace_bytes(dtype, arr, nd, axis, k)


def softmax_topk(inp, probs, values, indices, dtype, shape, axis, k, largest=1, workspace=0, workspace_bytes=0,
                 stream=0):
    arr, nd = _shape(shape)
    check(lib().vkop_hip_softmax_topk(inp, probs, values, indices, dtype, arr, nd, axis, int(k), int(largest),
                                      workspace, workspace_bytes, stream))


def softmax_topk_sampling(inp, values, indices, counts, dtype, shape, axis, k, scale, top_p, workspace=0, workspace_bytes=0,
                          stream=0):
    """Fused softmax -> top-k of fl32(x * scale); counts (0 = none): nucleus cut per row for top_p."""
    arr, nd = _shape(shape)
    check(lib().vkop_hip_softmax_topk_sampling(inp, values, indices, counts, dtype, arr, nd, axis, int(k), float(scale),
                                               float(top_p), workspace, workspace_bytes, stream))


STATIC_SCRATCH_BYTES = 4 << 20


def softmax_topk_static(inp, values, indices, dtype, shape, axis, k, largest=1, stream=0):
    """The fused call on the library's own static scratch: allocates nothing."""
    arr, nd = _shape(shape)
    check(lib().vkop_hip_softmax_topk_static(inp, values, indices, dtype, arr, nd, axis, int(k), int(largest), stream))


def reduce_max(inp, out, dtype, shape, axis, stream=0):
    arr, nd = _shape(shape)
    check(lib().vkop_hip_reduce_max(inp, out, dtype, arr, nd, axis, stream))


def topp_count(values, counts, dtype, rows, k, row_stride, p, stream=0):
    check(lib().vkop_hip_topp_count(values, counts, int(dtype), int(rows), int(k), int(row_stride), float(p), stream))


def tune(name, value):
    """Process-wide tuning / measurement knob (see include/vkop_hip.h)."""
    check(lib().vkop_hip_tune(name.encode(), int(value)))


def measure_stages(stages):
    """Benchmarks only (vkop_amd/csrc/vkop_hip_internal.h): launch only the first (1) or second (2) kernel of a
    two-kernel streaming call, or both (3, the normal state).  Results are not valid with 1 or 2.
    libvkop_hip_bench.so only (use_bench_library())."""
    if not hasattr(lib(), "vkop_hip_measure_stages"):
        raise RuntimeError("vkop_hip_measure_stages exists only in libvkop_hip_bench.so: call capi.use_bench_library() first")
    check(lib().vkop_hip_measure_stages(int(stages)))


def measure_path(dtype, shape, axis, k):
    """Benchmarks only: 2 = scan + pick kernels, 1 = chunk (+ merge) kernels, 0 = other kernels for this tensor."""
    arr, nd = _shape(shape)
    return lib().vkop_hip_measure_path(dtype, arr, nd, axis, int(k))


def rows_plan(dtype, shape, axis, k):
    """(threads, loads, chunks) of the streaming kernel for this tensor; zeros = general kernels."""
    arr, nd = _shape(shape)
    t, l, c = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    check(lib().vkop_hip_rows_plan(dtype, arr, nd, axis, k, ctypes.byref(t), ctypes.byref(l), ctypes.byref(c)))
    return t.value, l.value, c.value


def stream_wait_event(stream, event):
    """Work enqueued on `stream` after this call waits for `event`."""
    check(lib().vkop_hip_stream_wait_event(stream, event))


def memcpy_h2d(dst_device, src_host, nbytes, stream=0):
    """Blocking host -> device copy ordered on `stream`."""
    check(lib().vkop_hip_memcpy_h2d(dst_device, src_host, int(nbytes), stream))


def memcpy_d2h(dst_host, src_device, nbytes, stream=0):
    """Blocking device -> host copy ordered on `stream`."""
    check(lib().vkop_hip_memcpy_d2h(dst_host, src_device, int(nbytes), stream))


def softmax_reduce_max_workspace_bytes(dtype, shape, axis):
    arr, nd = _shape(shape)
    return lib().vkop_hip_softmax_reduce_max_workspace_bytes(dtype, arr, nd, axis)


def softmax_reduce_max(inp, out, dtype, shape, axis, workspace=0, workspace_bytes=0, stream=0):
    arr, nd = _shape(shape)
    check(lib().vkop_hip_softmax_reduce_max(inp, out, dtype, arr, nd, axis, workspace, workspace_bytes, stream))


def nms_workspace_bytes(B, C, N, max_output_boxes_per_class=0):
    return int(lib().vkop_hip_nms_workspace_bytes(int(B), int(C), int(N), int(max_output_boxes_per_class)))


def nms(boxes, scores, out, out_capacity, out_count, dtype, B, C, N, center_point_box, max_output_boxes_per_class,
        iou_threshold, score_threshold, workspace, workspace_bytes, stream=0):
    check(lib().vkop_hip_nms(boxes, scores, out, int(out_capacity), out_count, int(dtype), int(B), int(C), int(N),
                             int(center_point_box), int(max_output_boxes_per_class), float(iou_threshold),
                             float(score_threshold), workspace, int(workspace_bytes), stream))
