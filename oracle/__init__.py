"""numpy front-end of the CPU oracle (oracle/vkop_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg, never by the shipped package.  Every function
takes and returns host numpy arrays; half precision travels as uint16 bit
patterns or as numpy float16 (both accepted, float16 returned).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libvkop_oracle.so")
_lib = None


def build(force=False):
    """Compile oracle/libvkop_oracle.so with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libvkop_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        c_int, c_float, vp = ctypes.c_int, ctypes.c_float, ctypes.c_void_p
        L.vkop_oracle_half_to_float.restype = c_float
        L.vkop_oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.vkop_oracle_float_to_half.restype = ctypes.c_uint16
        L.vkop_oracle_float_to_half.argtypes = [c_float]
        for name in ("vkop_oracle_softmax_f32", "vkop_oracle_softmax_f16"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, vp, c_int, c_int, c_int, c_int, c_float]
        for name in ("vkop_oracle_topk_f32", "vkop_oracle_topk_f16"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, vp, vp, c_int, c_int, c_int, c_int, c_int]
        for name in ("vkop_oracle_softmax_topk_f32", "vkop_oracle_softmax_topk_f16"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, vp, vp, vp, c_int, c_int, c_int, c_int, c_int]
        L.vkop_oracle_softmax_topk_f32_mt.restype = c_int
        L.vkop_oracle_softmax_topk_f32_mt.argtypes = [vp, vp, vp, c_int, c_int, c_int, c_int, c_int, c_int]
        for name in ("vkop_oracle_softmax_topk_sampling_f32", "vkop_oracle_softmax_topk_sampling_f16"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, c_float, c_float, vp, vp, vp, c_int, c_int, c_int, c_int]
        L.vkop_oracle_reduce_max_f32.restype = None
        L.vkop_oracle_reduce_max_f32.argtypes = [vp, vp, c_int, c_int, c_int]
        L.vkop_oracle_get_top_k_predictions.restype = c_int
        L.vkop_oracle_get_top_k_predictions.argtypes = [vp, c_int, c_int, vp, vp]
        L.vkop_oracle_nms_f32.restype = c_int
        L.vkop_oracle_topp_count_f32.argtypes = [vp, c_int, c_int, c_int, c_float, vp]
        L.vkop_oracle_topp_count_f32.restype = None
        L.vkop_oracle_nms_f32.argtypes = [vp, vp, vp, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_int]
        _lib = L
    return _lib


def _split(shape, axis):
    """(outer, n, inner) of `shape` around `axis` (negative axis allowed)."""
    nd = len(shape)
    if axis < 0:
        axis += nd
    if not 0 <= axis < nd:
        raise ValueError("axis out of range")
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return outer, int(shape[axis]), inner, axis


def _canon(x):
    """-> (contiguous array of float32 or uint16 bits, is_half)."""
    x = np.asarray(x)
    if x.dtype == np.float32:
        return np.ascontiguousarray(x), False
    if x.dtype == np.float16:
        return np.ascontiguousarray(x).view(np.uint16), True
    if x.dtype == np.uint16:
        return np.ascontiguousarray(x), True
    raise TypeError("oracle takes float32, float16 or uint16 (half bits), got %s" % x.dtype)


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def half_to_float(h):
    h = np.asarray(h, dtype=np.uint16)
    f = lib().vkop_oracle_half_to_float
    return np.array([f(int(v)) for v in h.ravel()], dtype=np.float32).reshape(h.shape)


def float_to_half(x):
    x = np.asarray(x, dtype=np.float32)
    f = lib().vkop_oracle_float_to_half
    return np.array([f(float(v)) for v in x.ravel()], dtype=np.uint16).reshape(x.shape)


def softmax(x, axis=-1, nan_where=0, nan_value=0.0):
    a, half = _canon(x)
    if a.ndim == 0:
        raise ValueError("rank-0 input")
    outer, n, inner, _ = _split(a.shape, axis)
    out = np.empty_like(a)
    fn = lib().vkop_oracle_softmax_f16 if half else lib().vkop_oracle_softmax_f32
    fn(_ptr(a), _ptr(out), outer, n, inner, int(nan_where), float(nan_value))
    return out.view(np.float16) if half else out


def topk(x, k, axis=-1, largest=True):
    """-> (values, int32 indices), shape = x.shape with [axis] = k."""
    a, half = _canon(x)
    outer, n, inner, ax = _split(a.shape, axis)
    if not 0 <= k <= n:
        raise ValueError("k out of range")
    oshape = list(a.shape)
    oshape[ax] = k
    vals = np.empty(oshape, dtype=a.dtype)
    idx = np.empty(oshape, dtype=np.int32)
    fn = lib().vkop_oracle_topk_f16 if half else lib().vkop_oracle_topk_f32
    fn(_ptr(a), _ptr(vals), _ptr(idx), outer, n, inner, int(k), int(bool(largest)))
    return (vals.view(np.float16) if half else vals), idx


def softmax_topk(x, k, axis=-1, largest=True, return_probs=False):
    a, half = _canon(x)
    outer, n, inner, ax = _split(a.shape, axis)
    if not 0 <= k <= n:
        raise ValueError("k out of range")
    oshape = list(a.shape)
    oshape[ax] = k
    vals = np.empty(oshape, dtype=a.dtype)
    idx = np.empty(oshape, dtype=np.int32)
    probs = np.empty_like(a) if return_probs else None
    fn = lib().vkop_oracle_softmax_topk_f16 if half else lib().vkop_oracle_softmax_topk_f32
    fn(_ptr(a), _ptr(probs), _ptr(vals), _ptr(idx), outer, n, inner, int(k), int(bool(largest)))
    if half:
        vals = vals.view(np.float16)
        probs = probs.view(np.float16) if probs is not None else None
    return (vals, idx, probs) if return_probs else (vals, idx)


def softmax_topk_sampling(x, k, scale=1.0, top_p=None, axis=-1):
    """Fused softmax -> top-k of fl32(x * scale); with top_p also the nucleus counts.
    -> (values, indices) or (values, indices, counts)."""
    a, half = _canon(x)
    outer, n, inner, ax = _split(a.shape, axis)
    if not 0 <= k <= n:
        raise ValueError("k out of range")
    oshape = list(a.shape)
    oshape[ax] = k
    vals = np.empty(oshape, dtype=a.dtype)
    idx = np.empty(oshape, dtype=np.int32)
    cshape = list(a.shape)
    del cshape[ax]
    counts = np.empty(cshape, dtype=np.int32) if top_p is not None else None
    fn = lib().vkop_oracle_softmax_topk_sampling_f16 if half else lib().vkop_oracle_softmax_topk_sampling_f32
    fn(_ptr(a), float(np.float32(scale)), float(np.float32(top_p if top_p is not None else 0.0)), _ptr(vals), _ptr(idx),
       _ptr(counts), outer, n, inner, int(k))
    if half:
        vals = vals.view(np.float16)
    return (vals, idx, counts) if top_p is not None else (vals, idx)


def softmax_topk_mt(x, k, axis=-1, largest=True, threads=0):
    """Multi-threaded float32 fused oracle, for CPU-baseline timing.
    -> (values, indices, threads_used)."""
    a, half = _canon(x)
    if half:
        raise TypeError("float32 only")
    outer, n, inner, ax = _split(a.shape, axis)
    oshape = list(a.shape)
    oshape[ax] = k
    vals = np.empty(oshape, dtype=np.float32)
    idx = np.empty(oshape, dtype=np.int32)
    used = lib().vkop_oracle_softmax_topk_f32_mt(_ptr(a), _ptr(vals), _ptr(idx), outer, n, inner, int(k),
                                                 int(bool(largest)), int(threads))
    return vals, idx, used


def reduce_max(x, axis):
    a, half = _canon(x)
    if half:
        raise TypeError("float32 only")
    outer, n, inner, ax = _split(a.shape, axis)
    oshape = list(a.shape)
    del oshape[ax]
    out = np.empty(oshape, dtype=np.float32)
    lib().vkop_oracle_reduce_max_f32(_ptr(a), _ptr(out), outer, n, inner)
    return out


def get_top_k_predictions(logits, k):
    """core/function.cpp:150-183 restated -> list of (index, probability)."""
    a = np.ascontiguousarray(np.asarray(logits, dtype=np.float32).ravel())
    kk = min(int(k), a.size)
    idx = np.empty(max(kk, 1), dtype=np.int32)
    p = np.empty(max(kk, 1), dtype=np.float32)
    got = lib().vkop_oracle_get_top_k_predictions(_ptr(a), a.size, int(k), _ptr(idx), _ptr(p))
    return [(int(idx[j]), float(p[j])) for j in range(got)]


def nms(boxes, scores, iou_threshold, score_threshold, max_output_boxes_per_class=0, center_point_box=0,
        max_candidates=None):
    """Non-maximum suppression per (batch, class): boxes [B,N,4], scores [B,C,N] (float32).
    Returns an int32 array [M,3] of (batch, class, box index) records, ordered by
    batch, class, then selection order."""
    boxes = np.ascontiguousarray(boxes, dtype=np.float32)
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    B, N, four = boxes.shape
    assert four == 4 and scores.shape[0] == B and scores.shape[2] == N
    C = scores.shape[1]
    cap = B * C * N
    out = np.empty((max(cap, 1), 3), dtype=np.int32)
    m = lib().vkop_oracle_nms_f32(_ptr(boxes), _ptr(scores), _ptr(out), cap, B, C, N, int(center_point_box),
                                  int(max_output_boxes_per_class), float(iou_threshold), float(score_threshold),
                                  int(N if max_candidates is None else max_candidates))
    return out[:m].copy()


def topp_count(values, p):
    """Nucleus cut on sorted top-k probabilities [.., k] (float32, or float16 widened): per row the smallest
    count of leading values whose float sum, front to back, reaches p; k when it never does."""
    v = np.ascontiguousarray(np.asarray(values).astype(np.float32))
    k = v.shape[-1]
    rows = v.size // k if k else 0
    out = np.empty(v.shape[:-1], dtype=np.int32)
    lib().vkop_oracle_topp_count_f32(_ptr(v), rows, k, k, float(p), _ptr(out))
    return out
