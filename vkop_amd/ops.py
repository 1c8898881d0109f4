"""Operator front-ends over torch device tensors.

torch is used for device memory and streams only; every computation goes
through the C ABI (vkop_amd.capi).  Inputs must be contiguous CUDA/HIP tensors
of float32 or float16; results are new tensors on the same device, enqueued on
torch's current stream.
"""
import torch

from . import capi

_DTYPES = {torch.float32: capi.F32, torch.float16: capi.F16}


def _prep(x):
    if not isinstance(x, torch.Tensor) or not x.is_cuda:
        raise TypeError("expected a tensor on the GPU (there is no CPU path)")
    if x.dtype not in _DTYPES:
        raise TypeError("float32 or float16 expected, got %s" % x.dtype)
    if x.dim() < 1 or x.dim() > 4:
        raise ValueError("rank %d outside 1..4" % x.dim())
    return x.contiguous(), _DTYPES[x.dtype]


def _stream():
    return torch.cuda.current_stream().cuda_stream


class Workspace:
    """Scratch device memory an operator keeps between calls, like the
    ping-pong temporaries the reference's Topk owns (ops/Topk.hpp:46-55,221-224).
    Cleared once when (re)allocated; calls leave it ready for the next call.
    One workspace serves one stream at a time."""

    def __init__(self):
        self.buf = None

    def get(self, nbytes):
        nbytes = int(nbytes)
        if nbytes == 0:
            return 0, 0
        if self.buf is None or self.buf.numel() < nbytes:
            self.buf = torch.empty(nbytes + 256, dtype=torch.uint8, device="cuda")
            self._off = (-self.buf.data_ptr()) % 256
            self._size = (self.buf.numel() - self._off) // 4 * 4
            capi.workspace_init(self.buf.data_ptr() + self._off, self._size, _stream())
        return self.buf.data_ptr() + self._off, self._size


_default_ws = Workspace()


def softmax(x, axis=-1, nan_where=False, nan_value=0.0, out=None, workspace=None):
    """ops/Softmax.hpp:61-141 -- same shape and dtype as x."""
    x, dt = _prep(x)
    if out is None:
        out = torch.empty_like(x)
    ws = workspace or _default_ws
    ptr, size = ws.get(capi.softmax_workspace_bytes(dt, x.shape, axis))
    capi.softmax(x.data_ptr(), out.data_ptr(), dt, x.shape, axis, int(bool(nan_where)), nan_value, ptr, size, _stream())
    return out


def _out_shape(x, axis, k):
    shape = list(x.shape)
    shape[axis if axis >= 0 else axis + x.dim()] = int(k)
    return shape


def topk(x, k, axis=-1, largest=True, sorted=True, workspace=None):
    """ops/Topk.hpp:95-218 -- (values like x, int32 indices), [axis] = k."""
    x, dt = _prep(x)
    shape = _out_shape(x, axis, k)
    values = torch.empty(shape, dtype=x.dtype, device=x.device)
    indices = torch.empty(shape, dtype=torch.int32, device=x.device)
    ws = workspace or _default_ws
    ptr, size = ws.get(capi.topk_workspace_bytes(dt, x.shape, axis, k))
    capi.topk(x.data_ptr(), values.data_ptr(), indices.data_ptr(), dt, x.shape, axis, k, int(bool(largest)),
              int(bool(sorted)), ptr, size, _stream())
    return values, indices


def softmax_topk(x, k, axis=-1, largest=True, return_probs=False, workspace=None):
    """The registered post-proc pair of benchmark/main.cpp:85-101 in one call:
    top-k of softmax(x) along `axis`, without materialising the softmax tensor
    unless return_probs is set."""
    x, dt = _prep(x)
    shape = _out_shape(x, axis, k)
    values = torch.empty(shape, dtype=x.dtype, device=x.device)
    indices = torch.empty(shape, dtype=torch.int32, device=x.device)
    probs = torch.empty_like(x) if return_probs else None
    ws = workspace or _default_ws
    ptr, size = ws.get(capi.softmax_topk_workspace_bytes(dt, x.shape, axis, k))
    capi.softmax_topk(x.data_ptr(), probs.data_ptr() if return_probs else 0, values.data_ptr(), indices.data_ptr(),
                      dt, x.shape, axis, k, int(bool(largest)), ptr, size, _stream())
    return (values, indices, probs) if return_probs else (values, indices)


def softmax_topk_sampling(x, k, scale=1.0, top_p=None, axis=-1, workspace=None):
    """Sampling-style fused call: top-k of softmax(fl32(x * scale)); with top_p also the nucleus count per row.
    -> (values, indices) or (values, indices, counts)."""
    x, dt = _prep(x)
    shape = _out_shape(x, axis, k)
    values = torch.empty(shape, dtype=x.dtype, device=x.device)
    indices = torch.empty(shape, dtype=torch.int32, device=x.device)
    cshape = list(x.shape)
    del cshape[axis if axis >= 0 else axis + x.dim()]
    counts = torch.empty(cshape, dtype=torch.int32, device=x.device) if top_p is not None else None
    ws = workspace or _default_ws
    ptr, size = ws.get(capi.softmax_topk_workspace_bytes(dt, x.shape, axis, k))
    capi.softmax_topk_sampling(x.data_ptr(), values.data_ptr(), indices.data_ptr(), counts.data_ptr() if counts is not None else 0,
                               dt, x.shape, axis, k, scale, top_p if top_p is not None else 0.0, ptr, size, _stream())
    return (values, indices, counts) if top_p is not None else (values, indices)


def softmax_reduce_max(x, axis, workspace=None):
    """max over `axis` of softmax along `axis`, in one read (bit-equal to reduce_max(softmax(x, axis), axis))."""
    x, dt = _prep(x)
    shape = list(x.shape)
    del shape[axis if axis >= 0 else axis + x.dim()]
    out = torch.empty(shape, dtype=x.dtype, device=x.device)
    ws = workspace or _default_ws
    ptr, size = ws.get(capi.softmax_reduce_max_workspace_bytes(dt, x.shape, axis))
    capi.softmax_reduce_max(x.data_ptr(), out.data_ptr(), dt, x.shape, axis, ptr, size, _stream())
    return out


def reduce_max(x, axis):
    x, dt = _prep(x)
    shape = list(x.shape)
    del shape[axis if axis >= 0 else axis + x.dim()]
    out = torch.empty(shape, dtype=x.dtype, device=x.device)
    capi.reduce_max(x.data_ptr(), out.data_ptr(), dt, x.shape, axis, _stream())
    return out


def topp_count(values, p):
    """Nucleus cut on sorted top-k probabilities [.., k]: per row the smallest count of leading values whose float
    sum, taken front to back, reaches p (k when it never does).  -> int32 tensor of the leading shape."""
    values, dt = _prep(values)
    k = values.shape[-1]
    rows = values.numel() // k if k else 0
    counts = torch.empty(values.shape[:-1], dtype=torch.int32, device=values.device)
    capi.topp_count(values.data_ptr(), counts.data_ptr(), dt, rows, k, k, p, _stream())
    return counts


def nms(boxes, scores, iou_threshold, score_threshold, max_output_boxes_per_class=0, center_point_box=0,
        out_capacity=None, workspace=None):
    """Non-maximum suppression per (batch, class): boxes [B,N,4], scores [B,C,N] (both float32 or both float16).
    Returns (records, overflow): an int32 tensor [M,3] of (batch, class, box index), ordered by batch, class and
    selection, and whether some pair had more candidates than the kernel holds."""
    boxes, dt = _prep(boxes)
    scores, dt2 = _prep(scores)
    assert dt == dt2 and boxes.dim() == 3 and scores.dim() == 3 and boxes.shape[2] == 4
    B, N, _ = boxes.shape
    C = scores.shape[1]
    assert scores.shape[0] == B and scores.shape[2] == N
    per_pair = min(N, 2048) if max_output_boxes_per_class <= 0 else min(N, 2048, max_output_boxes_per_class)
    cap = B * C * per_pair if out_capacity is None else out_capacity
    out = torch.empty((max(cap, 1), 3), dtype=torch.int32, device=boxes.device)
    count = torch.zeros(2, dtype=torch.int32, device=boxes.device)
    ws = workspace or _default_ws
    ptr, size = ws.get(capi.nms_workspace_bytes(B, C, N, max_output_boxes_per_class))
    capi.nms(boxes.data_ptr(), scores.data_ptr(), out.data_ptr(), cap, count.data_ptr(), dt, B, C, N, center_point_box,
             max_output_boxes_per_class, iou_threshold, score_threshold, ptr, size, _stream())
    m, over = (int(v) for v in count.cpu().tolist())
    return out[:min(m, cap)], bool(over)
