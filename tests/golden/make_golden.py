"""Freezes libtorch-CPU expectations for the softmax / top-k path into a fixture.

The reference's tests compute every expectation at run time from libtorch 2.10.0
(tests/CMakeLists.txt:63) with fixed seeds -- torch::manual_seed(42) +
torch::randn + torch::softmax in tests/SoftmaxTest.cpp:118-138, and
torch::manual_seed(56) + torch::randn + torch::topk(input,k,axis,true,true) in
tests/TopkTest.cpp:71-75 -- and hold no stored vectors.  This script replays
exactly those calls through the same library (the torch 2.10.0 wheel installed
in this image; no file of the reference is imported or executed) and stores
inputs and outputs, so the tests need neither torch nor the seeds' RNG.

It also stores libtorch results on down-sized versions of the five benchmark
workloads (inputs from vkop_amd.synth).

Run from the repository root:  python tests/golden/make_golden.py
Writes tests/golden/libtorch_2_10_0.npz  (plain arrays, loadable with
numpy.load(allow_pickle=False)).
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from vkop_amd import synth  # noqa: E402

SOFTMAX_CASES = [  # tests/SoftmaxTest.cpp:195-202
    ((1, 10, 7, 7), 1),
    ((1, 6, 8, 8), 3),
    ((2, 4, 10, 10), 2),
    ((1, 8, 6, 6), 2),
    ((1, 16, 5, 5), 1),
    ((4, 1000), 1),
]
TOPK_CASES = [  # tests/TopkTest.cpp:93-99
    ((1, 200), 7, -1),
    ((1, 400), 8, -1),
    ((1, 600), 7, -1),
    ((3, 2000), 7, -1),
    ((1, 2000), 6, -1),
]


def bits(t):
    """torch tensor -> numpy array; halves as uint16 bit patterns."""
    a = t.contiguous().numpy()
    return a.view(np.uint16) if a.dtype == np.float16 else a


def main():
    assert torch.__version__.startswith("2.10.0"), torch.__version__
    out = {}
    for i, (shape, axis) in enumerate(SOFTMAX_CASES):
        for tag, dt in (("f32", torch.float32), ("f16", torch.float16)):
            torch.manual_seed(42)
            x = torch.randn(*shape, dtype=dt)
            y = torch.softmax(x, axis)
            out["softmax%d_%s_in" % (i, tag)] = bits(x)
            out["softmax%d_%s_out" % (i, tag)] = bits(y)
        out["softmax%d_axis" % i] = np.int32(axis)
    for i, (shape, k, axis) in enumerate(TOPK_CASES):
        for tag, dt in (("f32", torch.float32), ("f16", torch.float16)):
            torch.manual_seed(56)
            x = torch.randn(*shape, dtype=dt)
            v, ix = torch.topk(x, k, axis, True, True)
            out["topk%d_%s_in" % (i, tag)] = bits(x)
            out["topk%d_%s_val" % (i, tag)] = bits(v)
            out["topk%d_%s_idx" % (i, tag)] = ix.to(torch.int32).numpy()
        out["topk%d_k" % i] = np.int32(k)
        out["topk%d_axis" % i] = np.int32(axis)

    # down-sized benchmark workloads -------------------------------------
    def fused(x, k, name, keep_probs=True):
        t = torch.from_numpy(x)
        p = torch.softmax(t, -1)
        v, ix = torch.topk(p, k, -1, True, True)
        out[name + "_in"] = x
        out[name + "_k"] = np.int32(k)
        if keep_probs:
            out[name + "_prob"] = bits(p)
        out[name + "_val"] = bits(v)
        out[name + "_idx"] = ix.to(torch.int32).numpy()

    fused(synth.classifier_logits(1, 1000, synth.SEEDS["C1"]), 5, "c1")
    x2 = synth.classifier_logits(8, 1000, synth.SEEDS["C2"])
    fused(x2, 5, "c2")
    fused(x2.astype(np.float16), 5, "c2h")
    fused(synth.llm_logits(2, 8016, synth.SEEDS["C3"]), 50, "c3", keep_probs=False)
    # C4: tie heavy -- libtorch's tie order is implementation defined, only the
    # values are comparable
    x4 = synth.grid_values(2, 8192, synth.SEEDS["C4"])
    v4, _ = torch.topk(torch.from_numpy(x4), 256, -1, True, True)
    out["c4_in"] = x4
    out["c4_k"] = np.int32(256)
    out["c4_val"] = v4.numpy()
    # C5: softmax over axis 1, per-anchor class max, top-k along the anchors
    x5 = synth.detection_scores(2, 80, 200, synth.SEEDS["C5"])
    p5 = torch.softmax(torch.from_numpy(x5), 1)
    m5 = p5.amax(1)
    v5, i5 = torch.topk(m5, 30, -1, True, True)
    out["c5_in"] = x5
    out["c5_k"] = np.int32(30)
    out["c5_max"] = m5.numpy()
    out["c5_val"] = v5.numpy()
    out["c5_idx"] = i5.to(torch.int32).numpy()

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libtorch_2_10_0.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
