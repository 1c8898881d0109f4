"""The C++ operator interface (vkop_amd/host): its own test program, built from
vkop_amd/host/tests/test_ops.cpp, replays the reference's SoftmaxTest / TopkTest
case lists (tests/SoftmaxTest.cpp:188-230, tests/TopkTest.cpp:93-127, tests/NmsTest.cpp:165-169)
with libtorch-generated expectations, reads the .vkopbin fixtures and runs models from them.  Here it is only launched and its verdict read."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "vkop_amd", "host")
BIN = os.path.join(HOST, "build", "test_ops")


def _binary():
    if not os.path.exists(BIN):
        subprocess.check_call(["make", "-C", HOST])
    return BIN


def _run(args):
    r = subprocess.run([_binary()] + args, cwd=HOST, capture_output=True, text=True, timeout=300)
    print(r.stdout[-4000:])
    print(r.stderr[-2000:])
    return r


def test_host_logic_without_gpu():
    """Names and numbering, factory, attribute parsing, tensors, binary16 conversions, the model file reader."""
    r = _run(["--no-gpu"])
    assert r.returncode == 0
    assert " 0 failed" in r.stdout


@pytest.mark.gpu
def test_reference_case_lists_through_operator_interface():
    r = _run([])
    assert r.returncode == 0
    assert " 0 failed" in r.stdout
    for needle in ("Softmax fp32 shape [4,1000,] axis 1: ok", "TopK fp16 shape [3,2000] k 7 axis -1: ok",
                   "Softmax+TopK fp32 shape [4,128256] k 50: ok", "Runtime post-proc [64,128256] k 50, fused: ok",
                   "(not fusable): ok", "Nms fp32 boxes [1,50,4] classes 7: ok", "Nms fp16 boxes [2,300,4] classes 3: ok",
                   "Model classifier_head.vkopbin fp32 [8,1000] k 5, 1 operator(s) (node_topk): ok",
                   "Model classifier_head_k_input.vkopbin fp16 [4,1000] k 7, 2 operator(s) (node_topk): ok",
                   "Model detection_tail.vkopbin: ok", "Reduce max fp32 shape [16,80,8400] axis 1 keepdims 0: ok",
                   "Reduce max fp16 shape [4,80,1000] axis -2 keepdims 0: ok", "Model detection_chain.vkopbin, 2 operator(s): ok",
                   "Model detection_chain.vkopbin, 3 operator(s): ok", "Model two_heads.vkopbin, 3 operators in 2 levels: ok"):
        assert needle in r.stdout
