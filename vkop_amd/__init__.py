"""MI355X-native softmax / top-k logits post-processing (HIP, gfx950).

The product is the C-ABI library built from vkop_amd/csrc (declared in
include/vkop_hip.h) and the C++ operator layer in vkop_amd/host that mirrors the
reference's Operator / create_from_type / Tensor interface.  This Python
package is plumbing around them: a ctypes binding (vkop_amd.capi), thin
operator front-ends over torch device tensors (vkop_amd.ops) and the synthetic
workload generators (vkop_amd.synth).
"""
__all__ = ["capi", "ops", "synth"]
