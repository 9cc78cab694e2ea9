"""MI355X-native (gfx950) implementation of the INT8 hot path of zhanglei1172/triton_int.

Sub-modules keep the reference's layout and call signatures:

    triton_int_amd.kernels.linear / .bmm / .fused   launchers (reference: triton_int/kernels/*.py)
    triton_int_amd.functional.bmm / .fused / .quantization
    triton_int_amd.nn.linear / .bmm / .fused        torch.nn.Module wrappers

Every launcher enqueues hand-written HIP kernels from ``lib/libtriton_int_hip.so`` (C ABI in
``include/triton_int_hip.h``) on the current torch stream.  There is no Triton, no CPU fallback
and no other backend: without the built library, or on a device that is not gfx950, calls raise.
"""

__version__ = "0.1.0"
