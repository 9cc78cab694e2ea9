"""Dequant + residual add + LayerNorm (+ quantise) (reference: triton_int/functional/fused.py).

The reference ships only a PyTorch emulation (`dq_add_layernorm_q_py`, :6-15) and a stub that
calls an op it never imports (`dq_add_layernorm_q_cpp`, :27-32).  Here all three names run the
fused HIP kernel; the argument order and the returned pair are the reference's.
"""
from ..kernels.fused import dq_add_layernorm_q as _native


def dq_add_layernorm_q(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps):
    """-> (residual_output_fp32, ln_output_int8)"""
    return _native(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps, quantize=True)


def dq_add_layernorm_q_py(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps):
    return dq_add_layernorm_q(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps)


def dq_add_layernorm_q_cpp(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps):
    return dq_add_layernorm_q(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps)


def dq_add_layernorm(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps):
    """-> (residual_output_fp32, ln_output_fp32) (reference: functional/fused.py:18-24)"""
    return _native(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps, quantize=False)
