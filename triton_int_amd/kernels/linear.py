"""int8 linear launchers — same names and arguments as triton_int/kernels/linear.py.

a: [..., K] int8 (viewed as [M, K]); b: [N, K] int8 weight; scales: 0-dim fp32 device tensors
(python floats are accepted and uploaded once).  int8 outputs are
clamp(round_half_even(.), -128, 127); ``_round_mode=1`` selects the literal Triton truncation
for comparison runs.
"""
from __future__ import annotations

import torch

from .. import _lib as L
from ._gemm import linear as _linear
from ._gemm import linear_group as _linear_group


def linear_a8_w8_ofp32(a, b, scale, out=None, dtype=torch.float, *, _config=-1):
    """scale * acc -> fp (reference: kernels/linear.py:117-147)."""
    return _linear(a, b, epilogue=L.EPI_SCALE_F, out_dtype=dtype, alpha=scale, out=out, config=_config)


def linear_a8_w8_b8_o8(a, b, bias, scale_a, scale_b, out=None, *, _round_mode=L.ROUND_RNE_CLAMP, _config=-1):
    """q8(scale_a * acc + scale_b * bias_i8) (reference: kernels/linear.py:256-288)."""
    return _linear(a, b, epilogue=L.EPI_SCALE_I8, out_dtype=torch.int8, bias=bias, alpha=scale_a, beta=scale_b,
                   out=out, round_mode=_round_mode, config=_config)


def linear_group_a8_w8_b8_o8(a, b, bias, scale_a, scale_b, groups, out=None, *, _config=-1):
    """`groups` linear_a8_w8_b8_o8 projections of one input as a single launch (the q/k/v
    projections of an attention block: three W8A8B8O8Linear, nn/linear.py:18-67, which the
    reference launches one after the other).  b: the [N,K] weights stacked to [groups*N, K];
    bias int8 [groups*N]; scale_a, scale_b: fp32 device tensors [groups].  Returns
    [..., groups*N] int8, projection g in columns g*N .. g*N+N, each element exactly what
    linear_a8_w8_b8_o8 gives for that projection."""
    return _linear_group(a, b, groups, epilogue=L.EPI_SCALE_I8, out_dtype=torch.int8, bias=bias, alpha=scale_a,
                         beta=scale_b, out=out, config=_config)


def linear_relu_a8_w8_b8_o8(a, b, bias, scale_a, scale_b, out=None, *, _round_mode=L.ROUND_RNE_CLAMP, _config=-1):
    """max(q8(...), 0) (reference: kernels/linear.py:398-430)."""
    return _linear(a, b, epilogue=L.EPI_SCALE_RELU_I8, out_dtype=torch.int8, bias=bias, alpha=scale_a,
                   beta=scale_b, out=out, round_mode=_round_mode, config=_config)


def linear_a8_w8_b32_o32(a, b, bias, out=None, *, _config=-1):
    """acc + bias_i32, bit-exact int32 (reference: kernels/linear.py:536-566)."""
    return _linear(a, b, epilogue=L.EPI_I32, out_dtype=torch.int32, bias=bias, out=out, config=_config)


def linear_a8_w8_b32_o32_with_scaling(a, b, bias, scale_a, scale_b, out=None, *, _round_mode=L.ROUND_TRUNC,
                                      _config=-1):
    """int32(scale_a * acc + scale_b * bias_i32); the fp32->int32 conversion truncates toward
    zero as the reference's `.to(tl.int32)` does (reference: kernels/linear.py:676-708)."""
    return _linear(a, b, epilogue=L.EPI_SCALE_I32, out_dtype=torch.int32, bias=bias, alpha=scale_a, beta=scale_b,
                   out=out, round_mode=_round_mode, config=_config)


def linear_a8_w8_bfp32_ofp32(a, b, bias, scale_a, scale_b, out=None, dtype=None, *, _config=-1):
    """scale_a * acc + scale_b * bias -> fp32 / fp16 / bf16; the output dtype defaults to the
    bias dtype (reference: kernels/linear.py:819-853).  The bias is read as fp32."""
    if dtype is None:
        dtype = out.dtype if out is not None else bias.dtype
    if bias is not None and bias.dtype != torch.float32:
        bias = bias.to(torch.float32)
    return _linear(a, b, epilogue=L.EPI_SCALE_F, out_dtype=dtype, bias=bias, alpha=scale_a, beta=scale_b, out=out,
                   config=_config)
