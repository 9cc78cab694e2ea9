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
    bias dtype (reference: kernels/linear.py:819-853).  An fp16 / bf16 bias is widened to fp32 inside the
    kernel (no conversion launch)."""
    if dtype is None:
        dtype = out.dtype if out is not None else bias.dtype
    if bias is not None and bias.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        bias = bias.to(torch.float32)
    return _linear(a, b, epilogue=L.EPI_SCALE_F, out_dtype=dtype, bias=bias, alpha=scale_a, beta=scale_b, out=out,
                   config=_config)


def linear_a8_w8_bfp32_ofp32_residual(a, b, bias, scale_a, scale_b, residual, out=None):
    """`linear_a8_w8_bfp32_ofp32(a, b, bias, scale_a, scale_b) + residual` in fp32 as one library call
    (reference: kernels/linear.py:819-853 followed by the caller's add): with 16 or fewer rows the
    decode kernel adds the residual while it stores, the persistent kernels that serve large outputs add it in
    their epilogue, otherwise an add kernel follows the GEMM.
    `out` must not overlap `residual`."""
    L.require_cuda(a, b, bias, residual, out)
    assert a.dtype == torch.int8 and b.dtype == torch.int8, "operands must be int8"
    assert len(b.shape) == 2 and a.shape[-1] == b.shape[1], "Incompatible dimensions"
    N, K = b.shape
    lead = a.shape[:-1]
    a2 = a.reshape(-1, K)
    M = a2.shape[0]
    assert residual.dtype == torch.float32 and residual.numel() == M * N, "residual must be fp32 [*, N]"
    r2 = residual.reshape(M, N)
    if a2.stride(1) != 1:
        a2 = a2.contiguous()
    if r2.stride(1) != 1:
        r2 = r2.contiguous()
    if b.stride(1) != 1:
        b = b.contiguous()
    if bias is not None:
        assert bias.numel() == N
        bias = bias.to(torch.float32).contiguous()
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    else:
        assert out.dtype == torch.float32 and out.numel() == M * N and out.is_contiguous()
    o2 = out.view(M, N)
    dev = a.device
    alpha, beta = L.scale_tensor(scale_a, dev), L.scale_tensor(scale_b, dev)
    with L.on_device(dev):
        rc = L.lib().ti_linear_i8_residual_f32(a2.data_ptr(), a2.stride(0) if M > 1 else K, b.data_ptr(), b.stride(0),
                                               L.ptr(bias), alpha.data_ptr(), beta.data_ptr(), r2.data_ptr(),
                                               r2.stride(0) if M > 1 else N, o2.data_ptr(), N, M, N, K,
                                               L.current_stream(dev))
    L.check(rc, "ti_linear_i8_residual_f32")
    return o2.view(*lead, N)


def linear_qkv_decode_a8_w8_b8_o8(a, w3, bias3, scale_a3, scale_b3, k_cache, vt_cache, out=None):
    """The q / k / v projections of a decode step (`linear_group_a8_w8_b8_o8` with 3 groups) with the
    KV-cache append folded into the same launch: a [S, K] int8 (S <= 16), w3 [3N, K], bias3 int8 [3N],
    scale_a3 / scale_b3 fp32 device tensors [3]; k_cache int8 [heads, T, D] and vt_cache int8
    [heads, D, T] (contiguous, N = heads * D) receive the S new positions in their last S slots.
    Returns the [S, 3N] int8 projections, or None when the shapes do not fit the decode kernel (the
    caller then uses `linear_group_a8_w8_b8_o8` and `kv_append_i8`)."""
    L.require_cuda(a, w3, bias3, scale_a3, scale_b3, k_cache, vt_cache, out)
    S, K = a.shape
    N = w3.shape[0] // 3
    heads, T, D = k_cache.shape
    if not (S <= 16 and K >= 1024 and heads * D == N and D % 16 == 0 and S <= T and tuple(vt_cache.shape) == (heads, D, T)
            and k_cache.is_contiguous() and vt_cache.is_contiguous() and a.stride(1) == 1 and w3.is_contiguous()):
        return None
    assert a.dtype == w3.dtype == bias3.dtype == k_cache.dtype == vt_cache.dtype == torch.int8
    assert w3.shape == (3 * N, K) and bias3.numel() == 3 * N
    for t in (scale_a3, scale_b3):
        assert t.dtype == torch.float32 and t.numel() == 3 and t.is_contiguous()
    if out is None:
        out = torch.empty((S, 3 * N), dtype=torch.int8, device=a.device)
    assert out.dtype == torch.int8 and tuple(out.shape) == (S, 3 * N) and out.is_contiguous()
    with L.on_device(a.device):
        rc = L.lib().ti_qkv_decode_i8(a.data_ptr(), a.stride(0) if S > 1 else K, w3.data_ptr(), K, bias3.data_ptr(),
                                      scale_a3.data_ptr(), scale_b3.data_ptr(), out.data_ptr(), 3 * N, S, N, K,
                                      k_cache.data_ptr() + (T - S) * D, T * D, vt_cache.data_ptr() + (T - S), T, D,
                                      L.current_stream(a.device))
    if rc == -3:  # TI_E_COMBO: operands not eligible for the decode kernel
        return None
    L.check(rc, "ti_qkv_decode_i8")
    return out
