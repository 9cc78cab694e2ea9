"""Fused launchers — the entries of triton_int/kernels/fused.py (the int8 ones and the
floating-point LayerNorm / skip-LayerNorm trio) plus the two ops that file only sketches: the dequant + residual-add + LayerNorm + quantise kernel (its Triton stub at
kernels/fused.py:17-61 is never launched) and a launchable stand-alone GELU-quant
(fast_geluQ, kernels/fused.py:76-79, is a device function there).
"""
from __future__ import annotations

import torch

from .. import _lib as L
from ._gemm import linear as _linear


def linear_a8_w8_bfp32_ofp32_GeLu_Q(a, b, bias, scale_a, scale_b, out=None, *, _round_mode=L.ROUND_RNE_CLAMP,
                                    _config=-1):
    """x = scale_a * acc + bias_f32;  q8(gelu_tanh(x) * scale_b)   (reference: kernels/fused.py:197-231;
    scale_b is 1/output_scale, nn/fused.py:148-150)."""
    if bias is not None and bias.dtype != torch.float32:
        bias = bias.to(torch.float32)
    return _linear(a, b, epilogue=L.EPI_GELU_I8, out_dtype=torch.int8, bias=bias, alpha=scale_a, beta=scale_b,
                   out=out, round_mode=_round_mode, config=_config)


def layer_norm_fwd_fused_single_pass_q(x, weight, bias, eps, use_rms_norm=False, *, _round_mode=L.ROUND_RNE_CLAMP,
                                       _return_stats=False):
    """LayerNorm (or RMSNorm) over the last dim, output quantised to int8
    (reference: kernels/fused.py:336-382)."""
    assert x.dtype == weight.dtype, f"input and weight bias must have the same dtype: {x.dtype}, {weight.dtype}"
    if bias is not None:
        assert x.dtype == bias.dtype, f"input and bias must have the same dtype: {x.dtype}, {bias.dtype}"
    assert x.dtype == torch.float32, "the int8 LayerNorm kernel takes fp32 activations (nn/fused.py:43)"
    L.require_cuda(x, weight, bias)
    N = x.shape[-1]
    assert weight.numel() == N and (bias is None or bias.numel() == N)
    a_arg = x.view(-1, N)
    if a_arg.stride(1) != 1:
        a_arg = a_arg.contiguous()
    out = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    o2 = out.view(-1, N)
    M = a_arg.shape[0]
    weight = weight.contiguous()
    bias = None if bias is None else bias.contiguous()
    mean = rstd = None
    if _return_stats:
        mean = torch.empty(M, dtype=torch.float32, device=x.device)
        rstd = torch.empty(M, dtype=torch.float32, device=x.device)
    with L.on_device(x.device):
        rc = L.lib().ti_layernorm_q(L.ptr(a_arg), a_arg.stride(0) if M > 1 else N, L.ptr(weight), L.ptr(bias),
                                    float(eps), L.ptr(o2), N, M, N, int(bool(use_rms_norm)), int(_round_mode),
                                    L.ptr(mean), L.ptr(rstd), L.current_stream(x.device))
    L.check(rc, "ti_layernorm_q")
    return (out, mean, rstd) if _return_stats else out


def _layernorm_fp(x, skip, weight, bias, eps, use_rms_norm, want_out, want_skip_out):
    assert x.dtype == weight.dtype, f"input and weight bias must have the same dtype: {x.dtype}, {weight.dtype}"
    if bias is not None:
        assert x.dtype == bias.dtype, f"input and bias must have the same dtype: {x.dtype}, {bias.dtype}"
    assert x.dtype in (torch.float32, torch.float16, torch.bfloat16), f"floating-point LayerNorm takes fp32 / fp16 / bf16, got {x.dtype}"
    L.require_cuda(x, weight, bias, skip)
    # catch eps being too small if the tensors are fp16 (kernels/fused.py:501-503)
    if x.dtype == torch.float16:
        eps = max(eps, 1.6e-5)
    N = x.shape[-1]
    assert weight.numel() == N and (bias is None or bias.numel() == N)
    a_arg = x.view(-1, N)
    if a_arg.stride(1) != 1:
        a_arg = a_arg.contiguous()
    M = a_arg.shape[0]
    b_arg = None
    if skip is not None:
        assert skip.dtype == x.dtype and skip.numel() == x.numel(), "skip must match the input"
        b_arg = skip.view(-1, skip.shape[-1])
        assert tuple(b_arg.shape) == (M, N), "skip must match the input"
        if b_arg.stride(1) != 1:
            b_arg = b_arg.contiguous()
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device) if want_out else None
    skip_out = torch.empty(x.shape, dtype=x.dtype, device=x.device) if want_skip_out else None
    weight = weight.contiguous()
    bias = None if bias is None else bias.contiguous()
    with L.on_device(x.device):
        rc = L.lib().ti_layernorm_fp(L.ptr(a_arg), a_arg.stride(0) if M > 1 else N,
                                     L.ptr(b_arg), (b_arg.stride(0) if M > 1 else N) if b_arg is not None else 0,
                                     L.TORCH_TO_DT[x.dtype], L.ptr(weight), L.ptr(bias), float(eps),
                                     int(bool(use_rms_norm)), L.ptr(out), N, L.ptr(skip_out), N, M, N,
                                     L.current_stream(x.device))
    L.check(rc, "ti_layernorm_fp")
    return out, skip_out


def layer_norm_fwd_fused_single_pass(x, weight, bias, eps, use_rms_norm=False):
    """LayerNorm (or RMSNorm) over the last dim, output in x's dtype (fp32 / fp16 / bf16)
    (reference: kernels/fused.py:486-532)."""
    return _layernorm_fp(x, None, weight, bias, eps, use_rms_norm, True, False)[0]


def skip_layer_norm_fwd_fused_single_pass(x, skip, weight, bias, eps, use_rms_norm=False):
    """LayerNorm(x) rounded to x's dtype, plus skip (reference: kernels/fused.py:644-693)."""
    return _layernorm_fp(x, skip, weight, bias, eps, use_rms_norm, False, True)[1]


def skip_layer_norm_fwd_fused_single_pass2(x, skip, weight, bias, eps, use_rms_norm=False):
    """(LayerNorm(x), LayerNorm(x) + skip), both in x's dtype (reference: kernels/fused.py:811-862)."""
    return _layernorm_fp(x, skip, weight, bias, eps, use_rms_norm, True, True)


def dq_add_layernorm_q(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps, *, quantize=True,
                       _round_mode=L.ROUND_RNE_CLAMP, _return_stats=False):
    """residual_out = residual_in + input_scale * int32;  LayerNorm;  -> (residual_out fp32,
    int8) — or the fp32 LayerNorm output when quantize=False.  Semantics of
    functional/fused.py:6-24; the argument order is that of the intended native op,
    functional/fused.py:27-32."""
    L.require_cuda(input_int32, residual_input_fp, gamma, beta)
    assert input_int32.dtype == torch.int32, "input_int32 must be int32"
    assert input_int32.shape == residual_input_fp.shape, "Incompatible dimensions"
    shape = input_int32.shape
    H = shape[-1]
    assert gamma.numel() == H and (beta is None or beta.numel() == H)
    acc = input_int32.reshape(-1, H)
    rin = residual_input_fp.to(torch.float32).reshape(-1, H)
    if acc.stride(1) != 1:
        acc = acc.contiguous()
    if rin.stride(1) != 1:
        rin = rin.contiguous()
    rows = acc.shape[0]
    dev = acc.device
    gamma = gamma.to(torch.float32).contiguous()
    beta = None if beta is None else beta.to(torch.float32).contiguous()
    rout = torch.empty((rows, H), dtype=torch.float32, device=dev)
    y = torch.empty((rows, H), dtype=torch.int8, device=dev) if quantize else None
    ln = None if quantize else torch.empty((rows, H), dtype=torch.float32, device=dev)
    mean = rstd = None
    if _return_stats:
        mean = torch.empty(rows, dtype=torch.float32, device=dev)
        rstd = torch.empty(rows, dtype=torch.float32, device=dev)
    # the module holds a python float (nn/fused.py:62); a tensor scale is read on the device, so that
    # the call neither synchronises nor breaks a graph capture
    scale_t = None
    if torch.is_tensor(input_scale_fp):
        scale_t = input_scale_fp if input_scale_fp.is_cuda else None
        if scale_t is None:
            input_scale_fp = float(input_scale_fp)
        else:
            scale_t = L.scale_tensor(scale_t.reshape(()), dev)
            input_scale_fp = 0.0
    with L.on_device(dev):
        rc = L.lib().ti_dq_add_layernorm_q(
            L.ptr(acc), acc.stride(0) if rows > 1 else H, float(input_scale_fp), L.ptr(scale_t), L.ptr(rin),
            rin.stride(0) if rows > 1 else H, L.ptr(gamma), L.ptr(beta), float(eps), L.ptr(rout), H, L.ptr(y), H,
            L.ptr(ln), H, rows, H, int(_round_mode), L.ptr(mean), L.ptr(rstd), L.current_stream(dev))
    L.check(rc, "ti_dq_add_layernorm_q")
    res = (rout.view(shape), (y if quantize else ln).view(shape))
    return res + (mean, rstd) if _return_stats else res


def gelu_q(x, scale, *, _round_mode=L.ROUND_RNE_CLAMP):
    """q8(gelu_tanh(x) * scale) element-wise, x fp32 -> int8 (math of kernels/fused.py:76-79)."""
    L.require_cuda(x)
    x = x.to(torch.float32).contiguous()
    y = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = L.scale_tensor(scale, x.device)
    with L.on_device(x.device):
        rc = L.lib().ti_gelu_q(L.ptr(x), L.ptr(s), L.ptr(y), x.numel(), int(_round_mode), L.current_stream(x.device))
    L.check(rc, "ti_gelu_q")
    return y


def softmax_q(x, scale, causal_q_len=0):
    """int8 attention scores [..., cols] -> int8 probabilities round(softmax(x * scale) * 127) in [0, 127].
    The reference has no kernel for this step (callers of its BMM modules do it in fp32 torch between
    bmm_s8t_s8n_s8t and the P.V BMM).  `scale` is a python float; causal_q_len > 0 masks position i of
    every group of causal_q_len rows to columns 0 .. i + (cols - causal_q_len)."""
    L.require_cuda(x)
    assert x.dtype == torch.int8, "scores must be int8"
    cols = x.shape[-1]
    x2 = x.reshape(-1, cols)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    y = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    y2 = y.view(-1, cols)
    with L.on_device(x.device):
        rc = L.lib().ti_softmax_q(L.ptr(x2), x2.stride(0) if rows > 1 else cols, float(scale), L.ptr(y2), cols, rows,
                                  cols, int(causal_q_len), L.current_stream(x.device))
    L.check(rc, "ti_softmax_q")
    return y


def transpose_i8(src, out=None):
    """int8 [rows, cols] (unit column stride) -> [cols, rows].  `out` may be any int8 view of that
    shape with unit column stride, e.g. the last `rows` columns of a V^T cache [heads*D, T].  The
    reference's callers do this step with torch (`transpose(...).contiguous()`)."""
    L.require_cuda(src, out)
    assert src.dtype == torch.int8 and src.dim() == 2 and src.stride(1) == 1, "src must be int8 [rows, cols], unit column stride"
    rows, cols = src.shape
    if out is None:
        out = torch.empty((cols, rows), dtype=torch.int8, device=src.device)
    assert out.dtype == torch.int8 and tuple(out.shape) == (cols, rows) and (out.stride(1) == 1 or rows == 1)
    with L.on_device(src.device):
        rc = L.lib().ti_transpose_i8(L.ptr(src), src.stride(0), L.ptr(out), out.stride(0), rows, cols,
                                     L.current_stream(src.device))
    L.check(rc, "ti_transpose_i8")
    return out


def attention_i8(q, k, vt, qk_alpha, score_scale, pv_alpha, causal_q_len=0, out=None):
    """bmm_s8t_s8n_s8t(q, k, qk_alpha) -> softmax_q(., score_scale, causal_q_len) ->
    bmm_s8t_s8n_s8t(probs, vt, pv_alpha) as one kernel that keeps scores and probabilities in
    registers (reference: the same three steps are separate launches, kernels/bmm.py:576-612 twice
    plus the caller's softmax).  q [BH,S,128], k [BH,T,128], vt [BH,128,T] int8 with unit stride
    along the last dimension; `out` may be any int8 [BH,S,128] view with unit last stride (e.g. the
    head-merged [S, heads, 128] layout).  Scalars are python floats."""
    L.require_cuda(q, k, vt, out)
    assert q.dtype == torch.int8 and k.dtype == torch.int8 and vt.dtype == torch.int8, "operands must be int8"
    assert q.dim() == 3 and k.dim() == 3 and vt.dim() == 3, "q, k, vt must be 3-D"
    BH, S, D = q.shape
    T = k.shape[1]
    assert k.shape == (BH, T, D) and vt.shape == (BH, D, T), "Incompatible dimensions"
    assert q.stride(2) == 1 and k.stride(2) == 1 and vt.stride(2) == 1, "unit stride along the last dimension"
    if out is None:
        out = torch.empty((BH, S, D), dtype=torch.int8, device=q.device)
    assert out.dtype == torch.int8 and tuple(out.shape) == (BH, S, D) and out.stride(2) == 1
    with L.on_device(q.device):
        rc = L.lib().ti_attention_i8(L.ptr(q), q.stride(0), q.stride(1), L.ptr(k), k.stride(0), k.stride(1),
                                     L.ptr(vt), vt.stride(0), vt.stride(1), L.ptr(out), out.stride(0), out.stride(1),
                                     BH, S, T, D, float(qk_alpha), float(score_scale), float(pv_alpha),
                                     int(causal_q_len), L.current_stream(q.device))
    L.check(rc, "ti_attention_i8")
    return out


def quantize_per_token_absmax(t):
    """Dynamic per-token quantisation of fp32 / fp16 activations [..., cols]: returns
    (q int8 [..., cols], max_val [..., 1] in t's dtype) with max_val = clamp(absmax, 1e-8) / 127
    and q = clamp(round(t / max_val), -128, 127), bit-identical to
    dynamic_quantize_activation_per_token_absmax (reference: functional/quantization.py:61-67).
    Unlike that helper it leaves `t` untouched."""
    L.require_cuda(t)
    assert t.dtype in (torch.float32, torch.float16), "activations must be fp32 or fp16"
    cols = t.shape[-1]
    x2 = t.reshape(-1, cols)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    q = torch.empty((rows, cols), dtype=torch.int8, device=t.device)
    scale = torch.empty((rows, 1), dtype=t.dtype, device=t.device)
    with L.on_device(t.device):
        rc = L.lib().ti_quantize_per_token_absmax(L.ptr(x2), L.TORCH_TO_DT[t.dtype], x2.stride(0), L.ptr(q), cols,
                                                  L.ptr(scale), rows, cols, L.current_stream(t.device))
    L.check(rc, "ti_quantize_per_token_absmax")
    return q.view(t.shape), scale.view(*t.shape[:-1], 1)


def kv_append_i8(k_new, v_new, k_cache, vt_cache):
    """Write S new positions into the last S slots of an int8 KV cache with one launch.
    k_new, v_new: int8 [S, heads*D] (unit column stride; e.g. column slices of a fused q/k/v
    projection); k_cache int8 [heads, T, D]; vt_cache int8 [heads, D, T].  Replaces
    `k_cache[:, T-S:, :] = k_new.view(S, heads, D).transpose(0, 1)` and the V transpose."""
    L.require_cuda(k_new, v_new, k_cache, vt_cache)
    heads, T, D = k_cache.shape
    S, H = k_new.shape
    assert H == heads * D and tuple(v_new.shape) == (S, H) and tuple(vt_cache.shape) == (heads, D, T) and S <= T
    assert k_new.dtype == v_new.dtype == k_cache.dtype == vt_cache.dtype == torch.int8
    assert k_new.stride(1) == 1 and v_new.stride(1) == 1 and k_cache.is_contiguous() and vt_cache.is_contiguous()
    with L.on_device(k_new.device):
        rc = L.lib().ti_kv_append_i8(L.ptr(k_new), k_new.stride(0), L.ptr(v_new), v_new.stride(0),
                                     k_cache.data_ptr() + (T - S) * D, T * D, vt_cache.data_ptr() + (T - S), T,
                                     S, heads, D, L.current_stream(k_new.device))
    L.check(rc, "ti_kv_append_i8")
