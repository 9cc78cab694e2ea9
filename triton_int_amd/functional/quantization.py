"""Absmax quantisation helpers used by the modules' `from_float` constructors
(reference: triton_int/functional/quantization.py).  One-off host-side preparation in plain
torch, not part of the per-token path.  Like the reference, the quantisers that divide in place
modify their argument.
"""
import torch

_QMAX = 127


def _fp32_on_cpu(t):
    # CPU tensors are rounded in fp32 (half rounding is not available on the CPU)
    return t if t.is_cuda else t.float()


def _absmax_scale(t, dim=None):
    m = t.abs().max() if dim is None else t.abs().max(dim=dim, keepdim=True)[0]
    return m


@torch.no_grad()
def quantize_per_tensor_absmax(t):
    """-> (int8 tensor, scale) with scale = max|t| / 127; no clamp (reference: :5-14)."""
    scale = _absmax_scale(t) / _QMAX
    t = _fp32_on_cpu(t)
    t.div_(scale).round_()
    return t.to(torch.int8), scale


@torch.no_grad()
def quantize_weight_per_channel_absmax(w):
    """w [out, in] -> (int8 weight, scales [out, 1]) (reference: :16-27)."""
    scales = (w.abs().max(dim=1)[0] / _QMAX).view(-1, 1)
    w = _fp32_on_cpu(w)
    w.div_(scales).round_().clamp_(-128, 127)
    return w.to(torch.int8), scales


@torch.no_grad()
def dynamic_quantize_activation_per_tensor_zeropoint(t):
    """Asymmetric per-tensor quantisation -> (int8, scale, zero point) (reference: :30-45).
    The reference indexes the 0-dim results of max()/min() (`t.max()[0]`), which raises; the
    intended arithmetic is kept."""
    hi, lo = t.max(), t.min()
    step = (hi - lo) / (2 * _QMAX)
    zp = (hi + lo) / 2
    zp = (zp / step).round() * step
    t -= zp
    scale = torch.clamp((hi - lo) / 2, min=1e-8) / _QMAX
    q = (t / scale).round().clamp(-128, 127).to(torch.int8)
    return q, scale, zp


@torch.no_grad()
def dynamic_quantize_activation_per_tensor_absmax(t):
    scale = torch.clamp(_absmax_scale(t), min=1e-8) / _QMAX
    return (t / scale).round().clamp(-128, 127).to(torch.int8), scale


@torch.no_grad()
def dynamic_quantize_activation_per_token_absmax(t):
    if t.is_cuda and t.dtype in (torch.float32, torch.float16):
        # one HIP kernel instead of five torch passes; the reference helper also leaves the rounded
        # quotients in `t` (functional/quantization.py:65), kept here for callers that rely on it
        from ..kernels.fused import quantize_per_token_absmax
        q, scale = quantize_per_token_absmax(t)
        t.copy_(q)
        return q, scale
    scale = torch.clamp(_absmax_scale(t, dim=-1), min=1e-8) / _QMAX
    t.div_(scale).round_().clamp_(-128, 127)
    return t.to(torch.int8), scale


@torch.no_grad()
def fake_quantize_activation_per_tensor_absmax(t):
    scale = torch.clamp(_absmax_scale(t), min=1e-8) / _QMAX
    return t.div_(scale).round_().clamp_(-128, 127).mul_(scale)


@torch.no_grad()
def fake_quantize_activation_per_token_absmax(t):
    scale = torch.clamp(_absmax_scale(t, dim=-1), min=1e-8) / _QMAX
    return t.div_(scale).round_().clamp_(-128, 127).mul_(scale)


@torch.no_grad()
def dequantize_activation_w_per_channel_a_per_token(q_act, w_scales, a_scales):
    """q_act [B, dim], w_scales [dim], a_scales [B, 1] -> a_scales.dtype (reference: :78-86)."""
    out = q_act.to(torch.float32)
    out.mul_(w_scales.reshape(1, -1)).mul_(a_scales.reshape(-1, 1))
    return out.to(a_scales.dtype)


@torch.no_grad()
def dequantize_activation_w_per_channel_a_per_tensor(q_act, w_scales, a_scales):
    """q_act [..., dim], w_scales [dim], a_scales [1] (reference: :88-97)."""
    out = q_act.to(torch.float32) * w_scales.reshape(1, -1) * a_scales
    return out.to(a_scales.dtype)
