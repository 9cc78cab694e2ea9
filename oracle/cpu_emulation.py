"""The reference's "PyTorch CPU emulation path" for the linears and BMMs — TEST/BENCH INFRASTRUCTURE.

The reference has no such function for the GEMMs (its only live emulations are
functional/fused.py:6-15 and nn/fused.py:8-32); the baseline defines it as int32 torch.matmul
plus the same scaling.  This restates that path with stock torch calls so that the benchmark can
time it on the host beside the GPU kernels.  Not used by the product.
"""
import torch
import torch.nn.functional as F


def linear_o8(x, w, bias_i8, alpha, beta):
    acc = torch.matmul(x.to(torch.int32), w.to(torch.int32).T)
    v = alpha * acc.float() + beta * bias_i8.float()
    return torch.clamp(torch.round(v), -128, 127).to(torch.int8)


def linear_ofp32(x, w, bias_f32, alpha, beta=1.0):
    acc = torch.matmul(x.to(torch.int32), w.to(torch.int32).T)
    return alpha * acc.float() + beta * bias_f32


def linear_gelu_q(x, w, bias_f32, alpha, beta):
    acc = torch.matmul(x.to(torch.int32), w.to(torch.int32).T)
    y = F.gelu(alpha * acc.float() + bias_f32, approximate="tanh") * beta
    return torch.clamp(torch.round(y), -128, 127).to(torch.int8)


def bmm_o8(a, b, alpha):
    acc = torch.bmm(a.to(torch.int32), b.to(torch.int32).transpose(1, 2))
    return torch.clamp(torch.round(alpha * acc.float()), -128, 127).to(torch.int8)


def dq_add_layernorm_q(acc_i32, scale, resid, gamma, beta, eps):
    """functional/fused.py:6-15 verbatim in behaviour."""
    r = torch.add(resid, acc_i32, alpha=scale)
    ln = F.layer_norm(r, r.shape[-1:], gamma, beta, eps)
    return r, ln.clamp(-128, 127).round().to(torch.int8)
