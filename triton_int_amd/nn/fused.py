"""LayerNorm-quant, dequant+add+LayerNorm-quant, GELU-quant and the GELU-quant linear
(reference: triton_int/nn/fused.py).  `weight`/`bias` of the norm modules already hold
gamma / output_scale and beta / output_scale (reference: nn/fused.py:54-55)."""
from __future__ import annotations

import torch

from ..functional.fused import dq_add_layernorm_q_cpp
from ..functional.quantization import quantize_per_tensor_absmax
from ..kernels.fused import gelu_q, layer_norm_fwd_fused_single_pass_q, linear_a8_w8_bfp32_ofp32_GeLu_Q
from .linear import _Int8Linear, _scale_tensor


class _NormQ(torch.nn.Module):
    def __init__(self, dim, eps=1e-5):
        super().__init__()
        self.input_scale = 1.0
        self.eps = eps
        self.register_buffer("weight", torch.ones(dim, dtype=torch.float32))
        self.register_buffer("bias", torch.zeros(dim, dtype=torch.float32))

    @classmethod
    def from_float(cls, module: torch.nn.LayerNorm, output_scale: float):
        assert module.normalized_shape[0] == module.weight.numel()
        assert module.normalized_shape[0] == module.bias.numel()
        q = cls(module.normalized_shape[0], module.eps)
        q.weight = module.weight / output_scale
        q.bias = module.bias / output_scale
        return q


class LayerNormQ(_NormQ):
    """fp activations -> int8 normalised activations (reference: nn/fused.py:34-57)."""

    def forward(self, x):
        return layer_norm_fwd_fused_single_pass_q(x.to(self.weight.dtype), self.weight, self.bias, self.eps)


# The reference keeps a PyTorch emulation under this name (nn/fused.py:8-32); here it is the same
# kernel-backed module so callers of either name get the native path.
_LayerNormQ = LayerNormQ


class DQ_Add_LayerNorm_Q(_NormQ):
    """(residual fp32, int32 accumulator) -> (new residual fp32, int8) (reference: nn/fused.py:59-78)."""

    def forward(self, residual_input_fp, input_int32):
        return dq_add_layernorm_q_cpp(input_int32, self.input_scale, residual_input_fp, self.weight, self.bias,
                                      self.eps)


class GeLu_Q(torch.nn.Module):
    """Stand-alone tanh-GELU + quantise: int8 = q8(gelu(x) * a) (reference: nn/fused.py:81-87, whose
    forward cannot run because it calls a Triton device function from the host)."""

    def __init__(self, alpha=1):
        super().__init__()
        self.register_buffer("a", torch.tensor(float(alpha), dtype=torch.float32))

    def forward(self, x):
        return gelu_q(x, self.a)


class W8A8BFP32OFP32_GeLu_Q(_Int8Linear):
    """fc1 with the GELU-quant epilogue: int8 in, fp32 bias, int8 out; `b` = 1 / output scale
    (reference: nn/fused.py:90-151)."""

    bias_dtype = torch.float32

    def _launch(self, x):
        return linear_a8_w8_bfp32_ofp32_GeLu_Q(x, self.weight, self.bias, self.a, self.b)

    @classmethod
    def from_float(cls, module: torch.nn.Linear, input_scale, out_scale):
        q = cls(module.in_features, module.out_features)
        q.weight, weight_scale = quantize_per_tensor_absmax(module.weight)
        q.bias = module.bias.to(torch.float32)
        q.a = _scale_tensor(input_scale * weight_scale)
        q.b = _scale_tensor(1 / out_scale)
        q.input_scale, q.weight_scale = input_scale, weight_scale
        return q
