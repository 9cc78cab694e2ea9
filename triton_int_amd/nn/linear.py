"""W8A8 linear modules (reference: triton_int/nn/linear.py:18-278).

Same class names, constructor arguments, buffer names (`weight` int8 [out,in], `bias`, 0-dim fp32
scales `a`, `b`) and `from_float` algebra as the reference, so state_dicts interchange.  `forward`
flattens the leading dims, calls the HIP launcher and restores the shape.
"""
from __future__ import annotations

import torch

from ..functional.quantization import quantize_per_tensor_absmax
from ..kernels.linear import (
    linear_a8_w8_b8_o8,
    linear_a8_w8_b32_o32,
    linear_a8_w8_b32_o32_with_scaling,
    linear_a8_w8_bfp32_ofp32,
    linear_a8_w8_bfp32_ofp32_residual,
    linear_relu_a8_w8_b8_o8,
)


class _Int8Linear(torch.nn.Module):
    """int8 weight [out_features, in_features] + bias of `bias_dtype` + optional fp32 scales."""

    bias_dtype = torch.int8
    has_scales = True

    def __init__(self, in_features, out_features, alpha=1.0, beta=1.0):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        # random int8 weights in [-127, 127) like the reference constructor (nn/linear.py:25-35)
        self.register_buffer("weight", torch.randint(-127, 127, (out_features, in_features), dtype=torch.int8))
        self.register_buffer("bias", torch.zeros(out_features, dtype=self.bias_dtype))
        if self.has_scales:
            self.register_buffer("a", torch.tensor(alpha, dtype=torch.float32))
            self.register_buffer("b", torch.tensor(beta, dtype=torch.float32))

    def _apply(self, fn, *args, **kwargs):
        # .half()/.to(dtype) must not touch what the kernels read as fp32: the scales and an fp32 bias
        super()._apply(fn, *args, **kwargs)
        for name in ("a", "b", "bias"):
            t = getattr(self, name, None)
            if torch.is_tensor(t) and t.is_floating_point() and t.dtype != torch.float32:
                setattr(self, name, t.to(torch.float32))
        return self

    def _launch(self, x2d):
        raise NotImplementedError

    @torch.no_grad()
    def forward(self, x):
        lead = x.shape[:-1]
        y = self._launch(x.view(-1, x.shape[-1]))
        return y.view(*lead, -1)


def _scale_tensor(v):
    return v.to(torch.float32) if torch.is_tensor(v) else torch.tensor(v, dtype=torch.float32)


class W8A8B8O8Linear(_Int8Linear):
    """q/k/v projections: int8 in, int8 bias, int8 out (reference: nn/linear.py:18-67)."""

    def _launch(self, x):
        return linear_a8_w8_b8_o8(x, self.weight, self.bias, self.a, self.b)

    @classmethod
    def from_float(cls, module: torch.nn.Linear, input_scale, output_scale):
        q = cls(module.in_features, module.out_features)
        q.weight, weight_scale = quantize_per_tensor_absmax(module.weight)
        q.bias, bias_scale = quantize_per_tensor_absmax(module.bias)
        q.a = _scale_tensor(input_scale * weight_scale / output_scale)
        q.b = _scale_tensor(bias_scale / output_scale)
        return q


class W8A8B8O8LinearReLU(W8A8B8O8Linear):
    """fc1 with ReLU folded into the epilogue (reference: nn/linear.py:70-122)."""

    def _launch(self, x):
        return linear_relu_a8_w8_b8_o8(x, self.weight, self.bias, self.a, self.b)


class W8A8B32O32LinearWithoutScaling(_Int8Linear):
    """int32 bias, raw int32 accumulator out (reference: nn/linear.py:125-160)."""

    bias_dtype = torch.int32
    has_scales = False

    def __init__(self, in_features, out_features):
        super().__init__(in_features, out_features)

    def _launch(self, x):
        return linear_a8_w8_b32_o32(x, self.weight, self.bias)


class W8A8B32O32Linear(_Int8Linear):
    """int32 bias, scaled int32 out (reference: nn/linear.py:163-219)."""

    bias_dtype = torch.int32

    def _launch(self, x):
        return linear_a8_w8_b32_o32_with_scaling(x, self.weight, self.bias, self.a, self.b)

    @classmethod
    def from_float(cls, module: torch.nn.Linear, input_scale, output_scale):
        q = cls(module.in_features, module.out_features)
        q.weight, weight_scale = quantize_per_tensor_absmax(module.weight)
        module.bias = module.bias.float()
        bias_scale = module.bias.abs().max() / (2**31 - 1)
        q.bias = (module.bias / bias_scale).round().to(torch.int32)
        q.a = _scale_tensor(input_scale * weight_scale / output_scale)
        q.b = _scale_tensor(bias_scale / output_scale)
        q.input_scale, q.output_scale = input_scale, output_scale
        q.weight_scale, q.bias_scale = weight_scale, bias_scale
        return q


class W8A8BFP32OFP32Linear(_Int8Linear):
    """fc2 / out_proj: fp32 bias, fp32 out; `b` is fixed to 1 (reference: nn/linear.py:222-278)."""

    bias_dtype = torch.float32

    def __init__(self, in_features, out_features, alpha=1.0, beta=1.0):
        super().__init__(in_features, out_features, alpha, 1.0)

    def _launch(self, x):
        return linear_a8_w8_bfp32_ofp32(x, self.weight, self.bias, self.a, self.b)

    @torch.no_grad()
    def forward_add(self, x, residual):
        """forward(x) + residual (fp32, same shape as the output) as one library call."""
        lead = x.shape[:-1]
        y = linear_a8_w8_bfp32_ofp32_residual(x.view(-1, x.shape[-1]), self.weight, self.bias, self.a, self.b,
                                              residual.reshape(-1, self.out_features))
        return y.view(*lead, -1)

    @classmethod
    def from_float(cls, module: torch.nn.Linear, input_scale):
        q = cls(module.in_features, module.out_features)
        q.weight, weight_scale = quantize_per_tensor_absmax(module.weight)
        q.bias = module.bias.to(torch.float32)
        q.a = _scale_tensor(input_scale * weight_scale)
        q.input_scale, q.weight_scale = input_scale, weight_scale
        return q


class DynamicW8A8BFP32OFP32Linear(torch.nn.Module):
    """fc2 / out_proj with the activation quantised on the fly, per tensor (reference:
    nn/linear.py:281-342, `DanymicW8A8BFP32OFP32Linear`).  The reference's forward cannot run (it
    names an attribute that does not exist and registers `weight_scale` twice); this is the
    arithmetic it spells out: `x8, s = quantize_per_tensor_absmax(x)`, then
    `linear_a8_w8_bfp32_ofp32(x8, weight, bias, s * weight_scale, 1)`.  The scale stays a device
    tensor (no host synchronisation) and, unlike the helper, the caller's `x` is left untouched."""

    def __init__(self, in_features, out_features, alpha=1.0, beta=1.0):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        self.register_buffer("weight", torch.randint(-127, 127, (out_features, in_features), dtype=torch.int8))
        self.register_buffer("bias", torch.zeros(out_features, dtype=torch.float32))
        self.register_buffer("weight_scale", torch.tensor(alpha, dtype=torch.float32))
        self.register_buffer("b", torch.tensor(1.0, dtype=torch.float32))

    def _apply(self, fn, *args, **kwargs):
        super()._apply(fn, *args, **kwargs)
        for name in ("bias", "weight_scale", "b"):  # what the kernel reads as fp32 stays fp32 under .half()
            t = getattr(self, name)
            if t.dtype != torch.float32:
                setattr(self, name, t.to(torch.float32))
        return self

    @torch.no_grad()
    def forward(self, x):
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        scale = x2.abs().max() / 127                        # quantize_per_tensor_absmax (functional/quantization.py:5-14)
        x8 = (x2 / scale).round_().to(torch.int8)
        alpha = (scale.to(torch.float32) * self.weight_scale).to(torch.float32)
        y = linear_a8_w8_bfp32_ofp32(x8, self.weight, self.bias, alpha, self.b)
        return y.view(*lead, -1)

    @classmethod
    def from_float(cls, module: torch.nn.Linear):
        q = cls(module.in_features, module.out_features)
        q.weight, weight_scale = quantize_per_tensor_absmax(module.weight)
        q.bias = module.bias.to(torch.float32)
        q.weight_scale = weight_scale.to(torch.float32).reshape(())
        return q


DanymicW8A8BFP32OFP32Linear = DynamicW8A8BFP32OFP32Linear  # the reference's spelling (nn/linear.py:281)
