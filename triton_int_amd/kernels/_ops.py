"""`torch.ops.triton_op.*` registration of the launchers, with Meta (shape) implementations so that
they can be traced by torch.compile / fake tensors.

The reference registers its launchers under the same namespace (kernels/__init__.py:5-24) but
builds the schema from python annotations its functions do not carry (the result is malformed and
unused by its modules).  Here every schema is written out; the CUDA implementation is the launcher
of the same name, the Meta implementation only allocates an output of the right shape and dtype.
Scales are Tensors in the linear ops (the modules hold them as 0-dim fp32 buffers) and floats in
the BMM / row ops, as the launchers take them.
"""
from __future__ import annotations

import torch

from . import bmm as _bmm
from . import fused as _fused
from . import linear as _linear

NAMESPACE = "triton_op"


def _lin_out(a, b, dtype):
    return a.new_empty((*a.shape[:-1], b.shape[0]), dtype=dtype)


def _bmm_out(a, b, dtype, b_is_kn=False):
    return a.new_empty((a.shape[0], a.shape[1], b.shape[2] if b_is_kn else b.shape[1]), dtype=dtype)


# name -> (schema, CUDA implementation, Meta implementation)
_OPS = {
    "linear_a8_w8_b8_o8": (
        "(Tensor a, Tensor b, Tensor bias, Tensor scale_a, Tensor scale_b) -> Tensor",
        lambda a, b, bias, sa, sb: _linear.linear_a8_w8_b8_o8(a, b, bias, sa, sb),
        lambda a, b, bias, sa, sb: _lin_out(a, b, torch.int8)),
    "linear_relu_a8_w8_b8_o8": (
        "(Tensor a, Tensor b, Tensor bias, Tensor scale_a, Tensor scale_b) -> Tensor",
        lambda a, b, bias, sa, sb: _linear.linear_relu_a8_w8_b8_o8(a, b, bias, sa, sb),
        lambda a, b, bias, sa, sb: _lin_out(a, b, torch.int8)),
    "linear_a8_w8_b32_o32": (
        "(Tensor a, Tensor b, Tensor? bias) -> Tensor",
        lambda a, b, bias: _linear.linear_a8_w8_b32_o32(a, b, bias),
        lambda a, b, bias: _lin_out(a, b, torch.int32)),
    "linear_a8_w8_b32_o32_with_scaling": (
        "(Tensor a, Tensor b, Tensor bias, Tensor scale_a, Tensor scale_b) -> Tensor",
        lambda a, b, bias, sa, sb: _linear.linear_a8_w8_b32_o32_with_scaling(a, b, bias, sa, sb),
        lambda a, b, bias, sa, sb: _lin_out(a, b, torch.int32)),
    "linear_a8_w8_bfp32_ofp32": (
        "(Tensor a, Tensor b, Tensor? bias, Tensor scale_a, Tensor scale_b) -> Tensor",
        lambda a, b, bias, sa, sb: _linear.linear_a8_w8_bfp32_ofp32(a, b, bias, sa, sb, dtype=torch.float32),
        lambda a, b, bias, sa, sb: _lin_out(a, b, torch.float32)),
    "linear_a8_w8_bfp32_ofp32_residual": (
        "(Tensor a, Tensor b, Tensor? bias, Tensor scale_a, Tensor scale_b, Tensor residual) -> Tensor",
        lambda a, b, bias, sa, sb, r: _linear.linear_a8_w8_bfp32_ofp32_residual(a, b, bias, sa, sb, r),
        lambda a, b, bias, sa, sb, r: _lin_out(a, b, torch.float32)),
    "linear_a8_w8_ofp32": (
        "(Tensor a, Tensor b, Tensor scale) -> Tensor",
        lambda a, b, s: _linear.linear_a8_w8_ofp32(a, b, s),
        lambda a, b, s: _lin_out(a, b, torch.float32)),
    "linear_a8_w8_bfp32_ofp32_GeLu_Q": (
        "(Tensor a, Tensor b, Tensor bias, Tensor scale_a, Tensor scale_b) -> Tensor",
        lambda a, b, bias, sa, sb: _fused.linear_a8_w8_bfp32_ofp32_GeLu_Q(a, b, bias, sa, sb),
        lambda a, b, bias, sa, sb: _lin_out(a, b, torch.int8)),
    "bmm_s8t_s8n_s8t": (
        "(Tensor a, Tensor b, float scale) -> Tensor",
        lambda a, b, s: _bmm.bmm_s8t_s8n_s8t(a, b, s),
        lambda a, b, s: _bmm_out(a, b, torch.int8)),
    "bmm_s8t_s8n_f32t": (
        "(Tensor a, Tensor b, float scale) -> Tensor",
        lambda a, b, s: _bmm.bmm_s8t_s8n_f32t(a, b, s),
        lambda a, b, s: _bmm_out(a, b, torch.float32)),
    "bmm_s8t_s8n_s32t": (
        "(Tensor a, Tensor b) -> Tensor",
        lambda a, b: _bmm.bmm_s8t_s8n_s32t(a, b),
        lambda a, b: _bmm_out(a, b, torch.int32)),
    "bmm_s8t_s8t_s8t": (
        "(Tensor a, Tensor b, float scale) -> Tensor",
        lambda a, b, s: _bmm.bmm_s8t_s8t_s8t(a, b, s),
        lambda a, b, s: _bmm_out(a, b, torch.int8, b_is_kn=True)),
    "bmm_s8t_s8t_s32t": (
        "(Tensor a, Tensor b) -> Tensor",
        lambda a, b: _bmm.bmm_s8t_s8t_s32t(a, b),
        lambda a, b: _bmm_out(a, b, torch.int32, b_is_kn=True)),
    "layer_norm_fwd_fused_single_pass_q": (
        "(Tensor x, Tensor weight, Tensor? bias, float eps) -> Tensor",
        lambda x, w, b, eps: _fused.layer_norm_fwd_fused_single_pass_q(x, w, b, eps),
        lambda x, w, b, eps: x.new_empty(x.shape, dtype=torch.int8)),
    "layer_norm_fwd_fused_single_pass": (
        "(Tensor x, Tensor weight, Tensor? bias, float eps, bool use_rms_norm=False) -> Tensor",
        lambda x, w, b, eps, rms=False: _fused.layer_norm_fwd_fused_single_pass(x, w, b, eps, rms),
        lambda x, w, b, eps, rms=False: x.new_empty(x.shape)),
    "skip_layer_norm_fwd_fused_single_pass": (
        "(Tensor x, Tensor skip, Tensor weight, Tensor? bias, float eps, bool use_rms_norm=False) -> Tensor",
        lambda x, sk, w, b, eps, rms=False: _fused.skip_layer_norm_fwd_fused_single_pass(x, sk, w, b, eps, rms),
        lambda x, sk, w, b, eps, rms=False: x.new_empty(x.shape)),
    "skip_layer_norm_fwd_fused_single_pass2": (
        "(Tensor x, Tensor skip, Tensor weight, Tensor? bias, float eps, bool use_rms_norm=False) -> (Tensor, Tensor)",
        lambda x, sk, w, b, eps, rms=False: tuple(_fused.skip_layer_norm_fwd_fused_single_pass2(x, sk, w, b, eps, rms)),
        lambda x, sk, w, b, eps, rms=False: (x.new_empty(x.shape), x.new_empty(x.shape))),
    "dq_add_layernorm_q": (
        "(Tensor input_int32, float input_scale_fp, Tensor residual_input_fp, Tensor gamma, Tensor beta, float eps)"
        " -> (Tensor, Tensor)",
        lambda acc, s, res, g, b, eps: tuple(_fused.dq_add_layernorm_q(acc, s, res, g, b, eps)),
        lambda acc, s, res, g, b, eps: (res.new_empty(res.shape, dtype=torch.float32),
                                        res.new_empty(res.shape, dtype=torch.int8))),
    "gelu_q": (
        "(Tensor x, float scale) -> Tensor",
        lambda x, s: _fused.gelu_q(x, s),
        lambda x, s: x.new_empty(x.shape, dtype=torch.int8)),
    "softmax_q": (
        "(Tensor x, float scale, int causal_q_len=0) -> Tensor",
        lambda x, s, q=0: _fused.softmax_q(x, s, q),
        lambda x, s, q=0: x.new_empty(x.shape, dtype=torch.int8)),
    "attention_i8": (
        "(Tensor q, Tensor k, Tensor vt, float qk_alpha, float score_scale, float pv_alpha, int causal_q_len=0) -> Tensor",
        lambda q, k, vt, a, s, p, c=0: _fused.attention_i8(q, k, vt, a, s, p, c),
        lambda q, k, vt, a, s, p, c=0: q.new_empty(q.shape, dtype=torch.int8)),
    "quantize_per_token_absmax": (
        "(Tensor t) -> (Tensor, Tensor)",
        lambda t: tuple(_fused.quantize_per_token_absmax(t)),
        lambda t: (t.new_empty(t.shape, dtype=torch.int8), t.new_empty((*t.shape[:-1], 1)))),
}

_lib = None
registered = ()


def register():
    """Define the ops once per process.  A second definition of the namespace's ops (for example by
    the reference package imported next to this one) raises in torch; that case is left alone."""
    global _lib, registered
    if _lib is not None:
        return registered
    _lib = torch.library.Library(NAMESPACE, "FRAGMENT")
    done = []
    for name, (schema, cuda_impl, meta_impl) in _OPS.items():
        try:
            _lib.define(name + schema)
        except RuntimeError:
            continue  # already defined elsewhere in this process
        _lib.impl(name, cuda_impl, "CUDA")
        _lib.impl(name, meta_impl, "Meta")
        done.append(name)
    registered = tuple(done)
    return registered


register()
