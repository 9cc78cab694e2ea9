"""Shared launcher plumbing for the int8 GEMM / BMM entry point ti_bmm_i8."""
from __future__ import annotations

import torch

from .. import _lib as L


def _launch(a, sa, b, sb, c, sc, B, M, N, K, *, epilogue, bias, alpha, beta, round_mode, config, grouped=False):
    """One ti_bmm_i8_config call: a/b/c are tensors (for pointers, dtype, device), sa/sb/sc the
    (batch, row, column) element strides of the logical [B,M,K] / [B,N,K] / [B,M,N] views.
    grouped: the batches are B projections with their own bias rows ([B*N] elements) and their
    own scales (alpha / beta are fp32 device tensors of B elements): ti_bmm_i8_grouped."""
    L.require_cuda(a, b, c, bias)
    assert a.dtype == torch.int8 and b.dtype == torch.int8, "operands must be int8"
    dev = a.device
    assert b.device == dev and c.device == dev, "operands must be on one device"
    bias_kind = L.BIAS_NONE
    bias_ptr = 0
    if bias is not None:
        assert bias.device == dev
        assert bias.numel() == (B * N if grouped else N), "bias must have one element per output column"
        if not bias.is_contiguous():
            bias = bias.contiguous()
        bias_kind = L.TORCH_TO_BIAS[bias.dtype]
        bias_ptr = bias.data_ptr()
    if grouped:
        for t in (alpha, beta):
            assert t is None or (t.dtype == torch.float32 and t.device == dev and t.numel() == B and t.is_contiguous()), \
                "grouped scales must be fp32 device tensors with one element per projection"
        with L.on_device(dev):
            rc = L.lib().ti_bmm_i8_grouped(
                a.data_ptr(), sa[0], sa[1], sa[2], b.data_ptr(), sb[0], sb[1], sb[2], c.data_ptr(), sc[0], sc[1], sc[2],
                B, M, N, K, bias_ptr, bias_kind, N, 0 if alpha is None else alpha.data_ptr(),
                0 if beta is None else beta.data_ptr(), 1,
                int(epilogue), L.TORCH_TO_DT[c.dtype], int(round_mode), int(config), L.current_stream(dev))
        if rc != 0:
            L.check(rc, "ti_bmm_i8_grouped")
        return
    # the converted scales stay bound to locals until the launch is enqueued: a scale that is not
    # already fp32 on `dev` is a fresh copy, and a freed copy's block would be handed to the next one
    alpha_t = None if alpha is None else L.scale_tensor(alpha, dev)
    beta_t = None if beta is None else L.scale_tensor(beta, dev)
    with L.on_device(dev):
        rc = L.lib().ti_bmm_i8_config(
            a.data_ptr(), sa[0], sa[1], sa[2], b.data_ptr(), sb[0], sb[1], sb[2], c.data_ptr(), sc[0], sc[1], sc[2],
            B, M, N, K, bias_ptr, bias_kind, L.ptr(alpha_t), L.ptr(beta_t),
            int(epilogue), L.TORCH_TO_DT[c.dtype], int(round_mode), int(config), L.current_stream(dev))
    if rc != 0:
        L.check(rc, "ti_bmm_i8")


def launch_bmm(a3, b3, c3, *, epilogue, bias=None, alpha=None, beta=None, round_mode=L.ROUND_RNE_CLAMP,
               config=-1):
    """a3 [B,M,K] int8, b3 [B,N,K] int8 (logical; any strides), c3 [B,M,N] preallocated."""
    B, M, K = a3.shape
    _, N, _ = b3.shape
    _launch(a3, a3.stride(), b3, b3.stride(), c3, c3.stride(), B, M, N, K, epilogue=epilogue, bias=bias,
            alpha=alpha, beta=beta, round_mode=round_mode, config=config)
    return c3


def linear(a, w, *, epilogue, out_dtype, bias=None, alpha=None, beta=None, out=None,
           round_mode=L.ROUND_RNE_CLAMP, config=-1):
    """Common body of the linear_* launchers (reference: kernels/linear.py:257-288 and siblings)."""
    tmp_shape = a.shape[:-1]
    assert len(w.shape) == 2
    assert a.shape[-1] == w.shape[1], "Incompatible dimensions"
    N, K = w.shape
    M = 1
    for d in tmp_shape:
        M *= d
    a = a.view(M, K)
    if out is None:
        c = torch.empty((M, N), device=a.device, dtype=out_dtype)
    else:
        assert out.dtype == out_dtype and out.numel() == M * N, "out has the wrong dtype or size"
        c = out.view(M, N)
    _launch(a, (0, a.stride(0), a.stride(1)), w, (0, w.stride(0), w.stride(1)), c, (0, c.stride(0), c.stride(1)),
            1, M, N, K, epilogue=epilogue, bias=bias, alpha=alpha, beta=beta, round_mode=round_mode, config=config)
    return c.view(*tmp_shape, N)


def bmm(a, b, *, b_is_kn, epilogue, out_dtype, alpha=None, out=None, round_mode=L.ROUND_RNE_CLAMP, config=-1):
    """Common body of the bmm_* launchers (reference: kernels/bmm.py:577-612 and siblings)."""
    tmp_shape = a.shape[:-1]
    assert len(a.shape) == 3 and len(b.shape) == 3
    assert a.shape[0] == b.shape[0]
    if b_is_kn:
        assert a.shape[2] == b.shape[1], "Incompatible dimensions"
        b = b.transpose(1, 2)  # logical [B,N,K] view of the [B,K,N] operand
    else:
        assert a.shape[2] == b.shape[2], "Incompatible dimensions"
    _, M, K = a.shape
    B, N, K = b.shape
    if out is None:
        c = torch.empty((B, M, N), device=a.device, dtype=out_dtype)
    else:
        assert out.dtype == out_dtype and out.shape == (B, M, N), "out has the wrong dtype or shape"
        c = out
    launch_bmm(a, b, c, epilogue=epilogue, alpha=alpha, round_mode=round_mode, config=config)
    return c.view(*tmp_shape, N)


def linear_group(a, w, groups, *, epilogue, out_dtype, bias=None, alpha=None, beta=None, out=None,
                 round_mode=L.ROUND_RNE_CLAMP, config=-1):
    """`groups` linears that share the input, as one launch: w is their [N,K] weights stacked to
    [groups*N, K], bias [groups*N], alpha / beta fp32 device tensors [groups].  Returns
    [*, groups*N]: projection g is columns g*N .. g*N+N.  Same arithmetic per projection as
    `linear` (reference: kernels/linear.py:257-288 launched once per projection)."""
    tmp_shape = a.shape[:-1]
    assert len(w.shape) == 2 and w.shape[0] % groups == 0
    assert a.shape[-1] == w.shape[1], "Incompatible dimensions"
    GN, K = w.shape
    N = GN // groups
    M = 1
    for d in tmp_shape:
        M *= d
    a = a.view(M, K)
    if out is None:
        c = torch.empty((M, GN), device=a.device, dtype=out_dtype)
    else:
        assert out.dtype == out_dtype and out.numel() == M * GN, "out has the wrong dtype or size"
        c = out.view(M, GN)
    _launch(a, (0, a.stride(0), a.stride(1)), w, (N * w.stride(0), w.stride(0), w.stride(1)),
            c, (N * c.stride(1), c.stride(0), c.stride(1)), groups, M, N, K, epilogue=epilogue, bias=bias,
            alpha=alpha, beta=beta, round_mode=round_mode, config=config, grouped=True)
    return c.view(*tmp_shape, GN)
