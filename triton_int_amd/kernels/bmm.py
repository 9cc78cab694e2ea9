"""int8 batched-matmul launchers — same names and arguments as triton_int/kernels/bmm.py.

"s8t_s8n": a [B,M,K], b [B,N,K] (both K-contiguous);  "s8t_s8t": b is [B,K,N].
"""
from __future__ import annotations

import torch

from .. import _lib as L
from ._gemm import bmm as _bmm


def bmm_s8t_s8t_s32t(a, b, out=None, *, _config=-1):
    """acc, b = [B,K,N] (reference: kernels/bmm.py:125-160)."""
    return _bmm(a, b, b_is_kn=True, epilogue=L.EPI_I32, out_dtype=torch.int32, out=out, config=_config)


def bmm_s8t_s8n_s32t(a, b, out=None, *, _config=-1):
    """acc, bit-exact int32 (reference: kernels/bmm.py:276-311)."""
    return _bmm(a, b, b_is_kn=False, epilogue=L.EPI_I32, out_dtype=torch.int32, out=out, config=_config)


def bmm_s8t_s8n_f32t(a, b, scale, out=None, dtype=torch.float32, *, _config=-1):
    """scale * acc -> fp32 / fp16 / bf16 (reference: kernels/bmm.py:428-464)."""
    return _bmm(a, b, b_is_kn=False, epilogue=L.EPI_SCALE_F, out_dtype=dtype, alpha=scale, out=out, config=_config)


def bmm_s8t_s8n_s8t(a, b, scale, out=None, *, _round_mode=L.ROUND_RNE_CLAMP, _config=-1):
    """q8(scale * acc) (reference: kernels/bmm.py:576-612)."""
    return _bmm(a, b, b_is_kn=False, epilogue=L.EPI_SCALE_I8, out_dtype=torch.int8, alpha=scale, out=out,
                round_mode=_round_mode, config=_config)


def bmm_s8t_s8t_s8t(a, b, scale, out=None, *, _round_mode=L.ROUND_RNE_CLAMP, _config=-1):
    """q8(scale * acc), b = [B,K,N] (reference: kernels/bmm.py:724-760)."""
    return _bmm(a, b, b_is_kn=True, epilogue=L.EPI_SCALE_I8, out_dtype=torch.int8, alpha=scale, out=out,
                round_mode=_round_mode, config=_config)
