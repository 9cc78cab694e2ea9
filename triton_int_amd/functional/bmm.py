"""Aliases of the two most-used BMMs (reference: triton_int/functional/bmm.py:6-18)."""
from ..kernels.bmm import bmm_s8t_s8n_s8t, bmm_s8t_s8n_s32t


def bmm_i8_o8(a, b, scale):
    """a [B,M,K] int8, b [B,N,K] int8 -> int8 [B,M,N] = q8(scale * a @ b^T)."""
    return bmm_s8t_s8n_s8t(a, b, scale)


def bmm_i8_o32(a, b):
    """a [B,M,K] int8, b [B,N,K] int8 -> int32 [B,M,N] = a @ b^T."""
    return bmm_s8t_s8n_s32t(a, b)
