"""int8 batched-matmul modules (reference: triton_int/nn/bmm.py).  Buffer `a` holds alpha."""
from __future__ import annotations

import torch

from ..kernels.bmm import bmm_s8t_s8n_f32t, bmm_s8t_s8n_s8t, bmm_s8t_s8n_s32t, bmm_s8t_s8t_s8t


def _as_tensor(alpha):
    return alpha.to(torch.float32) if torch.is_tensor(alpha) else torch.tensor(alpha, dtype=torch.float32)


class _ScaledBMM(torch.nn.Module):
    def __init__(self, alpha):
        super().__init__()
        self.register_buffer("a", _as_tensor(alpha))

    def _apply(self, fn, *args, **kwargs):
        super()._apply(fn, *args, **kwargs)
        if self.a.dtype != torch.float32:  # the kernels read alpha as fp32
            self.a = self.a.to(torch.float32)
        return self


class BMM_S8T_S8N_S8T(_ScaledBMM):
    """a [B,M,K] int8, b [B,N,K] int8 -> int8 [B,M,N] (reference: nn/bmm.py:10-29)."""

    @torch.no_grad()
    def forward(self, a, b):
        return bmm_s8t_s8n_s8t(a, b, self.a)

    @classmethod
    def from_scale(cls, a_scale, b_scale, output_scale):
        return cls(a_scale * b_scale / output_scale)


class BMM_S8T_S8T_S8T(_ScaledBMM):
    """a [B,M,K] int8, b [B,K,N] int8 -> int8 [B,M,N] (reference: nn/bmm.py:32-51)."""

    @torch.no_grad()
    def forward(self, a, b):
        return bmm_s8t_s8t_s8t(a, b, self.a)

    @classmethod
    def from_scale(cls, a_scale, b_scale, output_scale):
        return cls(a_scale * b_scale / output_scale)


class BMM_S8T_S8N_F32T(_ScaledBMM):
    """a [B,M,K] int8, b [B,N,K] int8 -> `dtype` [B,M,N] (reference: nn/bmm.py:54-74)."""

    def __init__(self, alpha, dtype=torch.float32):
        super().__init__(alpha)
        self.dtype = dtype

    @torch.no_grad()
    def forward(self, a, b):
        return bmm_s8t_s8n_f32t(a, b, self.a, dtype=self.dtype)

    @classmethod
    def from_scale(cls, a_scale, b_scale, dtype=torch.float32):
        return cls(a_scale * b_scale, dtype=dtype)


class BMM_S8T_S8N_F16T(BMM_S8T_S8N_F32T):
    """fp16 output (reference: nn/bmm.py:77-96)."""

    def __init__(self, alpha):
        super().__init__(alpha, dtype=torch.float16)

    @classmethod
    def from_scale(cls, a_scale, b_scale):
        return cls(a_scale * b_scale)


class BMM_S8T_S8N_BF16T(BMM_S8T_S8N_F32T):
    """bf16 output (reference: nn/bmm.py:99-118)."""

    def __init__(self, alpha):
        super().__init__(alpha, dtype=torch.bfloat16)

    @classmethod
    def from_scale(cls, a_scale, b_scale):
        return cls(a_scale * b_scale)


class BMM_S8T_S8N_S32T(torch.nn.Module):
    """raw int32 accumulator (reference: nn/bmm.py:121-130)."""

    @torch.no_grad()
    def forward(self, a, b):
        return bmm_s8t_s8n_s32t(a, b)
