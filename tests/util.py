"""Shared helpers for the GPU parity tests: seeded inputs are generated on the CPU with numpy and
copied to the GPU, so the oracle and the HIP kernels see identical bytes."""
import numpy as np
import torch

DEV = "cuda:0"


def rng(seed):
    return np.random.default_rng(seed)


def rand_i8(g, *shape, lo=-127, hi=127):
    return g.integers(lo, hi + 1, size=shape, dtype=np.int8)


def gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def cpu(t):
    t = t.detach().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def mismatch_report(got, want):
    """(max abs diff, mismatch rate) for integer outputs"""
    d = np.abs(got.astype(np.int64) - want.astype(np.int64))
    return int(d.max()) if d.size else 0, float((d != 0).mean()) if d.size else 0.0
