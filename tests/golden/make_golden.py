"""Regenerates tests/golden/*.npz from fixed seeds with the CPU oracle (oracle/ti_oracle.c).

    python tests/golden/make_golden.py

The reference repository ships no golden vectors for this path, so these fixtures are produced by
this build's own oracle (itself pinned by tests/test_oracle_*.py).  They freeze the oracle's
behaviour (a later edit that changes a result fails tests/test_golden.py on the CPU) and give the
GPU tests inputs/outputs that do not depend on the oracle being built.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle as O  # noqa: E402


def gemm_case():
    g = np.random.default_rng(101)
    M, N, K = 64, 96, 80
    a = g.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = g.integers(-127, 128, size=(N, K), dtype=np.int8)
    a[0, :] = 127; w[0, :] = 127; w[1, :] = -128          # saturating rows
    a[1, :] = 0; a[1, 0] = 1; w[2:18, 0] = np.arange(-7, 9)  # exact ties with alpha = 0.5
    b8 = g.integers(-127, 128, size=N, dtype=np.int8)
    b32 = g.integers(-2**20, 2**20, size=N, dtype=np.int32)
    bf = g.standard_normal(N).astype(np.float32)
    alpha, beta = np.float32(0.5), np.float32(0.013)
    ag = np.float32(3.0 / (np.sqrt(K) * 127 * 127 / 3)); bg = np.float32(20.0)
    d = dict(a=a, w=w, b8=b8, b32=b32, bf=bf, alpha=alpha, beta=beta, ag=ag, bg=bg)
    d["o32"] = O.linear_a8_w8_b32_o32(a, w, b32)
    d["o32_scaled"] = O.linear_a8_w8_b32_o32_with_scaling(a, w, b32, np.float32(0.01), beta)
    for name, rm in (("rne", O.RNE_CLAMP), ("trunc", O.TRUNC)):
        d[f"o8_{name}"] = O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta, round_mode=rm)
        d[f"o8_relu_{name}"] = O.linear_relu_a8_w8_b8_o8(a, w, b8, alpha, beta, round_mode=rm)
        d[f"gelu_{name}"] = O.linear_a8_w8_bfp32_ofp32_GeLu_Q(a, w, bf, ag, bg, round_mode=rm)
    d["of32"] = O.linear_a8_w8_bfp32_ofp32(a, w, bf, np.float32(0.0037), np.float32(1.0))
    d["of16"] = O.linear_a8_w8_bfp32_ofp32(a, w, bf, np.float32(0.0037), np.float32(1.0), out_dtype=O.DT_F16)
    d["obf16"] = O.linear_a8_w8_bfp32_ofp32(a, w, bf, np.float32(0.0037), np.float32(1.0), out_dtype=O.DT_BF16)
    # |acc| > 2^24: K = 2048 of +-127
    ka = np.full((4, 2048), 127, np.int8); kw = np.full((6, 2048), 127, np.int8); kw[1::2] = -128
    d["big_a"], d["big_w"] = ka, kw
    d["big_o32"] = O.linear_a8_w8_b32_o32(ka, kw, None)
    d["big_of32"] = O.linear_a8_w8_ofp32(ka, kw, np.float32(1.0))
    return d


def bmm_case():
    g = np.random.default_rng(102)
    B, M, N, K = 3, 40, 24, 72
    a = g.integers(-127, 128, size=(B, M, K), dtype=np.int8)
    b = g.integers(-127, 128, size=(B, N, K), dtype=np.int8)
    alpha = np.float32(1e-3)
    return dict(a=a, b=b, alpha=alpha, s32=O.bmm_s8t_s8n_s32t(a, b), s8=O.bmm_s8t_s8n_s8t(a, b, alpha),
                f32=O.bmm_s8t_s8n_f32t(a, b, alpha))


def rows_case():
    g = np.random.default_rng(103)
    d = {}
    for cols in (128, 768, 5120):
        x = (g.standard_normal((6, cols)) * 1.5 + 0.25).astype(np.float32)
        x[0] = 5.0                      # constant row: var = 0 -> eps path
        x[1] += np.float32(1e4)         # large offset
        w = (g.normal(1.0, 0.1, cols) / 0.05).astype(np.float32)
        b = (g.normal(0.0, 0.1, cols) / 0.05).astype(np.float32)
        y, mean, rstd = O.layernorm_q(x, w, b, 1e-5, return_stats=True)
        d.update({f"x{cols}": x, f"w{cols}": w, f"b{cols}": b, f"y{cols}": y, f"mean{cols}": mean, f"rstd{cols}": rstd})
    cols = 768
    acc = g.integers(-2**20, 2**20 + 1, size=(5, cols), dtype=np.int32)
    acc[0, :2] = [2**20, -2**20]
    res = g.standard_normal((5, cols)).astype(np.float32)
    rout, q, ln, mean, rstd = O.dq_add_layernorm_q(acc, 1e-5, res, d["w768"], d["b768"], 1e-5, return_all=True)
    d.update(dq_acc=acc, dq_res=res, dq_rout=rout, dq_q=q, dq_ln=ln, dq_mean=mean, dq_rstd=rstd)
    gx = np.linspace(-8, 8, 4001).astype(np.float32)
    d.update(gelu_x=gx, gelu_scale=np.float32(20.0), gelu_y=O.gelu_q(gx, np.float32(20.0)))
    return d


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "gemm.npz"), **gemm_case())
    np.savez_compressed(os.path.join(HERE, "bmm.npz"), **bmm_case())
    np.savez_compressed(os.path.join(HERE, "rows.npz"), **rows_case())
    for f in ("gemm.npz", "bmm.npz", "rows.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
