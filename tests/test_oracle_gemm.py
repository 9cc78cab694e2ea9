"""Pins for oracle.bmm_i8 (the int8 GEMM/BMM restatement) against independent computations:
python-int brute force, torch int32 matmul, float64 BLAS, closed-form special cases.
None of these re-type the oracle's formula: they use torch's own round/clamp/gelu."""
import math

import numpy as np
import pytest
import torch

import oracle as O


def rng(seed):
    return np.random.default_rng(seed)


def rand_i8(g, *shape, lo=-127, hi=127):
    return g.integers(lo, hi + 1, size=shape, dtype=np.int8)


def brute_acc(a, b):
    """python-int accumulate, a [M,K], b [N,K]"""
    M, K = a.shape
    N = b.shape[0]
    out = [[0] * N for _ in range(M)]
    al, bl = a.tolist(), b.tolist()
    for m in range(M):
        for n in range(N):
            out[m][n] = sum(al[m][k] * bl[n][k] for k in range(K))
    return np.array(out, dtype=np.int64)


def test_acc_brute_force_tiny():
    g = rng(0)
    for (M, N, K) in [(1, 1, 1), (3, 5, 7), (4, 2, 33), (5, 3, 64)]:
        a, b = rand_i8(g, M, K, lo=-128), rand_i8(g, N, K, lo=-128)
        got = O.linear_a8_w8_b32_o32(a, b, None)
        assert got.dtype == np.int32
        assert np.array_equal(got.astype(np.int64), brute_acc(a, b))


def test_acc_vs_torch_int32_and_float64():
    g = rng(1)
    M, N, K = 96, 80, 2048
    a, b = rand_i8(g, M, K), rand_i8(g, N, K)
    got = O.linear_a8_w8_b32_o32(a, b, None)
    t = torch.matmul(torch.from_numpy(a).to(torch.int32), torch.from_numpy(b).to(torch.int32).T).numpy()
    assert np.array_equal(got, t)
    f64 = a.astype(np.float64) @ b.astype(np.float64).T  # exact: |acc| <= 2048*127^2 << 2^53
    assert np.array_equal(got.astype(np.float64), f64)


def test_acc_extreme_magnitude_over_2p24():
    # K=2048 of 127*127 = 33 032 192 > 2^24: the int32->fp32 conversion must round (RNE)
    K = 2048
    a = np.full((2, K), 127, np.int8)
    b = np.full((3, K), 127, np.int8)
    b[1] = -128
    acc = O.linear_a8_w8_b32_o32(a, b, None)
    assert acc[0, 0] == K * 127 * 127 and acc[0, 1] == -K * 127 * 128
    out = O.linear_a8_w8_ofp32(a, b, np.float32(1.0))
    want = torch.from_numpy(acc).to(torch.float32).numpy()  # torch int32->fp32 is RNE
    assert np.array_equal(out, want)
    assert out[0, 0] != acc[0, 0] or float(acc[0, 0]) == float(np.float32(acc[0, 0]))


def test_bias_i32_added_in_integer_domain():
    g = rng(2)
    a, b = rand_i8(g, 7, 40), rand_i8(g, 9, 40)
    bias = g.integers(-2**20, 2**20, size=9, dtype=np.int32)
    got = O.linear_a8_w8_b32_o32(a, b, bias)
    assert np.array_equal(got.astype(np.int64), brute_acc(a, b) + bias.astype(np.int64)[None, :])


def torch_epilogue_o8(acc, bias, alpha, beta):
    """the CPU emulation named by the baseline: alpha*acc.float() + beta*bias.float(), round, clamp"""
    v = torch.tensor(alpha, dtype=torch.float32) * torch.from_numpy(acc).to(torch.float32)
    if bias is not None:
        v = v + torch.tensor(beta, dtype=torch.float32) * torch.from_numpy(bias).to(torch.float32)
    return torch.clamp(torch.round(v), -128, 127).to(torch.int8).numpy(), v.numpy()


@pytest.mark.parametrize("alpha,beta", [(0.0021, 0.013), (0.0004, 0.11), (1.0, 0.0), (0.03, 1.0)])
def test_o8_matches_torch_emulation(alpha, beta):
    g = rng(3)
    M, N, K = 64, 96, 80
    a, b, bias = rand_i8(g, M, K), rand_i8(g, N, K), rand_i8(g, N)
    acc = brute_acc(a, b).astype(np.int32)
    want, v = torch_epilogue_o8(acc, bias, alpha, beta)
    got = O.linear_a8_w8_b8_o8(a, b, bias, alpha, beta)
    assert np.array_equal(got, want)
    got_relu = O.linear_relu_a8_w8_b8_o8(a, b, bias, alpha, beta)
    assert np.array_equal(got_relu, np.maximum(want, 0))
    # the trunc switch: on unsaturated values it is within 1 of the contract and equals torch.trunc
    got_tr = O.linear_a8_w8_b8_o8(a, b, bias, alpha, beta, round_mode=O.TRUNC)
    want_tr = np.clip(np.trunc(v), -128, 127).astype(np.int8)
    assert np.array_equal(got_tr, want_tr)
    assert np.max(np.abs(got_tr.astype(np.int32) - got.astype(np.int32))) <= 1


def test_o8_exact_ties_round_half_even_and_saturation():
    # alpha = 0.5 makes every odd accumulator an exact tie k+0.5 (positive and negative)
    a = np.zeros((1, 16), np.int8)
    a[0, 0] = 1
    vals = np.array([1, 3, 5, 7, -1, -3, -5, -7, 2, -2, 127, -127, 125, -125, 0, 9], np.int8)
    b = np.zeros((16, 16), np.int8)
    b[:, 0] = vals
    got = O.linear_a8_w8_b8_o8(a, b, None, 0.5, 0.0)[0]
    want = [0, 2, 2, 4, 0, -2, -2, -4, 1, -1, 64, -64, 62, -62, 0, 4]  # half-to-even by hand
    assert got.tolist() == want
    # saturation both ways, incl. -128
    a2 = np.full((1, 64), 127, np.int8)
    b2 = np.stack([np.full(64, 127, np.int8), np.full(64, -127, np.int8)])
    got2 = O.linear_a8_w8_b8_o8(a2, b2, None, 1.0, 0.0)[0]
    assert got2.tolist() == [127, -128]
    # -128.5 -> rne = -128 ; -127.5 -> -128 ; 126.5 -> 126 ; 127.5 -> clamp 127
    a3 = np.ones((1, 16), np.int8)
    for target, exp in [(-257, -128), (-255, -128), (253, 126), (255, 127)]:
        b3 = np.zeros((1, 16), np.int8)
        rest = target
        for i in range(16):  # spread the target over entries within +-127
            step = max(-127, min(127, rest))
            b3[0, i] = step
            rest -= step
        assert rest == 0
        assert int(O.linear_a8_w8_b32_o32(a3, b3, None)[0, 0]) == target
        assert int(O.linear_a8_w8_b8_o8(a3, b3, None, 0.5, 0.0)[0, 0]) == exp


def test_identity_scale_reduces_to_acc():
    g = rng(5)
    a, b = rand_i8(g, 8, 4, lo=-5, hi=5), rand_i8(g, 6, 4, lo=-5, hi=5)
    acc = brute_acc(a, b)
    assert np.abs(acc).max() <= 127
    assert np.array_equal(O.linear_a8_w8_b8_o8(a, b, None, 1.0, 0.0).astype(np.int64), acc)
    assert np.array_equal(O.linear_a8_w8_ofp32(a, b, 1.0).astype(np.int64), acc)
    assert np.array_equal(O.linear_a8_w8_b32_o32_with_scaling(a, b, None, 1.0, 0.0).astype(np.int64), acc)


def test_scaled_i32_is_truncation_toward_zero_by_default():
    g = rng(6)
    a, b = rand_i8(g, 16, 64), rand_i8(g, 24, 64)
    bias = g.integers(-50000, 50000, size=24, dtype=np.int32)
    alpha, beta = np.float32(0.37), np.float32(0.011)
    acc = torch.from_numpy(brute_acc(a, b).astype(np.int32))
    v = torch.from_numpy(bias).float() * torch.tensor(beta) + acc.float() * torch.tensor(alpha)
    want = v.to(torch.int32).numpy()  # torch fp->int conversion truncates toward zero
    got = O.linear_a8_w8_b32_o32_with_scaling(a, b, bias, alpha, beta)
    assert np.array_equal(got, want)


def test_fp32_out_matches_torch_and_half_conversions():
    g = rng(7)
    a, b = rand_i8(g, 32, 128), rand_i8(g, 48, 128)
    bias = g.standard_normal(48).astype(np.float32)
    alpha, beta = np.float32(0.0037), np.float32(1.0)
    acc = torch.from_numpy(brute_acc(a, b).astype(np.int32))
    want = torch.from_numpy(bias) * torch.tensor(beta) + acc.float() * torch.tensor(alpha)
    got = O.linear_a8_w8_bfp32_ofp32(a, b, bias, alpha, beta)
    assert np.array_equal(got, want.numpy())
    got16 = O.linear_a8_w8_bfp32_ofp32(a, b, bias, alpha, beta, out_dtype=O.DT_F16)
    assert np.array_equal(got16, want.to(torch.float16).view(torch.int16).numpy().view(np.uint16))
    gotb = O.linear_a8_w8_bfp32_ofp32(a, b, bias, alpha, beta, out_dtype=O.DT_BF16)
    assert np.array_equal(gotb, want.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))


def test_half_conversion_edge_cases():
    # drive the f16/bf16 converters through a 1x1 GEMM with alpha as the value
    vals = [0.0, 1.0, -1.0, 65504.0, 65519.9, 65520.0, 70000.0, 6e-8, 5.96e-8, 2.98e-8, 2.9802322e-8,
            3.1e-8, 6.1e-5, 6.0975e-5, 1e-7, 0.33333334, 1.0009766, 1.00048828125, 1.0014648, 3.3895314e38]
    a = np.ones((1, 1), np.int8); b = np.ones((1, 1), np.int8)
    for v in vals:
        for s in (1.0, -1.0):
            x = np.float32(v * s)
            t = torch.tensor([x])
            h = O.linear_a8_w8_ofp32(a, b, x, out_dtype=O.DT_F16)[0, 0]
            assert h == t.to(torch.float16).view(torch.int16).numpy().view(np.uint16)[0], v
            bf = O.linear_a8_w8_ofp32(a, b, x, out_dtype=O.DT_BF16)[0, 0]
            assert bf == t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)[0], v


def test_gelu_epilogue_vs_torch_gelu_tanh():
    g = rng(8)
    M, N, K = 48, 64, 96
    a, b = rand_i8(g, M, K), rand_i8(g, N, K)
    bias = g.standard_normal(N).astype(np.float32)
    alpha = np.float32(3.0 / (math.sqrt(K) * 127 * 127 / 3))  # x ~ N(0, 3): covers both GELU tails
    beta = np.float32(1.0 / 0.05)
    acc = torch.from_numpy(brute_acc(a, b).astype(np.int32))
    x = acc.float() * torch.tensor(alpha) + torch.from_numpy(bias)
    yf = torch.nn.functional.gelu(x, approximate="tanh") * torch.tensor(beta)
    want = torch.clamp(torch.round(yf), -128, 127).to(torch.int8).numpy()
    got = O.linear_a8_w8_bfp32_ofp32_GeLu_Q(a, b, bias, alpha, beta)
    diff = np.abs(got.astype(np.int32) - want.astype(np.int32))
    # ATen's tanh-gelu groups the cubic differently (x + k*x^3 inside one vectorised expression):
    # identical up to fp32 rounding, so only values on a rounding boundary may differ, by 1.
    assert diff.max() <= 1
    assert (diff != 0).mean() < 2e-3
    near_tie = np.abs((yf.numpy() - np.floor(yf.numpy())) - 0.5) < 1e-3
    assert np.all(near_tie[diff != 0])


def test_bmm_layouts_and_strides():
    g = rng(9)
    B, M, N, K = 3, 40, 24, 72
    a_big = rand_i8(g, B, M, K + 8)
    a = a_big[:, :, 4:4 + K]          # non-contiguous rows
    b = rand_i8(g, B, N, K)
    b_kn = np.ascontiguousarray(b.transpose(0, 2, 1))
    want = np.stack([brute_acc(a[i], b[i]) for i in range(B)]).astype(np.int32)
    assert np.array_equal(O.bmm_s8t_s8n_s32t(a, b), want)
    assert np.array_equal(O.bmm_s8t_s8t_s32t(a, b_kn), want)
    alpha = np.float32(1e-3)
    w8, _ = torch_epilogue_o8(want, None, alpha, 0.0)
    assert np.array_equal(O.bmm_s8t_s8n_s8t(a, b, alpha), w8)
    assert np.array_equal(O.bmm_s8t_s8t_s8t(a, b_kn, alpha), w8)
    wf = (torch.from_numpy(want).float() * torch.tensor(alpha)).numpy()
    assert np.array_equal(O.bmm_s8t_s8n_f32t(a, b, alpha), wf)
    # linear with bias 0 == bmm with batch 1
    assert np.array_equal(O.linear_a8_w8_b32_o32(a[0], b[0], np.zeros(N, np.int32)), want[0])


def test_k_zero_and_empty():
    a = np.zeros((2, 0), np.int8); b = np.zeros((3, 0), np.int8)
    assert np.array_equal(O.linear_a8_w8_b32_o32(a, b, np.array([1, 2, 3], np.int32)), [[1, 2, 3], [1, 2, 3]])
    assert O.linear_a8_w8_b32_o32(np.zeros((0, 4), np.int8), np.zeros((3, 4), np.int8), None).shape == (0, 3)
