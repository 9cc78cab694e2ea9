"""GPU parity of the int8 GEMM / BMM kernels against the CPU oracle, called through the package's
launchers (which go through the C ABI).  int32 and scale epilogues must be bit-exact; the GELU
epilogue may differ by 1 LSB where tanh's last ulp decides a rounding tie (rate asserted)."""
import numpy as np
import pytest
import torch

import oracle as O
from tests.util import DEV, cpu, gpu, mismatch_report, rand_i8, rng

pytestmark = pytest.mark.gpu


def _lib():
    from triton_int_amd import _lib as L
    return L


def _configs(M=1, N=None, out8=False, K=None, bias8=True):
    """(index, name) of every kernel configuration that can run M activation rows (and, for the
    persistent kernels with an int8 output, N output columns: they store whole 16-byte segments of a
    row; for the short-K kernel "shortk_..._k<max>", a K of 16..max and, for int8 outputs, neither bias
    nor GELU: bias8=False says the int8 launches have none)"""
    L = _lib()
    n = L.lib().ti_gemm_num_configs()
    out = [(i, L.lib().ti_gemm_config_name(i).decode()) for i in range(n)]
    def fits(nm):  # "skinny_m<rows>_..." configurations take at most <rows> activation rows
        if nm.startswith(("skinny", "rows4")):
            return M <= int(nm.split("_")[1][1:])
        if nm.startswith("shortk_") and (not (K is not None and 16 <= K <= int(nm.rsplit("_k", 1)[1])) or (out8 and bias8)):
            return False
        if nm.startswith(("stream", "ws_", "shortk_")) and out8:
            return N is not None and N % 16 == 0
        return True
    return [(i, nm) for i, nm in out if fits(nm)]


def _kl():
    from triton_int_amd.kernels import linear, bmm, fused
    return linear, bmm, fused


# shapes: (M, N, K); all K % 16 == 0 so that every configuration can run them
SHAPES = [(512, 768, 768), (300, 272, 384), (256, 128, 128), (33, 100, 48), (1, 16, 16), (700, 130, 1040)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_all_configs_int32_bit_exact(shape):
    linear, _, _ = _kl()
    M, N, K = shape
    g = rng(M * 7 + N)
    a, w = rand_i8(g, M, K, lo=-128), rand_i8(g, N, K, lo=-128)
    bias = g.integers(-2**24, 2**24, size=N, dtype=np.int32)
    want = O.linear_a8_w8_b32_o32(a, w, bias)
    ga, gw, gb = gpu(a), gpu(w), gpu(bias)
    for cfg, name in _configs(M, K=K):
        got = cpu(linear.linear_a8_w8_b32_o32(ga, gw, gb, _config=cfg))
        assert np.array_equal(got, want), f"config {name}"
    got = cpu(linear.linear_a8_w8_b32_o32(ga, gw, gb))
    assert np.array_equal(got, want), "auto config"


@pytest.mark.parametrize("shape", SHAPES[:4], ids=lambda s: "x".join(map(str, s)))
def test_all_configs_int8_epilogues_bit_exact(shape):
    linear, _, _ = _kl()
    M, N, K = shape
    g = rng(M * 3 + K)
    a, w, bias = rand_i8(g, M, K), rand_i8(g, N, K), rand_i8(g, N)
    ga, gw, gb = gpu(a), gpu(w), gpu(bias)
    std = np.sqrt(K) * 127 * 127 / 3
    for alpha, beta in [(0.0021, 0.013), (40.0 / std, 0.11), (0.5, 1.0)]:  # saturating, spread, exact ties
        want = O.linear_a8_w8_b8_o8(a, w, bias, alpha, beta)
        want_relu = O.linear_relu_a8_w8_b8_o8(a, w, bias, alpha, beta)
        want_tr = O.linear_a8_w8_b8_o8(a, w, bias, alpha, beta, round_mode=O.TRUNC)
        for cfg, name in _configs(M, N, out8=True, K=K):
            got = cpu(linear.linear_a8_w8_b8_o8(ga, gw, gb, alpha, beta, _config=cfg))
            assert np.array_equal(got, want), f"o8 config {name} alpha {alpha}"
            got = cpu(linear.linear_relu_a8_w8_b8_o8(ga, gw, gb, alpha, beta, _config=cfg))
            assert np.array_equal(got, want_relu), f"relu config {name}"
        got = cpu(linear.linear_a8_w8_b8_o8(ga, gw, gb, alpha, beta, _round_mode=1))
        assert np.array_equal(got, want_tr)
        # the literal-Triton truncation differs from the contract by at most 1 on unsaturated values
        assert np.abs(want_tr.astype(int) - want.astype(int)).max() <= 1


@pytest.mark.parametrize("shape", [(300, 272, 384), (16, 1280, 2048), (7, 48, 64), (520, 320, 1040)],
                         ids=lambda s: "x".join(map(str, s)))
def test_grouped_linear_equals_separate_linears(shape):
    """Three projections of one input as one launch (per-projection bias rows and scales): every
    configuration must give, per projection, exactly the single linear's int8 result."""
    linear, _, _ = _kl()
    M, N, K = shape
    g = rng(M * 5 + N)
    G = 3
    a = rand_i8(g, M, K)
    w, bias = rand_i8(g, G * N, K), rand_i8(g, G * N)
    std = np.sqrt(K) * 127 * 127 / 3
    alphas = np.array([0.0021, 40.0 / std, 0.5], dtype=np.float32)
    betas = np.array([0.013, 0.11, 1.0], dtype=np.float32)
    want = np.concatenate([O.linear_a8_w8_b8_o8(a, w[i * N:(i + 1) * N], bias[i * N:(i + 1) * N], alphas[i], betas[i])
                           for i in range(G)], axis=1)
    ga, gw, gb, gal, gbe = gpu(a), gpu(w), gpu(bias), gpu(alphas), gpu(betas)
    ran = set()
    for cfg, name in [(-1, "auto")] + _configs(M, N, out8=True, K=K):
        got = cpu(linear.linear_group_a8_w8_b8_o8(ga, gw, gb, gal, gbe, G, _config=cfg))
        assert got.shape == (M, G * N) and np.array_equal(got, want), f"config {name}"
        ran.add(name.split("_")[0])
    assert {"gather", "mfma", "stream", "ws"} <= ran
    # leading dimensions are kept
    got = cpu(linear.linear_group_a8_w8_b8_o8(ga.view(1, M, K), gw, gb, gal, gbe, G))
    assert got.shape == (1, M, G * N) and np.array_equal(got[0], want)


@pytest.mark.parametrize("shape", SHAPES[:4], ids=lambda s: "x".join(map(str, s)))
def test_all_configs_float_and_scaled_i32(shape):
    linear, _, _ = _kl()
    M, N, K = shape
    g = rng(M + N + K)
    a, w = rand_i8(g, M, K), rand_i8(g, N, K)
    bias_f = g.standard_normal(N).astype(np.float32)
    bias_i = g.integers(-10**6, 10**6, size=N, dtype=np.int32)
    alpha, beta = np.float32(0.0037), np.float32(0.71)
    ga, gw = gpu(a), gpu(w)
    want_f = O.linear_a8_w8_bfp32_ofp32(a, w, bias_f, alpha, beta)
    want_h = O.linear_a8_w8_bfp32_ofp32(a, w, bias_f, alpha, beta, out_dtype=O.DT_F16)
    want_b = O.linear_a8_w8_bfp32_ofp32(a, w, bias_f, alpha, beta, out_dtype=O.DT_BF16)
    want_nb = O.linear_a8_w8_ofp32(a, w, alpha)
    want_s = O.linear_a8_w8_b32_o32_with_scaling(a, w, bias_i, alpha, beta)
    for cfg, name in _configs(M, K=K):
        got = cpu(linear.linear_a8_w8_bfp32_ofp32(ga, gw, gpu(bias_f), alpha, beta, _config=cfg))
        assert got.dtype == np.float32 and np.array_equal(got, want_f), f"f32 {name}"
        got = cpu(linear.linear_a8_w8_bfp32_ofp32(ga, gw, gpu(bias_f), alpha, beta, dtype=torch.float16, _config=cfg))
        assert np.array_equal(got, want_h), f"f16 {name}"
        got = cpu(linear.linear_a8_w8_bfp32_ofp32(ga, gw, gpu(bias_f), alpha, beta, dtype=torch.bfloat16, _config=cfg))
        assert np.array_equal(got, want_b), f"bf16 {name}"
        # a bias given in fp16 / bf16 (the reference's "triton-i8-fp16" / "-bf16" benchmark legs, kernels/linear.py:
        # 1015-1050) sets the output dtype and is widened inside the kernel: the result is that of bias.float()
        for tdt, odt in ((torch.float16, O.DT_F16), (torch.bfloat16, O.DT_BF16)):
            b16 = gpu(bias_f).to(tdt)
            want16 = O.linear_a8_w8_bfp32_ofp32(a, w, b16.float().cpu().numpy(), alpha, beta, out_dtype=odt)
            out16 = linear.linear_a8_w8_bfp32_ofp32(ga, gw, b16, alpha, beta, _config=cfg)
            assert out16.dtype == tdt and np.array_equal(cpu(out16), want16), f"{tdt} bias {name}"
        got = cpu(linear.linear_a8_w8_ofp32(ga, gw, alpha, _config=cfg))
        assert np.array_equal(got, want_nb), f"ofp32 {name}"
        got = cpu(linear.linear_a8_w8_b32_o32_with_scaling(ga, gw, gpu(bias_i), alpha, beta, _config=cfg))
        assert np.array_equal(got, want_s), f"scaled i32 {name}"


def test_half_outputs_paired_and_single_stores():
    """fp16 / bf16 outputs go out as dword pairs where a row keeps pairs aligned (even N, even pitch,
    4-byte aligned base) and element by element otherwise: both ways give the oracle's bits, and the
    columns around a view stay untouched."""
    linear, _, _ = _kl()
    g = rng(77)
    alpha, beta = np.float32(0.0037), np.float32(0.71)
    for (M, N, K, pitch, col0) in ((300, 272, 384, 272, 0),    # pairs
                                  (300, 273, 384, 273, 0),    # odd N: single elements
                                  (300, 272, 384, 281, 0),    # odd pitch
                                  (300, 272, 384, 280, 3),    # view starting at an odd element
                                  (300, 272, 384, 280, 4),    # view at an even element: pairs inside a wider matrix
                                  (513, 130, 128, 130, 0)):
        a, w = rand_i8(g, M, K), rand_i8(g, N, K)
        bias_f = g.standard_normal(N).astype(np.float32)
        ga, gw, gb = gpu(a), gpu(w), gpu(bias_f)
        for dt, odt in ((torch.float16, O.DT_F16), (torch.bfloat16, O.DT_BF16)):
            want = O.linear_a8_w8_bfp32_ofp32(a, w, bias_f, alpha, beta, out_dtype=odt)
            for cfg, name in [(-1, "auto")] + _configs(M, K=K):
                wide = torch.zeros((M, pitch), dtype=dt, device=DEV)
                linear.linear_a8_w8_bfp32_ofp32(ga, gw, gb, alpha, beta, dtype=dt, out=wide[:, col0:col0 + N], _config=cfg)
                got = wide.view(torch.int16).cpu().numpy().view(np.uint16)
                assert np.array_equal(got[:, col0:col0 + N], want.view(np.uint16)), f"{(M, N, K, pitch, col0)} {dt} {name}"
                assert not got[:, :col0].any() and not got[:, col0 + N:].any(), f"outside the view: {(M, N, K, pitch, col0)} {name}"


@pytest.mark.parametrize("shape", SHAPES[:3], ids=lambda s: "x".join(map(str, s)))
def test_all_configs_gelu_q(shape):
    _, _, fused = _kl()
    M, N, K = shape
    g = rng(K)
    a, w = rand_i8(g, M, K), rand_i8(g, N, K)
    bias = g.standard_normal(N).astype(np.float32)
    alpha = np.float32(3.0 / (np.sqrt(K) * 127 * 127 / 3))
    beta = np.float32(1 / 0.05)
    want = O.linear_a8_w8_bfp32_ofp32_GeLu_Q(a, w, bias, alpha, beta)
    assert np.unique(want).size > 100  # the case really exercises the rounding, not only the clamp
    ga, gw, gb = gpu(a), gpu(w), gpu(bias)
    for cfg, name in _configs(M, N, out8=True, K=K):
        got = cpu(fused.linear_a8_w8_bfp32_ofp32_GeLu_Q(ga, gw, gb, alpha, beta, _config=cfg))
        mx, rate = mismatch_report(got, want)
        assert mx <= 1 and rate < 1e-3, f"{name}: max {mx} rate {rate}"


def test_scales_given_as_fp16_fp64_or_host_tensors():
    """The launchers convert a scale tensor that is not fp32 on the device; both converted copies
    must be alive at the launch (alpha != beta shows a copy that was freed and re-used)."""
    linear, bmm, _ = _kl()
    g = rng(77)
    a, w, bias = rand_i8(g, 96, 256), rand_i8(g, 80, 256), rand_i8(g, 80)
    ga, gw, gb = gpu(a), gpu(w), gpu(bias)
    for alpha, beta in [(0.00390625, 0.25), (0.001953125, 0.75)]:  # exact in fp16
        want = O.linear_a8_w8_b8_o8(a, w, bias, alpha, beta)
        for mk in (lambda v: torch.tensor(v, dtype=torch.float16, device=DEV),
                   lambda v: torch.tensor(v, dtype=torch.float64, device=DEV),
                   lambda v: torch.tensor(v, dtype=torch.float32),          # host tensor
                   lambda v: torch.tensor([v], dtype=torch.bfloat16, device=DEV)):
            got = cpu(linear.linear_a8_w8_b8_o8(ga, gw, gb, mk(alpha), mk(beta)))
            assert np.array_equal(got, want)
    bf = g.standard_normal(80).astype(np.float32)
    got = cpu(linear.linear_a8_w8_bfp32_ofp32(ga, gw, gpu(bf), torch.tensor(0.001953125, dtype=torch.float16, device=DEV),
                                              torch.tensor(0.75, dtype=torch.float64, device=DEV)))
    np.testing.assert_array_equal(got, O.linear_a8_w8_bfp32_ofp32(a, w, bf, 0.001953125, 0.75))


def test_extreme_accumulators_over_2p24():
    linear, _, _ = _kl()
    K = 2048
    a = np.full((40, K), 127, np.int8)
    w = np.full((48, K), 127, np.int8)
    w[1::2] = -128
    want = O.linear_a8_w8_b32_o32(a, w, None)
    assert want.max() == K * 127 * 127
    got = cpu(linear.linear_a8_w8_b32_o32(gpu(a), gpu(w), None))
    assert np.array_equal(got, want)
    # int32 -> fp32 conversion must round to nearest even, like the oracle's
    wantf = O.linear_a8_w8_ofp32(a, w, np.float32(1.0))
    gotf = cpu(linear.linear_a8_w8_ofp32(gpu(a), gpu(w), 1.0))
    assert np.array_equal(gotf, wantf)


def test_bmm_layouts_strides_and_batch():
    _, bmm, _ = _kl()
    g = rng(5)
    B, M, N, K = 3, 40, 24, 72
    a_big = rand_i8(g, B, M, K + 8)
    b = rand_i8(g, B, N, K)
    a_np = a_big[:, :, 4:4 + K]
    ga = gpu(a_big)[:, :, 4:4 + K]          # non-contiguous, unaligned rows -> gather kernel
    gb = gpu(b)
    gb_kn = gpu(np.ascontiguousarray(b.transpose(0, 2, 1)))
    want32 = O.bmm_s8t_s8n_s32t(a_np, b)
    assert np.array_equal(cpu(bmm.bmm_s8t_s8n_s32t(ga, gb)), want32)
    assert np.array_equal(cpu(bmm.bmm_s8t_s8t_s32t(ga, gb_kn)), want32)
    alpha = np.float32(1e-3)
    want8 = O.bmm_s8t_s8n_s8t(a_np, b, alpha)
    assert np.array_equal(cpu(bmm.bmm_s8t_s8n_s8t(ga, gb, float(alpha))), want8)
    assert np.array_equal(cpu(bmm.bmm_s8t_s8t_s8t(ga, gb_kn, gpu(np.array(alpha)))), want8)
    wantf = O.bmm_s8t_s8n_f32t(a_np, b, alpha)
    assert np.array_equal(cpu(bmm.bmm_s8t_s8n_f32t(ga, gb, alpha)), wantf)
    got16 = bmm.bmm_s8t_s8n_f32t(ga, gb, alpha, dtype=torch.float16)
    assert got16.dtype == torch.float16
    assert np.array_equal(cpu(got16), O.bmm_s8t_s8n_f32t(a_np, b, alpha, out_dtype=O.DT_F16))


@pytest.mark.parametrize("B,M,N,K", [(5, 256, 384, 128), (2, 300, 200, 64), (7, 64, 64, 256)])
def test_bmm_fast_path_all_configs(B, M, N, K):
    _, bmm, _ = _kl()
    g = rng(B * M)
    a, b = rand_i8(g, B, M, K), rand_i8(g, B, N, K)
    ga, gb = gpu(a), gpu(b)
    want32 = O.bmm_s8t_s8n_s32t(a, b)
    alpha = np.float32(1e-3)
    want8 = O.bmm_s8t_s8n_s8t(a, b, alpha)
    wantf = O.bmm_s8t_s8n_f32t(a, b, alpha)
    out8_ok = {c for c, _ in _configs(M, N, out8=True, K=K, bias8=False)}
    for cfg, name in _configs(M, K=K):
        assert np.array_equal(cpu(bmm.bmm_s8t_s8n_s32t(ga, gb, _config=cfg)), want32), name
        if cfg in out8_ok:
            assert np.array_equal(cpu(bmm.bmm_s8t_s8n_s8t(ga, gb, alpha, _config=cfg)), want8), name
        assert np.array_equal(cpu(bmm.bmm_s8t_s8n_f32t(ga, gb, alpha, _config=cfg)), wantf), name


# The persistent kernels walk several tiles per workgroup with the operand loads of the next tile
# in flight during the epilogue of the current one: these shapes give every workgroup more than
# one tile (more than 768 tiles of 128x128, more than 256 of 256x256), ragged in M, N and K, with
# one, two and many k-tiles per tile.
@pytest.mark.parametrize("B,M,N,K", [(80, 500, 464, 48), (80, 500, 464, 128), (72, 520, 496, 400), (1, 4100, 4368, 208)])
def test_stream_configs_many_tiles_per_workgroup(B, M, N, K):
    _, bmm, _ = _kl()
    g = rng(B + M + K)
    a, b = rand_i8(g, B, M, K), rand_i8(g, B, N, K)
    ga, gb = gpu(a), gpu(b)
    want32 = O.bmm_s8t_s8n_s32t(a, b)
    alpha = np.float32(2.5 / (np.sqrt(K) * 127 * 127 / 3))
    want8 = O.bmm_s8t_s8n_s8t(a, b, alpha)
    wantf = O.bmm_s8t_s8n_f32t(a, b, alpha)
    ran = 0
    for cfg, name in _configs(M, N, out8=True, K=K, bias8=False):
        if not name.startswith(("stream", "ws_", "shortk_")):
            continue
        ran += 1
        assert np.array_equal(cpu(bmm.bmm_s8t_s8n_s32t(ga, gb, _config=cfg)), want32), name
        assert np.array_equal(cpu(bmm.bmm_s8t_s8n_s8t(ga, gb, alpha, _config=cfg)), want8), name
        assert np.array_equal(cpu(bmm.bmm_s8t_s8n_f32t(ga, gb, alpha, _config=cfg)), wantf), name
    assert ran >= 1


def test_odd_k_and_unaligned_fall_back_to_gather():
    linear, _, _ = _kl()
    g = rng(77)
    for (M, N, K) in [(37, 29, 50), (64, 64, 1), (5, 3, 129)]:
        a, w = rand_i8(g, M, K), rand_i8(g, N, K)
        want = O.linear_a8_w8_b32_o32(a, w, None)
        got = cpu(linear.linear_a8_w8_b32_o32(gpu(a), gpu(w), None))
        assert np.array_equal(got, want), (M, N, K)
    # a fast configuration must refuse what it cannot run, not compute garbage
    a, w = rand_i8(g, 8, 50), rand_i8(g, 8, 50)
    with pytest.raises(AssertionError):
        linear.linear_a8_w8_b32_o32(gpu(a), gpu(w), None, _config=1)


def test_k_zero_empty_and_errors():
    linear, bmm, _ = _kl()
    a = torch.zeros((4, 0), dtype=torch.int8, device=DEV)
    w = torch.zeros((6, 0), dtype=torch.int8, device=DEV)
    bias = torch.arange(6, dtype=torch.int32, device=DEV)
    got = cpu(linear.linear_a8_w8_b32_o32(a, w, bias))
    assert np.array_equal(got, np.tile(np.arange(6, dtype=np.int32), (4, 1)))
    assert linear.linear_a8_w8_b32_o32(torch.zeros((0, 16), dtype=torch.int8, device=DEV),
                                       torch.zeros((6, 16), dtype=torch.int8, device=DEV), None).shape == (0, 6)
    with pytest.raises(AssertionError, match="Incompatible dimensions"):
        linear.linear_a8_w8_b32_o32(torch.zeros((4, 16), dtype=torch.int8, device=DEV),
                                    torch.zeros((4, 32), dtype=torch.int8, device=DEV), None)
    with pytest.raises(AssertionError):
        bmm.bmm_s8t_s8n_s32t(torch.zeros((2, 4, 16), dtype=torch.int8, device=DEV),
                             torch.zeros((3, 4, 16), dtype=torch.int8, device=DEV))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        linear.linear_a8_w8_b32_o32(torch.zeros((4, 16), dtype=torch.int8), torch.zeros((4, 16), dtype=torch.int8), None)


def test_out_argument_and_leading_dims():
    linear, _, _ = _kl()
    g = rng(9)
    a, w, bias = rand_i8(g, 2, 3, 5, 64), rand_i8(g, 48, 64), rand_i8(g, 48)
    want = O.linear_a8_w8_b8_o8(a, w, bias, 0.002, 0.1)
    out = torch.empty((30, 48), dtype=torch.int8, device=DEV)
    got = linear.linear_a8_w8_b8_o8(gpu(a), gpu(w), gpu(bias), 0.002, 0.1, out=out)
    assert got.shape == (2, 3, 5, 48)
    assert got.data_ptr() == out.data_ptr()
    assert np.array_equal(cpu(got), want)


def test_baseline_config1_single_w8a8b8o8_linear():
    """x int8 [512,768], W int8 [768,768], bias int8 [768], alpha=0.0021, beta=0.013."""
    from triton_int_amd.nn.linear import W8A8B8O8Linear
    g = rng(2024)
    x, w, bias = rand_i8(g, 512, 768), rand_i8(g, 768, 768), rand_i8(g, 768)
    m = W8A8B8O8Linear(768, 768, alpha=0.0021, beta=0.013)
    m.weight, m.bias = torch.from_numpy(w), torch.from_numpy(bias)
    m = m.to(DEV)
    got = cpu(m(gpu(x)))
    want = O.linear_a8_w8_b8_o8(x, w, bias, 0.0021, 0.013)
    assert np.array_equal(got, want)
    # the CPU emulation path the baseline names: int32 matmul + the same scaling
    acc = torch.matmul(torch.from_numpy(x).to(torch.int32), torch.from_numpy(w).to(torch.int32).T)
    emu = torch.clamp(torch.round(torch.tensor(0.0021) * acc.float() + torch.tensor(0.013) * torch.from_numpy(bias).float()), -128, 127)
    assert np.array_equal(got, emu.to(torch.int8).numpy())
    # how much of this mandated case is decided by the clamp alone
    sat = float(((want == 127) | (want == -128)).mean())
    assert 0.3 < sat < 0.9


@pytest.mark.parametrize("which", ["qkv", "fc1_gelu", "fc2"])
def test_baseline_config2_opt67b_shapes_sampled_rows(which):
    """Full OPT-6.7B shapes at M=2048 on the GPU; the oracle checks 24 sampled rows (rows are
    independent) plus int32 linearity over the whole output."""
    linear, _, fused = _kl()
    g = rng({"qkv": 1, "fc1_gelu": 2, "fc2": 3}[which])
    M = 2048
    K, N = {"qkv": (4096, 4096), "fc1_gelu": (4096, 16384), "fc2": (16384, 4096)}[which]
    x, w = rand_i8(g, M, K), rand_i8(g, N, K)
    alpha = np.float32(g.uniform(1e-3, 1e-2)); beta = np.float32(g.uniform(1e-3, 1e-2))
    rows = np.sort(g.choice(M, size=24, replace=False))
    gx, gw = gpu(x), gpu(w)
    if which == "qkv":
        bias = rand_i8(g, N)
        got = cpu(linear.linear_a8_w8_b8_o8(gx, gw, gpu(bias), alpha, beta))
        assert np.array_equal(got[rows], O.linear_a8_w8_b8_o8(x[rows], w, bias, alpha, beta))
        # non-saturating scale so that rounding is exercised, not only the clamp
        a2 = np.float32(40.0 / (np.sqrt(K) * 127 * 127 / 3))
        got2 = cpu(linear.linear_a8_w8_b8_o8(gx, gw, gpu(bias), a2, beta))
        want2 = O.linear_a8_w8_b8_o8(x[rows], w, bias, a2, beta)
        assert np.unique(want2).size > 200 and np.array_equal(got2[rows], want2)
    elif which == "fc1_gelu":
        bias = g.standard_normal(N).astype(np.float32)
        a2 = np.float32(3.0 / (np.sqrt(K) * 127 * 127 / 3)); b2 = np.float32(20.0)
        got = cpu(fused.linear_a8_w8_bfp32_ofp32_GeLu_Q(gx, gw, gpu(bias), a2, b2))
        mx, rate = mismatch_report(got[rows], O.linear_a8_w8_bfp32_ofp32_GeLu_Q(x[rows], w, bias, a2, b2))
        print(f"GELU-Q fc1: max diff {mx}, mismatch rate {rate:.2e}")
        assert mx <= 1 and rate < 1e-3
    else:
        bias = g.standard_normal(N).astype(np.float32)
        got = cpu(linear.linear_a8_w8_bfp32_ofp32(gx, gw, gpu(bias), alpha, 1.0))
        want = O.linear_a8_w8_bfp32_ofp32(x[rows], w, bias, alpha, 1.0)
        assert np.array_equal(got[rows], want)
    # size-independent property over the whole output: acc(x1 + x2) == acc(x1) + acc(x2) in int32
    x1 = rand_i8(g, M, K, lo=-60, hi=60); x2 = rand_i8(g, M, K, lo=-60, hi=60)
    s = cpu(linear.linear_a8_w8_b32_o32(gpu((x1 + x2).astype(np.int8)), gw, None))
    p1 = cpu(linear.linear_a8_w8_b32_o32(gpu(x1), gw, None)); p2 = cpu(linear.linear_a8_w8_b32_o32(gpu(x2), gw, None))
    assert np.array_equal(s, p1 + p2)


@pytest.mark.parametrize("M,N,K", [(16, 5120, 5120), (1, 5120, 5120), (17, 272, 1040), (48, 100, 64), (64, 20480, 5120), (16, 5120, 20480)])
def test_decode_shapes_skinny_kernel(M, N, K):
    """M <= 16 takes a weight-streaming kernel (row pieces, or slabs with K split across waves); up to
    128 rows against a long K take 32 x 128 or 64 x 128 tiles with K split over workgroups; short K the slabs."""
    linear, _, fused = _kl()
    L = _lib()
    g = rng(M * 13 + N)
    a, w = rand_i8(g, M, K, lo=-128), rand_i8(g, N, K, lo=-128)
    b32 = g.integers(-2**20, 2**20, size=N, dtype=np.int32)
    b8 = rand_i8(g, N); bf = g.standard_normal(N).astype(np.float32)
    ga, gw = gpu(a), gpu(w)
    got = cpu(linear.linear_a8_w8_b32_o32(ga, gw, gpu(b32)))
    used = L.lib().ti_gemm_config_name(L.lib().ti_gemm_last_config()).decode()
    assert used.startswith(("skinny", "rows4") if (M <= 16 or K < 1024) else ("ws_32x128" if M <= 32 else "ws_64x128")), used
    assert np.array_equal(got, O.linear_a8_w8_b32_o32(a, w, b32))
    alpha = np.float32(40.0 / (np.sqrt(K) * 127 * 127 / 3)); beta = np.float32(0.05)
    assert np.array_equal(cpu(linear.linear_a8_w8_b8_o8(ga, gw, gpu(b8), alpha, beta)), O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta))
    assert np.array_equal(cpu(linear.linear_a8_w8_b8_o8(ga, gw, gpu(b8), alpha, beta, _round_mode=1)),
                          O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta, round_mode=O.TRUNC))
    assert np.array_equal(cpu(linear.linear_relu_a8_w8_b8_o8(ga, gw, gpu(b8), alpha, beta)), O.linear_relu_a8_w8_b8_o8(a, w, b8, alpha, beta))
    assert np.array_equal(cpu(linear.linear_a8_w8_bfp32_ofp32(ga, gw, gpu(bf), alpha, 1.0)), O.linear_a8_w8_bfp32_ofp32(a, w, bf, alpha, 1.0))
    ag = np.float32(3.0 / (np.sqrt(K) * 127 * 127 / 3))
    mx, rate = mismatch_report(cpu(fused.linear_a8_w8_bfp32_ofp32_GeLu_Q(ga, gw, gpu(bf), ag, 20.0)),
                               O.linear_a8_w8_bfp32_ofp32_GeLu_Q(a, w, bf, ag, np.float32(20.0)))
    assert mx <= 1 and rate < 1e-3


@pytest.mark.parametrize("M,N,K", [(16, 5120, 4096), (16, 4096, 2048 + 48), (5, 2052, 3072), (16, 1024, 1024 + 16)])
def test_decode_kernel_wave_layouts_bit_exact(M, N, K):
    """The M <= 16 kernel with 8 streaming waves x 3 ring stages, 6 x 4 (what the library picks for 6
    or fewer units of 4 weight rows per workgroup) and 4 x 6, and with K split over 2 / 4 / 8 waves
    (forced through bits 8..15 of the configuration argument: low nibble the split, high nibble the
    waves): every layout must give the oracle's bits for int32, int8 and fp32 outputs."""
    linear, _, _ = _kl()
    L = _lib()
    lib = L.lib()
    names = [lib.ti_gemm_config_name(i).decode() for i in range(lib.ti_gemm_num_configs())]
    c = names.index("rows4_m16")
    g = rng(M + N + K)
    a, w = rand_i8(g, M, K, lo=-128), rand_i8(g, N, K, lo=-128)
    b32 = g.integers(-2**20, 2**20, size=N, dtype=np.int32)
    b8 = rand_i8(g, N); bf = g.standard_normal(N).astype(np.float32)
    ga, gw, gb32, gb8, gbf = gpu(a), gpu(w), gpu(b32), gpu(b8), gpu(bf)
    alpha = np.float32(40.0 / (np.sqrt(K) * 127 * 127 / 3)); beta = np.float32(0.05)
    want32 = O.linear_a8_w8_b32_o32(a, w, b32)
    want8 = O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta)
    wantf = O.linear_a8_w8_bfp32_ofp32(a, w, bf, alpha, 1.0)
    per = -(-((N + 3) // 4) // 256)  # units per workgroup
    ran = 0
    for forced in (0, 1, 2, 4, 8, 0x80, 0x60, 0x40):
        fits = ((forced >> 4) in (0, 8) or per <= (forced >> 4)) and ((forced & 15) <= 1 or per <= (8 // (forced & 15)) * 4)
        cfg = c | (forced << 8)
        if not fits:
            with pytest.raises(AssertionError):  # TI_E_COMBO
                linear.linear_a8_w8_b32_o32(ga, gw, gb32, _config=cfg)
            continue
        assert np.array_equal(cpu(linear.linear_a8_w8_b32_o32(ga, gw, gb32, _config=cfg)), want32), hex(forced)
        assert np.array_equal(cpu(linear.linear_a8_w8_b8_o8(ga, gw, gb8, alpha, beta, _config=cfg)), want8), hex(forced)
        assert np.array_equal(cpu(linear.linear_a8_w8_bfp32_ofp32(ga, gw, gbf, alpha, 1.0, _config=cfg)), wantf), hex(forced)
        ran += 1
    assert ran >= 5
    with pytest.raises(AssertionError):
        linear.linear_a8_w8_b32_o32(ga, gw, gb32, _config=c | (3 << 8))
    with pytest.raises(AssertionError):
        linear.linear_a8_w8_b32_o32(ga, gw, gb32, _config=c | (0x50 << 8))


@pytest.mark.parametrize("M,N,K", [(130, 272, 2064), (300, 400, 1040), (64, 400, 4096), (33, 112, 2048), (700, 144, 4112)])
def test_split_k_every_ws_config_bit_exact(M, N, K):
    """K dealt to 2..8 work items per tile (forced through bits 8..15 of the configuration argument):
    int32 partial sums meet in the library's workspace, the last item of a tile stores it.  Integer
    sums, so every split count must give the oracle's bits, twice in a row (the ticket counters must
    be back at zero after a launch), for ragged M / N, a K tail and more splits than k-tiles."""
    linear, _, fused = _kl()
    L = _lib()
    g = rng(M + 3 * N + K)
    a, w = rand_i8(g, M, K, lo=-128), rand_i8(g, N, K, lo=-128)
    b32 = g.integers(-2**20, 2**20, size=N, dtype=np.int32)
    b8 = rand_i8(g, N); bf = g.standard_normal(N).astype(np.float32)
    ga, gw, gb32, gb8, gbf = gpu(a), gpu(w), gpu(b32), gpu(b8), gpu(bf)
    alpha = np.float32(40.0 / (np.sqrt(K) * 127 * 127 / 3)); beta = np.float32(0.05)
    want32 = O.linear_a8_w8_b32_o32(a, w, b32)
    want8 = O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta)
    wantf = O.linear_a8_w8_bfp32_ofp32(a, w, bf, alpha, 1.0)
    ran = 0
    for cfg, name in _configs(M, N, out8=True):
        if not name.startswith("ws_"):
            continue
        for splits in (2, 3, 5, 8, 40):
            forced = cfg | (splits << 8)
            for _ in range(2):
                assert np.array_equal(cpu(linear.linear_a8_w8_b32_o32(ga, gw, gb32, _config=forced)), want32), (name, splits)
                used = L.lib().ti_gemm_last_splits()
                bk = int(name.split("_")[1].split("x")[2])
                assert 1 < used <= min(splits, (K + bk - 1) // bk), (name, splits, used)
                assert np.array_equal(cpu(linear.linear_a8_w8_b8_o8(ga, gw, gb8, alpha, beta, _config=forced)), want8), (name, splits)
                assert np.array_equal(cpu(linear.linear_a8_w8_bfp32_ofp32(ga, gw, gbf, alpha, 1.0, _config=forced)), wantf), (name, splits)
            ran += 1
    assert ran >= 15
    # a configuration that cannot split refuses a forced split; the automatic choice never fails
    with pytest.raises(AssertionError, match="cannot split K"):
        linear.linear_a8_w8_b32_o32(ga, gw, gb32, _config=1 | (2 << 8))
    assert np.array_equal(cpu(linear.linear_a8_w8_b32_o32(ga, gw, gb32)), want32)


def test_split_k_on_two_streams_and_under_graph_capture():
    """Launches on different streams get their own workspace (they may overlap); a launch captured into
    a graph uses the workspace its stream already has and replays correctly."""
    linear, _, _ = _kl()
    L = _lib()
    g = rng(5)
    M, N, K = 128, 1024, 8192  # long enough for the library to split K on its own
    a, w, b32 = rand_i8(g, M, K), rand_i8(g, N, K), g.integers(-2**20, 2**20, size=N, dtype=np.int32)
    ga, gw, gb = gpu(a), gpu(w), gpu(b32)
    want = O.linear_a8_w8_b32_o32(a, w, b32)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    torch.cuda.synchronize()
    for _ in range(4):
        for st in (s1, s2):
            with torch.cuda.stream(st):
                outs.append(linear.linear_a8_w8_b32_o32(ga, gw, gb))
                assert L.lib().ti_gemm_last_splits() > 1
    torch.cuda.synchronize()
    for o in outs:
        assert np.array_equal(cpu(o), want)
    out = torch.empty((M, N), dtype=torch.int32, device=DEV)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s1):
        with torch.cuda.graph(graph, stream=s1):
            linear.linear_a8_w8_b32_o32(ga, gw, gb, out=out)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(cpu(out), want)


def test_split_k_workspaces_of_short_lived_streams_are_released():
    """A caller that creates a stream per request and releases the library's workspace before dropping it
    leaves the device's free memory where it was: 200 streams, each with a split-K launch."""
    linear, _, _ = _kl()
    L = _lib()
    g = rng(6)
    M, N, K = 128, 1024, 8192
    a, w, b32 = rand_i8(g, M, K), rand_i8(g, N, K), g.integers(-2**20, 2**20, size=N, dtype=np.int32)
    ga, gw, gb = gpu(a), gpu(w), gpu(b32)
    want = O.linear_a8_w8_b32_o32(a, w, b32)
    out = torch.empty((M, N), dtype=torch.int32, device=DEV)
    L.release_workspaces(all_streams=True)   # what earlier tests left behind
    # torch hands out streams from a pool it creates on first use, and a new HIP stream takes device memory of
    # its own: create the pool before the reference reading
    pool = [torch.cuda.Stream() for _ in range(64)]
    for st in pool:
        with torch.cuda.stream(st):
            out.zero_()
    torch.cuda.synchronize()
    del pool
    free0 = torch.cuda.mem_get_info()[0]
    slack = 4 << 20
    for i in range(200):
        st = torch.cuda.Stream()
        with torch.cuda.stream(st):
            linear.linear_a8_w8_b32_o32(ga, gw, gb, out=out)
            assert L.lib().ti_gemm_last_splits() > 1
            freed = L.release_workspaces()   # waits for the stream, frees its blocks
        assert freed > 0
        if i % 50 == 0:
            assert np.array_equal(cpu(out), want)
        del st
    torch.cuda.synchronize()
    # 200 workspaces of about 2.3 MB each would be 460 MB
    assert torch.cuda.mem_get_info()[0] >= free0 - slack, "workspaces of released streams still hold device memory"
    # without a release a stream's workspace stays (that is the documented default)
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        linear.linear_a8_w8_b32_o32(ga, gw, gb, out=out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] <= free0 - (1 << 20)
    assert L.release_workspaces(all_streams=True) > 0
    assert np.array_equal(cpu(out), want)


@pytest.mark.parametrize("M,N,K", [(16, 5136, 1104), (9, 400, 2048), (1, 48, 64), (13, 5120, 5120)])
def test_every_skinny_config_ragged_shapes(M, N, K):
    """Each weight-streaming configuration (one or two 16-row slabs per wave) forced on shapes whose
    N is not a multiple of the slab group, whose K has left-over k-steps and a 16-byte tail."""
    linear, _, _ = _kl()
    g = rng(M + N + K)
    a, w = rand_i8(g, M, K, lo=-128), rand_i8(g, N, K, lo=-128)
    b32 = g.integers(-2**20, 2**20, size=N, dtype=np.int32)
    b8 = rand_i8(g, N)
    ga, gw = gpu(a), gpu(w)
    want32 = O.linear_a8_w8_b32_o32(a, w, b32)
    alpha = np.float32(40.0 / (np.sqrt(K) * 127 * 127 / 3)); beta = np.float32(0.05)
    want8 = O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta)
    ran = 0
    for cfg, name in _configs(M):
        if not name.startswith(("skinny", "rows4")):
            continue
        ran += 1
        assert np.array_equal(cpu(linear.linear_a8_w8_b32_o32(ga, gw, gpu(b32), _config=cfg)), want32), name
        assert np.array_equal(cpu(linear.linear_a8_w8_b8_o8(ga, gw, gpu(b8), alpha, beta, _config=cfg)), want8), name
    assert ran >= 4


def test_decode_attention_bmms():
    """16 query tokens against a 2048-long int8 KV, 40 heads of 128 (OPT-13B decode)."""
    _, bmm, _ = _kl()
    g = rng(99)
    H, T, S, D = 40, 16, 2048, 128
    q, k = rand_i8(g, H, T, D), rand_i8(g, H, S, D)
    sc = bmm.bmm_s8t_s8n_s8t(gpu(q), gpu(k), 1e-3)
    assert sc.shape == (H, T, S)
    assert np.array_equal(cpu(sc), O.bmm_s8t_s8n_s8t(q, k, np.float32(1e-3)))
    pr = rand_i8(g, H, T, S, lo=0, hi=127); vt = rand_i8(g, H, D, S)
    out = bmm.bmm_s8t_s8n_f32t(gpu(pr), gpu(vt), 1.0 / 16129)
    assert np.array_equal(cpu(out), O.bmm_s8t_s8n_f32t(pr, vt, np.float32(1.0 / 16129)))
    assert np.array_equal(cpu(bmm.bmm_s8t_s8n_s32t(gpu(pr), gpu(vt))), O.bmm_s8t_s8n_s32t(pr, vt))


@pytest.mark.parametrize("kind,M,N", [("f32", 32768, 16400), ("i8", 65536, 32784)])
def test_outputs_beyond_2_gib(kind, M, N):
    """An output of more than 2^31 bytes: the persistent kernels index it with 32-bit offsets and must
    not be chosen; whatever runs has to address every row correctly.  K is tiny to keep it cheap;
    first, last and random rows are checked against numpy's exact integer product."""
    linear, _, _ = _kl()
    K = 16
    g = rng(M + N)
    a, w = rand_i8(g, M, K), rand_i8(g, N, K)
    ga, gw = gpu(a), gpu(w)
    rows = np.concatenate([np.arange(8), np.arange(M - 8, M), g.integers(0, M, size=16),
                           [2**31 // (N * (4 if kind == "f32" else 1)) + d for d in (-1, 0, 1)]])
    acc = a[rows].astype(np.int32) @ w.astype(np.int32).T
    if kind == "f32":
        bias = g.standard_normal(N).astype(np.float32)
        out = linear.linear_a8_w8_bfp32_ofp32(ga, gw, gpu(bias), 0.01, 1.0)
        want = (np.float32(0.01) * acc.astype(np.float32)) + bias * np.float32(1.0)
        assert out.numel() * 4 > 2**31 and out.dtype == torch.float32
        got = out[torch.from_numpy(rows).to(DEV)].cpu().numpy()
        assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    else:
        bias = rand_i8(g, N)
        out = linear.linear_a8_w8_b8_o8(ga, gw, gpu(bias), 0.002, 0.5)
        want = O.bmm_i8(a[rows][None], w[None], epilogue=O.EPI_SCALE_I8, out_dtype=O.DT_I8, bias=bias,
                        alpha=np.float32(0.002), beta=np.float32(0.5))[0]
        assert out.numel() > 2**31 and out.dtype == torch.int8
        got = out[torch.from_numpy(rows).to(DEV)].cpu().numpy()
        assert np.array_equal(got, want)
    name = _lib().lib().ti_gemm_config_name(_lib().lib().ti_gemm_last_config()).decode()
    assert not name.startswith(("stream", "ws_")), name
    del out
    torch.cuda.empty_cache()


def test_decode_kernel_several_passes_strided_and_16bit_outputs():
    """The M <= 16 weight-streaming kernel where a workgroup needs several passes over K (more than
    32 units of 4 weight rows each: a vocabulary-sized N), with a ragged N, with outputs that are rows
    of a wider matrix or have a non-unit column stride (element-wise stores), and with fp16 / bf16
    outputs (4 elements = one 8-byte store)."""
    linear, _, _ = _kl()
    L = _lib()
    g = rng(99)
    M, N, K = 16, 50272 + 2, 1024
    a, w = rand_i8(g, M, K, lo=-128), rand_i8(g, N, K, lo=-128)
    b32 = g.integers(-2**20, 2**20, size=N, dtype=np.int32)
    b8 = rand_i8(g, N); bf = g.standard_normal(N).astype(np.float32)
    ga, gw = gpu(a), gpu(w)
    got = cpu(linear.linear_a8_w8_b32_o32(ga, gw, gpu(b32)))
    assert L.lib().ti_gemm_config_name(L.lib().ti_gemm_last_config()).decode().startswith("rows4")
    assert np.array_equal(got, O.linear_a8_w8_b32_o32(a, w, b32))
    alpha = np.float32(40.0 / (np.sqrt(K) * 127 * 127 / 3)); beta = np.float32(0.05)
    want8 = O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta)
    assert np.array_equal(cpu(linear.linear_a8_w8_b8_o8(ga, gw, gpu(b8), alpha, beta)), want8)
    # rows of a wider matrix, starting at an odd column (unaligned: element-wise stores)
    wide = torch.zeros((M, N + 7), dtype=torch.int8, device=DEV)
    linear.linear_a8_w8_b8_o8(ga, gw, gpu(b8), alpha, beta, out=wide[:, 3:3 + N])
    assert np.array_equal(cpu(wide)[:, 3:3 + N], want8) and not cpu(wide)[:, :3].any() and not cpu(wide)[:, 3 + N:].any()
    # transposed output (column stride != 1)
    M2, N2, K2 = 7, 644, 2064
    a2, w2 = rand_i8(g, M2, K2), rand_i8(g, N2, K2)
    bf2 = g.standard_normal(N2).astype(np.float32)
    outT = torch.zeros((N2, M2), dtype=torch.float32, device=DEV)
    cfg = [i for i, nm in _configs(M2) if nm.startswith("rows4")][0]
    linear.linear_a8_w8_bfp32_ofp32(gpu(a2), gpu(w2), gpu(bf2), alpha, 1.0, out=outT.t(), _config=cfg)
    assert np.array_equal(cpu(outT).T, O.linear_a8_w8_bfp32_ofp32(a2, w2, bf2, alpha, 1.0))
    # 16-bit outputs
    for dt, odt in ((torch.float16, O.DT_F16), (torch.bfloat16, O.DT_BF16)):
        got16 = cpu(linear.linear_a8_w8_bfp32_ofp32(ga, gw, gpu(bf), alpha, 1.0, dtype=dt))
        assert np.array_equal(got16, O.linear_a8_w8_bfp32_ofp32(a, w, bf, alpha, 1.0, out_dtype=odt))


@pytest.mark.parametrize("M,N,K", [(16, 5120, 20480), (1, 272, 1040), (7, 5124, 1024), (300, 320, 256), (2048, 768, 512), (16, 50272, 1024),
                                   (2048, 5120, 1024), (1000, 4096, 512), (2049, 4100, 256), (513, 640, 128), (4096, 6848, 512)])
def test_linear_with_residual_equals_linear_then_add(M, N, K):
    """ti_linear_i8_residual_f32: the decode kernel's fused add (M <= 16), the persistent kernels' fused add (large
    outputs, whole and ragged tiles) and the GEMM + add-kernel pair give the bits of the fp32 linear followed by an
    fp32 add."""
    linear, _, _ = _kl()
    g = rng(M + N + K)
    a, w = rand_i8(g, M, K), rand_i8(g, N, K)
    bf = g.standard_normal(N).astype(np.float32)
    res = (g.standard_normal((M, N)) * 3).astype(np.float32)
    alpha = np.float32(40.0 / (np.sqrt(K) * 127 * 127 / 3))
    want = O.linear_a8_w8_bfp32_ofp32(a, w, bf, alpha, 1.0) + res
    ga, gw, gb, gr = gpu(a), gpu(w), gpu(bf), gpu(res)
    got = linear.linear_a8_w8_bfp32_ofp32_residual(ga, gw, gb, alpha, 1.0, gr)
    assert got.dtype == torch.float32 and np.array_equal(cpu(got), want)
    assert np.array_equal(cpu(gr), res)  # the residual is left alone
    # into a given buffer, without a bias; an output that is the residual itself is refused
    buf = torch.empty((M, N), dtype=torch.float32, device=DEV)
    got2 = linear.linear_a8_w8_bfp32_ofp32_residual(ga, gw, None, alpha, 1.0, gr, out=buf)
    assert got2.data_ptr() == buf.data_ptr()
    assert np.array_equal(cpu(buf), O.linear_a8_w8_ofp32(a, w, alpha) + res)
    with pytest.raises(AssertionError):
        linear.linear_a8_w8_bfp32_ofp32_residual(ga, gw, None, alpha, 1.0, gr, out=gr)


@pytest.mark.parametrize("S,heads,D,K,T", [(16, 40, 128, 5120, 2048), (1, 8, 64, 1024, 40), (7, 3, 128, 2064, 96), (16, 5, 16, 1040, 16)])
def test_qkv_decode_with_kv_append_equals_grouped_linear_plus_append(S, heads, D, K, T):
    """ti_qkv_decode_i8: projections identical to the grouped launch (hence to three separate linears),
    caches identical to numpy indexing; cache positions before the last S are untouched."""
    linear, _, _ = _kl()
    g = rng(S * 3 + heads + K)
    N = heads * D
    a, w3 = rand_i8(g, S, K), rand_i8(g, 3 * N, K)
    b3 = rand_i8(g, 3 * N)
    al = (g.uniform(0.5, 1.5, 3) * 40.0 / (np.sqrt(K) * 127 * 127 / 3)).astype(np.float32)
    be = g.uniform(0.01, 0.1, 3).astype(np.float32)
    k_cache = g.integers(-128, 128, size=(heads, T, D), dtype=np.int8)
    vt_cache = g.integers(-128, 128, size=(heads, D, T), dtype=np.int8)
    want = np.concatenate([O.linear_a8_w8_b8_o8(a, w3[i * N:(i + 1) * N], b3[i * N:(i + 1) * N], al[i], be[i]) for i in range(3)], axis=1)
    want_k, want_vt = k_cache.copy(), vt_cache.copy()
    want_k[:, T - S:, :] = want[:, N:2 * N].reshape(S, heads, D).transpose(1, 0, 2)
    want_vt[:, :, T - S:] = want[:, 2 * N:].reshape(S, heads, D).transpose(1, 2, 0)
    gk, gvt = gpu(k_cache), gpu(vt_cache)
    got = linear.linear_qkv_decode_a8_w8_b8_o8(gpu(a), gpu(w3), gpu(b3), gpu(al), gpu(be), gk, gvt)
    assert got is not None and np.array_equal(cpu(got), want)
    assert np.array_equal(cpu(gk), want_k) and np.array_equal(cpu(gvt), want_vt)


def test_qkv_decode_declines_what_the_decode_kernel_cannot_take():
    linear, _, _ = _kl()
    g = rng(1)
    a, w3, b3 = rand_i8(g, 32, 1024), rand_i8(g, 3 * 128, 1024), rand_i8(g, 3 * 128)
    s3 = gpu(np.ones(3, np.float32))
    kc, vc = gpu(np.zeros((1, 64, 128), np.int8)), gpu(np.zeros((1, 128, 64), np.int8))
    assert linear.linear_qkv_decode_a8_w8_b8_o8(gpu(a), gpu(w3), gpu(b3), s3, s3, kc, vc) is None       # 32 rows
    assert linear.linear_qkv_decode_a8_w8_b8_o8(gpu(a[:4, :512].copy()), gpu(w3[:, :512].copy()), gpu(b3), s3, s3, kc, vc) is None  # K < 1024
