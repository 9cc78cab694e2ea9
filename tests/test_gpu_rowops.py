"""GPU parity of the row kernels (LayerNormQ, dequant+add+LayerNormQ, GELU-quant) against the
CPU oracle.  fp32 statistics are summed in a different order on the GPU, so int8 outputs may
differ by 1 LSB at rounding ties; the rate is printed and bounded.  Tolerances: row statistics
1e-4, fp32 outputs rtol 1e-5."""
import numpy as np
import pytest
import torch

import oracle as O
from tests.util import DEV, cpu, gpu, mismatch_report, rng

pytestmark = pytest.mark.gpu

STAT_TOL = 1e-4
INT8_MISMATCH_RATE = 2e-4


def _fused():
    from triton_int_amd.kernels import fused
    return fused


def _ln_inputs(g, rows, cols, out_scale=0.05):
    x = (g.standard_normal((rows, cols)) * 1.3 + 0.2).astype(np.float32)
    w = (g.normal(1.0, 0.1, cols) / out_scale).astype(np.float32)
    b = (g.normal(0.0, 0.1, cols) / out_scale).astype(np.float32)
    return x, w, b


@pytest.mark.parametrize("rows,cols", [(64, 128), (33, 768), (128, 5120), (7, 4096), (5, 8192), (3, 20480),
                                       (9, 1023), (4, 7), (2, 1), (16, 2052)])
def test_layernorm_q(rows, cols):
    fused = _fused()
    g = rng(rows * 100 + cols)
    x, w, b = _ln_inputs(g, rows, cols)
    want, wmean, wrstd = O.layernorm_q(x, w, b, 1e-5, return_stats=True)
    got, mean, rstd = fused.layer_norm_fwd_fused_single_pass_q(gpu(x), gpu(w), gpu(b), 1e-5, _return_stats=True)
    assert got.dtype == torch.int8 and got.shape == x.shape
    assert np.allclose(cpu(mean), wmean, rtol=0, atol=STAT_TOL)
    assert np.allclose(cpu(rstd), wrstd, rtol=STAT_TOL, atol=0)
    mx, rate = mismatch_report(cpu(got), want)
    print(f"LayerNormQ [{rows},{cols}]: max diff {mx}, mismatch rate {rate:.2e}")
    assert mx <= 1 and rate <= max(INT8_MISMATCH_RATE, 1.5 / want.size)


def test_layernorm_q_variants_no_bias_rms_trunc_3d():
    fused = _fused()
    g = rng(3)
    x, w, b = _ln_inputs(g, 24, 640)
    x3 = x.reshape(2, 12, 640)
    want = O.layernorm_q(x3, w, None, 1e-5)
    got = cpu(fused.layer_norm_fwd_fused_single_pass_q(gpu(x3), gpu(w), None, 1e-5))
    assert got.shape == (2, 12, 640)
    mx, rate = mismatch_report(got, want)
    assert mx <= 1 and rate <= INT8_MISMATCH_RATE
    want = O.layernorm_q(x, w, None, 1e-5, rms=True)
    mx, rate = mismatch_report(cpu(fused.layer_norm_fwd_fused_single_pass_q(gpu(x), gpu(w), None, 1e-5, True)), want)
    assert mx <= 1 and rate <= INT8_MISMATCH_RATE
    want = O.layernorm_q(x, w, b, 1e-5, round_mode=O.TRUNC)
    mx, rate = mismatch_report(cpu(fused.layer_norm_fwd_fused_single_pass_q(gpu(x), gpu(w), gpu(b), 1e-5, _round_mode=1)), want)
    assert mx <= 1 and rate <= INT8_MISMATCH_RATE
    # dtype check mirrors the reference's assert (kernels/fused.py:344-350)
    with pytest.raises(AssertionError):
        fused.layer_norm_fwd_fused_single_pass_q(gpu(x).half(), gpu(w), gpu(b), 1e-5)


def test_layernorm_constant_rows_exact():
    fused = _fused()
    cols = 5120
    w = np.full(cols, 10.0, np.float32); b = np.full(cols, 3.0, np.float32)
    x = np.full((4, cols), 5.0, np.float32)
    got, mean, rstd = fused.layer_norm_fwd_fused_single_pass_q(gpu(x), gpu(w), gpu(b), 1e-5, _return_stats=True)
    assert np.all(cpu(got) == 3)
    assert np.allclose(cpu(mean), 5.0, atol=1e-5)


def test_baseline_config3_dq_add_layernorm_q_full_size():
    """acc int32 [8192,5120] in [-2^20, 2^20], scale 1e-5, residual N(0,1), gamma N(1,.1)/0.05,
    beta N(0,.1)/0.05, eps 1e-5.  Oracle on 96 sampled rows; the whole residual output is checked
    through its closed form on the GPU side."""
    fused = _fused()
    g = rng(33)
    rows, cols = 8192, 5120
    acc = g.integers(-2**20, 2**20 + 1, size=(rows, cols), dtype=np.int32)
    res = g.standard_normal((rows, cols), dtype=np.float32)
    w = (g.normal(1.0, 0.1, cols) / 0.05).astype(np.float32)
    b = (g.normal(0.0, 0.1, cols) / 0.05).astype(np.float32)
    s = 1e-5
    gacc, gres = gpu(acc), gpu(res)
    rout, q, mean, rstd = fused.dq_add_layernorm_q(gacc, s, gres, gpu(w), gpu(b), 1e-5, _return_stats=True)
    assert rout.dtype == torch.float32 and q.dtype == torch.int8 and rout.shape == (rows, cols)
    # whole-output closed form (un-fused product and sum, each rounded once)
    torch_rout = gres + (torch.tensor(s, dtype=torch.float32, device=DEV) * gacc.to(torch.float32))
    assert torch.equal(rout, torch_rout)
    sel = np.sort(g.choice(rows, size=96, replace=False))
    o_rout, o_q, o_ln, o_mean, o_rstd = O.dq_add_layernorm_q(acc[sel], s, res[sel], w, b, 1e-5, return_all=True)
    assert np.array_equal(cpu(rout)[sel], o_rout)                      # fp32 residual: bit-exact (tolerance rtol 1e-5)
    assert np.allclose(cpu(mean)[sel], o_mean, rtol=0, atol=STAT_TOL)
    assert np.allclose(cpu(rstd)[sel], o_rstd, rtol=STAT_TOL, atol=0)
    mx, rate = mismatch_report(cpu(q)[sel], o_q)
    print(f"dq_add_layernorm_q cfg3: max diff {mx}, mismatch rate {rate:.2e}")
    assert mx <= 1 and rate <= INT8_MISMATCH_RATE
    # un-quantised variant (functional/fused.py:18-24): fp32 LayerNorm output within rtol 1e-5
    from triton_int_amd.functional.fused import dq_add_layernorm
    rout2, ln = dq_add_layernorm(gacc[:256], s, gres[:256], gpu(w), gpu(b), 1e-5)
    o_rout2, _, o_ln2, _, _ = O.dq_add_layernorm_q(acc[:256], s, res[:256], w, b, 1e-5, return_all=True)
    assert np.array_equal(cpu(rout2), o_rout2)
    assert np.allclose(cpu(ln), o_ln2, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("rows,cols", [(17, 768), (5, 1001), (3, 12288), (1, 4)])
def test_dq_add_layernorm_q_shapes(rows, cols):
    fused = _fused()
    g = rng(cols)
    acc = g.integers(-2**20, 2**20 + 1, size=(rows, cols), dtype=np.int32)
    acc.flat[:2] = [2**20, -2**20]
    res = g.standard_normal((rows, cols), dtype=np.float32)
    w = (g.normal(1.0, 0.1, cols) / 0.05).astype(np.float32)
    b = (g.normal(0.0, 0.1, cols) / 0.05).astype(np.float32)
    o_rout, o_q = O.dq_add_layernorm_q(acc, 3e-5, res, w, b, 1e-5)
    rout, q = fused.dq_add_layernorm_q(gpu(acc), 3e-5, gpu(res), gpu(w), gpu(b), 1e-5)
    assert np.array_equal(cpu(rout), o_rout)
    mx, rate = mismatch_report(cpu(q), o_q)
    assert mx <= 1 and rate <= max(INT8_MISMATCH_RATE, 1.5 / o_q.size)
    # the scale as a device tensor is read by the kernel (no host synchronisation): same bits
    s_dev = torch.tensor(3e-5, dtype=torch.float32, device=DEV)
    rout2, q2 = fused.dq_add_layernorm_q(gpu(acc), s_dev, gpu(res), gpu(w), gpu(b), 1e-5)
    assert torch.equal(rout2, rout) and torch.equal(q2, q)
    rout3, q3 = fused.dq_add_layernorm_q(gpu(acc), torch.tensor(3e-5, dtype=torch.float64), gpu(res), gpu(w), gpu(b), 1e-5)
    assert torch.equal(rout3, rout) and torch.equal(q3, q)


@pytest.mark.parametrize("n", [1, 3, 4, 1000, 4099, 2048 * 16384])
def test_gelu_q(n):
    fused = _fused()
    g = rng(n % 1000)
    x = (g.standard_normal(n, dtype=np.float32) * 2.5)
    scale = np.float32(1 / 0.05)
    got = cpu(fused.gelu_q(gpu(x), scale))
    m = min(n, 1 << 22)  # the oracle checks the first 4M elements of the large case
    want = O.gelu_q(x[:m], scale)
    mx, rate = mismatch_report(got[:m], want)
    print(f"GeLu_Q n={n}: max diff {mx}, mismatch rate {rate:.2e}")
    assert mx <= 1 and rate <= max(1e-3, 1.5 / m)
    if n > m:  # size-independent properties on the rest: bounded, monotone in x for x > 0, sign of x for big |x|
        xs, ys = x[m:], got[m:].astype(np.int32)
        assert ys.min() >= -128 and ys.max() <= 127
        assert np.all(ys[xs > 6.4] == 127) and np.all(ys[xs < -6] == 0)
        order = np.argsort(xs[xs > 0][:1 << 20])
        assert np.all(np.diff(ys[xs > 0][:1 << 20][order]) >= 0)


def test_gelu_q_grid_and_module():
    from triton_int_amd.nn.fused import GeLu_Q
    x = np.linspace(-8, 8, 40001).astype(np.float32)
    m = GeLu_Q(alpha=20.0).to(DEV)
    got = cpu(m(gpu(x)))
    want = O.gelu_q(x, np.float32(20.0))
    mx, rate = mismatch_report(got, want)
    assert mx <= 1 and rate < 1e-3


@pytest.mark.parametrize("rows,cols,q_len", [(64, 2048, 0), (48, 2048, 16), (10, 300, 5), (7, 17, 0), (6, 4096, 3), (4, 8192, 0), (5, 1, 0), (9, 1040, 3), (12, 1536, 12)])
def test_softmax_q(rows, cols, q_len):
    fused = _fused()
    g = rng(rows + cols)
    x = g.integers(-128, 128, size=(rows, cols), dtype=np.int8)
    for scale in (0.05, 0.5):
        got = cpu(fused.softmax_q(gpu(x), scale, causal_q_len=q_len))
        want = O.softmax_q(x, scale, causal_q_len=q_len)
        mx, rate = mismatch_report(got, want)
        print(f"softmax_q [{rows},{cols}] q_len {q_len} scale {scale}: max diff {mx}, mismatch rate {rate:.2e}")
        assert mx <= 1 and rate <= max(2e-3, 1.5 / want.size)
        assert got.min() >= 0
    x3 = x.reshape(1, rows, cols)
    assert fused.softmax_q(gpu(x3), 0.05).shape == (1, rows, cols)
    # scale 0 (every unmasked column equally likely) goes through the general kernel
    got = cpu(fused.softmax_q(gpu(x), 0.0, causal_q_len=q_len))
    mx, rate = mismatch_report(got, O.softmax_q(x, 0.0, causal_q_len=q_len))
    assert mx <= 1


@pytest.mark.parametrize("rows,cols", [(2048, 5120), (16, 5120), (1, 128), (70, 33), (64, 64), (129, 257)])
def test_transpose_i8(rows, cols):
    """Pure data movement: the checker is numpy's transpose.  Covers whole tiles, ragged edges,
    unaligned sizes, and the KV-cache form (writing the last `rows` columns of a wider matrix)."""
    fused = _fused()
    g = rng(rows * 3 + cols)
    x = g.integers(-128, 128, size=(rows, cols), dtype=np.int8)
    got = cpu(fused.transpose_i8(gpu(x)))
    assert got.shape == (cols, rows) and np.array_equal(got, x.T)
    # source with a row pitch (a column slice of a wider matrix)
    wide = g.integers(-128, 128, size=(rows, cols + 48), dtype=np.int8)
    got = cpu(fused.transpose_i8(gpu(wide)[:, 16:16 + cols]))
    assert np.array_equal(got, wide[:, 16:16 + cols].T)
    # destination = the last `rows` columns of a [cols, T] cache; the rest must stay untouched
    T = rows + 37
    cache = g.integers(-128, 128, size=(cols, T), dtype=np.int8)
    gc = gpu(cache)
    fused.transpose_i8(gpu(x), out=gc[:, T - rows:])
    want = cache.copy(); want[:, T - rows:] = x.T
    assert np.array_equal(cpu(gc), want)


def _attention_chain_checked(q, k, vt, qk_alpha, score_scale, pv_alpha, q_len):
    """The three-launch chain on the GPU, each stage checked against the oracle applied to that
    stage's own GPU input: scores and context bit-exact, probabilities within one step on rounding
    boundaries.  Returns the chain's context (a device tensor)."""
    from triton_int_amd.kernels import bmm
    fused = _fused()
    gq, gk, gvt = gpu(q), gpu(k), gpu(vt)
    scores = bmm.bmm_s8t_s8n_s8t(gq, gk, qk_alpha)
    assert np.array_equal(cpu(scores), O.bmm_s8t_s8n_s8t(q, k, np.float32(qk_alpha)))
    probs = fused.softmax_q(scores, score_scale, causal_q_len=q_len)
    mx, rate = mismatch_report(cpu(probs), O.softmax_q(cpu(scores), score_scale, causal_q_len=q_len))
    assert mx <= 1 and rate <= max(2e-3, 1.5 / probs.numel()), (mx, rate)
    ctx = bmm.bmm_s8t_s8n_s8t(probs, gvt, pv_alpha)
    assert np.array_equal(cpu(ctx), O.bmm_s8t_s8n_s8t(cpu(probs), vt, np.float32(pv_alpha)))
    return ctx


@pytest.mark.parametrize("BH,S,T,q_len", [(3, 128, 128, 128), (2, 200, 336, 0), (2, 48, 272, 48), (1, 16, 2048, 16),
                                           (2, 300, 300 + 4, 0), (4, 256, 256, 64), (1, 1, 16, 0), (2, 130, 4096, 0),
                                           (3, 384, 2048, 384)])
def test_attention_i8_against_the_three_kernel_chain(BH, S, T, q_len):
    """Fused Q.K^T -> softmax -> P.V.  Its int8 scores are the BMM's and its probabilities the softmax
    kernel's bit for bit (a row's exponentials are summed as integers, so the order in which the
    kernels visit the keys does not matter): the context must EQUAL the three-launch chain's, whose
    stages are checked against the oracle one by one."""
    fused = _fused()
    T = (T + 15) // 16 * 16
    g = rng(BH * 1000 + S + T)
    D = 128
    q = g.integers(-127, 128, size=(BH, S, D), dtype=np.int8)
    k = g.integers(-127, 128, size=(BH, T, D), dtype=np.int8)
    vt = g.integers(-127, 128, size=(BH, D, T), dtype=np.int8)
    seen_nontrivial = False
    for qk_alpha, score_scale, pv_alpha in ((1e-3, 0.05, 1.0 / 127.0), (4e-3, 0.02, 0.03), (-2e-3, 0.5, 0.02)):
        want = _attention_chain_checked(q, k, vt, qk_alpha, score_scale, pv_alpha, q_len)
        got = fused.attention_i8(gpu(q), gpu(k), gpu(vt), qk_alpha, score_scale, pv_alpha, causal_q_len=q_len)
        assert got.shape == (BH, S, D) and torch.equal(got, want), f"alpha {qk_alpha} scale {score_scale}: {int((got != want).sum())} values differ"
        seen_nontrivial = seen_nontrivial or np.unique(cpu(got)).size > 8
    assert seen_nontrivial or T >= 1024  # long rows of random scores spread the probabilities below 1/254


@pytest.mark.parametrize("BH,S,T,q_len", [(40, 16, 2048, 16), (3, 5, 80, 5), (2, 16, 4096, 0), (2, 9, 1040, 9),
                                           (5, 16, 1024, 16), (2, 7, 3008, 7), (1, 16, 16, 16), (3, 2, 2064, 0),
                                           (2, 12, 48, 4)])
def test_attention_i8_few_query_rows(BH, S, T, q_len):
    """16 or fewer query rows per head (decode, short chunks) run the one-workgroup-per-head kernel:
    same checker and same bar as above: equal to the chain."""
    fused = _fused()
    g = rng(BH * 77 + S * 5 + T)
    D = 128
    q = g.integers(-127, 128, size=(BH, S, D), dtype=np.int8)
    k = g.integers(-127, 128, size=(BH, T, D), dtype=np.int8)
    vt = g.integers(-127, 128, size=(BH, D, T), dtype=np.int8)
    for qk_alpha, score_scale, pv_alpha in ((1e-3, 0.05, 1.0 / 127.0), (4e-3, 0.02, 0.03), (2e-3, 0.3, 0.02), (3e-3, 1.5, 0.02)):
        want = _attention_chain_checked(q, k, vt, qk_alpha, score_scale, pv_alpha, q_len)
        out = torch.full((BH, S, D), 77, dtype=torch.int8, device=DEV)
        fused.attention_i8(gpu(q), gpu(k), gpu(vt), qk_alpha, score_scale, pv_alpha, causal_q_len=q_len, out=out)
        assert torch.equal(out, want), f"scale {score_scale}: {int((out != want).sum())} values differ"


def test_attention_i8_strided_views_and_errors():
    fused = _fused()
    g = rng(77)
    S, heads, D, T = 160, 3, 128, 160
    # the layer's layouts: q / k as head views of a [S, heads*D] projection, out head-merged
    qflat = g.integers(-127, 128, size=(S, heads * D), dtype=np.int8)
    kflat = g.integers(-127, 128, size=(T, heads * D), dtype=np.int8)
    vt_wide = g.integers(-127, 128, size=(heads, D, T + 32), dtype=np.int8)
    vt = vt_wide[:, :, :T]
    gq = gpu(qflat).view(S, heads, D).transpose(0, 1)
    gk = gpu(kflat).view(T, heads, D).transpose(0, 1)
    gvt = gpu(vt_wide)[:, :, :T]  # row pitch T + 32
    out = torch.zeros((S, heads * D), dtype=torch.int8, device=DEV)
    fused.attention_i8(gq, gk, gvt, 1e-3, 0.05, 1.0 / 127.0, causal_q_len=S,
                       out=out.view(S, heads, D).transpose(0, 1))
    q3 = qflat.reshape(S, heads, D).transpose(1, 0, 2)
    k3 = kflat.reshape(T, heads, D).transpose(1, 0, 2)
    want = O.attention_i8(np.ascontiguousarray(q3), np.ascontiguousarray(k3), np.ascontiguousarray(vt), 1e-3, 0.05,
                          1.0 / 127.0, causal_q_len=S)
    mx, rate = mismatch_report(cpu(out).reshape(S, heads, D).transpose(1, 0, 2), want)
    assert mx <= 1 and rate < 5e-3
    with pytest.raises(AssertionError):  # head dimension other than 128
        fused.attention_i8(gpu(q3[:, :, :64].copy()), gpu(k3[:, :, :64].copy()), gpu(vt[:, :64].copy()), 1e-3, 0.05, 0.01)
    with pytest.raises(AssertionError):  # the exponent is taken against the row's largest score: the scale must be positive
        fused.attention_i8(gq, gk, gvt, 1e-3, -0.5, 0.01)
    with pytest.raises(AssertionError):
        fused.softmax_q(gpu(np.zeros((4, 32), np.int8)), -0.1)


@pytest.mark.parametrize("rows,cols", [(2048, 5120), (37, 300), (5, 1), (3, 8193), (64, 768), (9, 20480), (2, 40000)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_quantize_per_token_absmax(rows, cols, dtype):
    """Per-token dynamic quantisation: int8 values and scales bit-identical to the oracle's
    restatement of the reference helper, fp32 and fp16, vector and scalar paths."""
    fused = _fused()
    g = rng(rows * 7 + cols)
    x = (g.standard_normal((rows, cols)) * np.logspace(-3, 2, rows)[:, None]).astype(dtype)
    x[rows // 2] = dtype(0.25)
    want_q, want_s = O.quantize_per_token_absmax(x)
    gx = gpu(x)
    q, s = fused.quantize_per_token_absmax(gx)
    assert q.shape == (rows, cols) and s.shape == (rows, 1) and s.dtype == gx.dtype
    bits = (lambda a: a.view(np.uint16)) if dtype == np.float16 else (lambda a: a)  # cpu() returns fp16 as bits
    assert np.array_equal(cpu(s), bits(want_s)) and np.array_equal(cpu(q), want_q)
    assert torch.equal(gx, gpu(x))  # the kernel leaves its input alone
    # the functional helper keeps the reference's side effect
    from triton_int_amd.functional.quantization import dynamic_quantize_activation_per_token_absmax
    q2, s2 = dynamic_quantize_activation_per_token_absmax(gx.view(1, rows, cols))
    assert q2.shape == (1, rows, cols) and s2.shape == (1, rows, 1)
    assert np.array_equal(cpu(q2)[0], want_q) and np.array_equal(gx.float().cpu().numpy(), want_q.astype(np.float32))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_quantize_per_token_division_is_the_true_quotient(dtype):
    """The kernel divides a row by its scale with the reciprocal part of the division hoisted out of the
    elements; the quotients must still be the correctly rounded ones.  20 M elements per dtype against torch's own
    element-wise steps on the GPU (true divisions), rows spanning 60 orders of magnitude, including rows whose
    scale is outside the hoisted form's range (they take the ordinary division), an all-zero row and a row of
    exact ties."""
    fused = _fused()
    rows, cols = 4096, 5120
    gen = torch.Generator(device=DEV).manual_seed(11)
    x = torch.randn((rows, cols), generator=gen, device=DEV, dtype=torch.float32)
    mags = torch.logspace(-30, 30, rows, device=DEV) if dtype == torch.float32 else torch.logspace(-4, 4, rows, device=DEV)
    x = (x * mags[:, None]).to(dtype)
    if dtype == torch.float32:
        x[7] = 0   # (in fp16 the clamp's 1e-8 rounds to 0 and an all-zero row is 0 / 0: not a defined case)
    x[9] = torch.arange(cols, device=DEV).to(dtype) % 255 * 0.5 - 60.0      # k + 0.5 quotients once the scale is 1
    x[9, 0] = 127.0
    if dtype == torch.float32:
        x[11] = x[11].abs() * 0 + 3.0e38
        x[13] = torch.randn(cols, device=DEV) * 1e-38
    # the steps of functional/quantization.py:61-67.  The scale is formed on the CPU: there torch divides by
    # 127, as the kernel and the oracle do, where its GPU kernel for a scalar divisor multiplies by 1 / 127
    max_val = x.abs().max(dim=-1, keepdim=True)[0].cpu()
    max_val = (torch.clamp(max_val, min=1e-8) / 127).to(DEV)
    want = x.clone().div_(max_val).round_().clamp_(-128, 127).to(torch.int8)  # tensor / tensor: true division
    q, s = fused.quantize_per_token_absmax(x)
    assert torch.equal(s, max_val)
    bad = (q != want)
    assert not bad.any(), (int(bad.sum()), bad.nonzero()[:4].tolist())


@pytest.mark.parametrize("S,heads,D,T", [(16, 40, 128, 2048), (48, 4, 128, 80), (70, 3, 64, 100), (1, 2, 16, 5)])
def test_kv_append_i8(S, heads, D, T):
    """Pure data movement: K rows into a head-major cache, V transposed into V^T columns; the
    checker is numpy indexing.  Sources are column slices of a wider matrix, as in the layer."""
    fused = _fused()
    g = rng(S + heads * D + T)
    H = heads * D
    qkv = g.integers(-128, 128, size=(S, 3 * H), dtype=np.int8)
    k_cache = g.integers(-128, 128, size=(heads, T, D), dtype=np.int8)
    vt_cache = g.integers(-128, 128, size=(heads, D, T), dtype=np.int8)
    want_k, want_vt = k_cache.copy(), vt_cache.copy()
    want_k[:, T - S:, :] = qkv[:, H:2 * H].reshape(S, heads, D).transpose(1, 0, 2)
    want_vt[:, :, T - S:] = qkv[:, 2 * H:].reshape(S, heads, D).transpose(1, 2, 0)
    gq, gk, gv = gpu(qkv), gpu(k_cache), gpu(vt_cache)
    fused.kv_append_i8(gq[:, H:2 * H], gq[:, 2 * H:], gk, gv)
    assert np.array_equal(cpu(gk), want_k) and np.array_equal(cpu(gv), want_vt)
    # unaligned sources (a slice that starts at an odd column) take the byte path
    wide = g.integers(-128, 128, size=(S, 2 * H + 1), dtype=np.int8)
    gw = gpu(wide)
    gk, gv = gpu(k_cache), gpu(vt_cache)
    fused.kv_append_i8(gw[:, 1:H + 1], gw[:, H + 1:], gk, gv)
    want_k[:, T - S:, :] = wide[:, 1:H + 1].reshape(S, heads, D).transpose(1, 0, 2)
    want_vt[:, :, T - S:] = wide[:, H + 1:].reshape(S, heads, D).transpose(1, 2, 0)
    assert np.array_equal(cpu(gk), want_k) and np.array_equal(cpu(gv), want_vt)


_FP_KINDS = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


@pytest.mark.parametrize("rows,cols", [(128, 5120), (33, 768), (7, 4096), (5, 8192), (3, 20480), (9, 1023), (4, 7),
                                       (2, 1), (16, 2052), (1, 128)])
@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
def test_layer_norm_fp_and_skip_variants(rows, cols, kind):
    """layer_norm_fwd_fused_single_pass and the two skip variants against the oracle: fp32 outputs
    within rtol 1e-5 (+ 1e-5 absolute for values near zero), fp16 / bf16 outputs at most one step
    of the type apart (the fp32 statistics are summed in another order, which moves a value across a
    rounding boundary now and then; rate bounded).  The skip output is exact given the LayerNorm output."""
    fused = _fused()
    tdt = _FP_KINDS[kind]
    g = torch.Generator().manual_seed(rows * 31 + cols)
    x = (torch.randn((rows, cols), generator=g) * 1.3 + 0.2).to(tdt)
    sk = torch.randn((rows, cols), generator=g).to(tdt)
    w = (torch.randn(cols, generator=g) * 0.1 + 1.0).to(tdt)
    b = (torch.randn(cols, generator=g) * 0.1).to(tdt)
    eps = 1e-5
    eps_eff = max(eps, 1.6e-5) if kind == "f16" else eps  # kernels/fused.py:502-503
    xn, skn, wn, bn = (t.float().numpy() for t in (x, sk, w, b))
    gx, gsk, gw, gb = (t.to(DEV) for t in (x, sk, w, b))
    ulp = {"f32": 2.0 ** -23, "f16": 2.0 ** -10, "bf16": 2.0 ** -7}[kind]

    def check(got, want):
        assert got.dtype == tdt and tuple(got.shape) == want.shape
        got = got.float().cpu().numpy()
        if kind == "f32":
            assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
        else:
            err = np.abs(got - want)
            assert np.all(err <= 1.01 * ulp * np.maximum(np.abs(want), 2.0 ** -14)), err.max()
            assert (err > 0).mean() < 5e-3
        return got

    for rms in (False, True):
        for bias in (gb, None):
            want, _ = O.layer_norm_fp(xn, wn, None if bias is None else bn, eps_eff, rms=rms, kind=kind)
            out = check(fused.layer_norm_fwd_fused_single_pass(gx, gw, bias, eps, rms), want)
            o2, s2 = fused.skip_layer_norm_fwd_fused_single_pass2(gx, gsk, gw, bias, eps, rms)
            assert np.array_equal(o2.float().cpu().numpy(), out)
            # the skip output: exact given this LayerNorm output
            want_skip = O._round_fp(out + skn, kind)
            assert np.array_equal(s2.float().cpu().numpy(), want_skip)
            s1 = fused.skip_layer_norm_fwd_fused_single_pass(gx, gsk, gw, bias, eps, rms)
            assert torch.equal(s1, s2)
    assert torch.equal(gx.cpu(), x) and torch.equal(gsk.cpu(), sk)


def test_layer_norm_fp_views_and_errors():
    fused = _fused()
    g = torch.Generator().manual_seed(5)
    x = torch.randn((2, 9, 256), generator=g)
    w, b = torch.randn(256, generator=g), torch.randn(256, generator=g)
    want, _ = O.layer_norm_fp(x.numpy(), w.numpy(), b.numpy(), 1e-5)
    got = fused.layer_norm_fwd_fused_single_pass(x.to(DEV), w.to(DEV), b.to(DEV), 1e-5)
    assert tuple(got.shape) == (2, 9, 256) and np.allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-5)
    # rows of a wider matrix (row stride 512 elements) and an unaligned column window
    wide = torch.randn((18, 512), generator=g).to(DEV)
    for sl in (slice(0, 256), slice(3, 259)):
        v = wide[:, sl]
        want, _ = O.layer_norm_fp(v.cpu().numpy(), w.numpy(), b.numpy(), 1e-5)
        assert np.allclose(fused.layer_norm_fwd_fused_single_pass(v, w.to(DEV), b.to(DEV), 1e-5).cpu().numpy(), want,
                           rtol=1e-5, atol=1e-5)
    with pytest.raises(AssertionError):  # dtype mismatch between input and weight (kernels/fused.py:494-496)
        fused.layer_norm_fwd_fused_single_pass(x.to(DEV).half(), w.to(DEV), b.to(DEV), 1e-5)
    with pytest.raises(RuntimeError):  # CPU tensors: no fallback
        fused.layer_norm_fwd_fused_single_pass(x, w, b, 1e-5)
    empty = fused.layer_norm_fwd_fused_single_pass(torch.empty((0, 256), device=DEV), w.to(DEV), b.to(DEV), 1e-5)
    assert tuple(empty.shape) == (0, 256)


def test_row_kernels_beyond_2_31_elements():
    """More than 2^31 elements per tensor: element offsets must be 64-bit.  Inputs are generated on
    the device; the head, the 2^31 boundary and the tail are checked against the oracle."""
    fused = _fused()
    n = 2**31 + 4096 + 3
    x = torch.empty(n, dtype=torch.float32, device=DEV)
    gen = torch.Generator(device=DEV).manual_seed(11)
    for s in range(0, n, 2**28):
        x[s:s + 2**28].normal_(0.0, 2.0, generator=gen)
    y = fused.gelu_q(x, 20.0)
    assert y.numel() == n
    for lo, hi in ((0, 4096), (2**31 - 2048, 2**31 + 2048), (n - 4099, n)):
        want = O.gelu_q(x[lo:hi].cpu().numpy(), 20.0)
        mx, rate = mismatch_report(y[lo:hi].cpu().numpy(), want)
        assert mx <= 1 and rate < 2e-3, (lo, mx, rate)
    del y
    cols = 8192
    rows = n // cols  # 262144 full rows
    rows_x = x[:rows * cols].view(rows, cols)
    g = rng(8)
    w = (g.normal(1.0, 0.1, cols) / 0.05).astype(np.float32)
    b = (g.normal(0.0, 0.1, cols) / 0.05).astype(np.float32)
    # a row stride of cols + 4 elements puts the last rows' offsets beyond 2^31 elements
    wide = torch.empty((rows, cols + 4), dtype=torch.float32, device=DEV)
    wide[:, :cols] = rows_x
    del x, rows_x
    xs = wide[:, :cols]
    assert (rows - 1) * (cols + 4) > 2**31
    q = fused.layer_norm_fwd_fused_single_pass_q(xs, gpu(w), gpu(b), 1e-5)
    for lo, hi in ((0, 4), (rows - 4, rows), (rows // 2, rows // 2 + 2)):
        want = O.layernorm_q(xs[lo:hi].cpu().numpy(), w, b, 1e-5)
        mx, rate = mismatch_report(q[lo:hi].cpu().numpy(), want)
        assert mx <= 1 and rate < 2e-3, (lo, mx, rate)
    del wide, q
    torch.cuda.empty_cache()
