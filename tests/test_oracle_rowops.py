"""Pins for the oracle's LayerNormQ, dq+add+LayerNormQ and GELU-quant restatements against
torch's own library routines (the calls the reference's CPU emulation makes:
functional/fused.py:6-15, nn/fused.py:15-22) and against closed forms."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as O


def rng(seed):
    return np.random.default_rng(seed)


def torch_lnq(x, w, b, eps):
    y = F.layer_norm(torch.from_numpy(x), (x.shape[-1],), torch.from_numpy(w), None if b is None else torch.from_numpy(b), eps)
    return y.round().clamp(-128, 127).to(torch.int8).numpy(), y.numpy()


@pytest.mark.parametrize("cols", [1, 7, 128, 768, 5120])
def test_layernorm_q_vs_torch_layer_norm(cols):
    g = rng(cols)
    rows = 33
    x = (g.standard_normal((rows, cols)) * 1.7 + 0.3).astype(np.float32)
    w = (g.normal(1.0, 0.1, cols) / 0.05).astype(np.float32)
    b = (g.normal(0.0, 0.1, cols) / 0.05).astype(np.float32)
    got, mean, rstd = O.layernorm_q(x, w, b, 1e-5, return_stats=True)
    want, yf = torch_lnq(x, w, b, 1e-5)
    # statistics against float64
    x64 = x.astype(np.float64)
    assert np.allclose(mean, x64.mean(1), rtol=0, atol=1e-6)
    assert np.allclose(rstd, 1.0 / np.sqrt(x64.var(1) + 1e-5), rtol=2e-6)
    diff = np.abs(got.astype(np.int32) - want.astype(np.int32))
    assert diff.max() <= 1
    # only values sitting on a rounding boundary may differ (summation-order ulps)
    frac = np.abs(yf - np.floor(yf) - 0.5)
    assert np.all(frac[diff != 0] < 2e-3)
    assert (diff != 0).mean() < 1e-3
    # fp64 layer_norm as the tie-breaker: the oracle must agree with it wherever not near a tie
    y64 = F.layer_norm(torch.from_numpy(x64), (cols,), torch.from_numpy(w).double(), torch.from_numpy(b).double(), 1e-5)
    want64 = y64.round().clamp(-128, 127).to(torch.int8).numpy()
    safe = np.abs(y64.numpy() - np.floor(y64.numpy()) - 0.5) > 1e-3
    assert np.array_equal(got[safe], want64[safe])


def test_layernorm_q_no_bias_and_rms():
    g = rng(11)
    x = g.standard_normal((9, 320)).astype(np.float32) * 3
    w = (g.normal(1.0, 0.1, 320) * 20).astype(np.float32)
    got = O.layernorm_q(x, w, None, 1e-5)
    want, _ = torch_lnq(x, w, None, 1e-5)
    assert np.abs(got.astype(int) - want.astype(int)).max() <= 1 and (got != want).mean() < 1e-3
    # RMSNorm branch (kernels/fused.py:291-292,307-308): mean stays 0, var = mean(x^2)
    got_r, mean, rstd = O.layernorm_q(x, w, None, 1e-5, rms=True, return_stats=True)
    x64 = x.astype(np.float64)
    r64 = 1.0 / np.sqrt((x64 ** 2).mean(1) + 1e-5)
    assert np.all(mean == 0) and np.allclose(rstd, r64, rtol=2e-6)
    y64 = x64 * r64[:, None] * w.astype(np.float64)
    safe = np.abs(y64 - np.floor(y64) - 0.5) > 1e-3
    assert np.array_equal(got_r[safe], np.clip(np.rint(y64), -128, 127).astype(np.int8)[safe])


def test_layernorm_constant_row_and_large_offset():
    cols = 256
    w = np.full(cols, 10.0, np.float32)
    b = np.full(cols, 3.0, np.float32)
    x = np.full((2, cols), 5.0, np.float32)
    got, mean, rstd = O.layernorm_q(x, w, b, 1e-5, return_stats=True)
    assert np.all(mean == 5.0) and np.allclose(rstd, 1 / np.sqrt(1e-5), rtol=1e-6)
    assert np.all(got == 3)  # (x-mean) == 0 exactly -> bias only
    # shift invariance: adding a large representable offset leaves the result unchanged
    g = rng(12)
    base = g.integers(-64, 64, size=(4, cols)).astype(np.float32) / 8  # exact in fp32 after +1e4
    q0 = O.layernorm_q(base, w, b, 1e-5)
    q1 = O.layernorm_q(base + np.float32(1e4), w, b, 1e-5)
    assert np.array_equal(q0, q1)


def test_dq_add_layernorm_q_vs_torch_emulation_calls():
    g = rng(13)
    rows, cols = 17, 5120
    acc = g.integers(-2**20, 2**20 + 1, size=(rows, cols), dtype=np.int32)
    acc[0, :4] = [2**20, -2**20, 0, 1]
    s = 1e-5
    res = g.standard_normal((rows, cols)).astype(np.float32)
    w = (g.normal(1.0, 0.1, cols) / 0.05).astype(np.float32)
    b = (g.normal(0.0, 0.1, cols) / 0.05).astype(np.float32)
    rout, q, ln, mean, rstd = O.dq_add_layernorm_q(acc, s, res, w, b, 1e-5, return_all=True)
    # the emulation's own calls
    t_res = torch.add(torch.from_numpy(res), torch.from_numpy(acc), alpha=s)
    t_ln = F.layer_norm(t_res, (cols,), torch.from_numpy(w), torch.from_numpy(b), 1e-5)
    t_q = t_ln.clamp(-128, 127).round().to(torch.int8).numpy()
    assert np.allclose(rout, t_res.numpy(), rtol=1e-6, atol=1e-7)      # FMA vs mul+add: <= 1 ulp
    assert np.allclose(ln, t_ln.numpy(), rtol=1e-5, atol=2e-5)
    diff = np.abs(q.astype(int) - t_q.astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 1e-3
    # exactness of the un-fused dequant: resid_out == fl(res + fl(s*x))
    p = (np.float32(s) * acc.astype(np.float32)).astype(np.float32)
    assert np.array_equal(rout, res + p)
    x64 = rout.astype(np.float64)
    assert np.allclose(mean, x64.mean(1), atol=1e-6)
    assert np.allclose(rstd, 1 / np.sqrt(x64.var(1) + 1e-5), rtol=2e-6)


def test_dq_add_exact_when_representable():
    # s = 2^-10 and small ints: s*x and the sum are exact, so resid_out - resid_in == s*x exactly
    acc = np.arange(-512, 512, dtype=np.int32).reshape(4, 256)
    res = np.full((4, 256), 0.25, np.float32)
    w = np.ones(256, np.float32); b = np.zeros(256, np.float32)
    rout, _ = O.dq_add_layernorm_q(acc, 2.0 ** -10, res, w, b, 1e-5)
    assert np.array_equal(rout - res, acc.astype(np.float32) * np.float32(2.0 ** -10))


def test_gelu_q_vs_torch_and_closed_forms():
    x = np.linspace(-8, 8, 20001).astype(np.float32)
    scale = np.float32(1 / 0.05)
    got = O.gelu_q(x, scale)
    yf = (F.gelu(torch.from_numpy(x), approximate="tanh") * torch.tensor(scale))
    want = yf.round().clamp(-128, 127).to(torch.int8).numpy()
    diff = np.abs(got.astype(int) - want.astype(int))
    assert diff.max() <= 1
    frac = np.abs(yf.numpy() - np.floor(yf.numpy()) - 0.5)
    assert np.all(frac[diff != 0] < 1e-3)
    # closed forms on the un-quantised value
    one = np.float32(1.0)
    assert O.gelu_f32(np.zeros(1, np.float32), one)[0] == 0.0
    big = np.array([9.0, 20.0, 100.0], np.float32)
    assert np.array_equal(O.gelu_f32(big, one), big)             # tanh saturates to 1: gelu(x) = x
    assert np.all(np.abs(O.gelu_f32(-big, one)) == 0.0)          # and to -1: gelu(-x) = 0
    xs = np.linspace(0.01, 6, 997).astype(np.float32)
    odd = O.gelu_f32(xs, one).astype(np.float64) - O.gelu_f32(-xs, one).astype(np.float64)
    assert np.allclose(odd, xs, rtol=0, atol=1e-6)               # gelu(x) - gelu(-x) = x
    # float64 evaluation of the same closed form
    x64 = xs.astype(np.float64)
    ref = 0.5 * x64 * (1 + np.tanh(np.sqrt(2 / np.pi) * (x64 + 0.044715 * x64 ** 3)))
    assert np.allclose(O.gelu_f32(xs, one), ref, rtol=2e-6, atol=1e-7)
    # saturation of the quantiser
    assert O.gelu_q(np.array([100.0], np.float32), scale)[0] == 127
    assert O.gelu_q(np.array([-0.75], np.float32), np.float32(1000.0))[0] == -128


def test_softmax_q_vs_torch_softmax():
    g = rng(21)
    x = g.integers(-128, 128, size=(37, 300), dtype=np.int8)
    x[0] = 5                      # uniform row
    x[1] = -128; x[1, 17] = 127   # (nearly) one-hot row
    for scale in (0.05, 0.5, 1e-3):
        got = O.softmax_q(x, scale)
        p = torch.softmax(torch.from_numpy(x).float() * scale, dim=-1)
        want = p.mul(127).round().to(torch.int8).numpy()
        diff = np.abs(got.astype(int) - want.astype(int))
        assert diff.max() <= 1 and (diff != 0).mean() < 2e-3
        frac = np.abs(p.numpy() * 127 - np.floor(p.numpy() * 127) - 0.5)
        assert np.all(frac[diff != 0] < 1e-3)          # only rounding boundaries may differ
        assert got.min() >= 0 and got.max() <= 127
    assert np.all(O.softmax_q(x, 0.05)[0] == round(127 / 300))          # uniform row: 127/300 -> 0
    oh = O.softmax_q(x, 0.5)[1]
    assert oh[17] == 127 and oh.sum() == 127
    # causal mask: position i of each group of q rows sees columns 0 .. i + (cols - q)
    q_len, cols = 5, 12
    xs = g.integers(-128, 128, size=(2 * q_len, cols), dtype=np.int8)
    got = O.softmax_q(xs, 0.1, causal_q_len=q_len)
    for r in range(2 * q_len):
        lim = (r % q_len) + (cols - q_len) + 1
        p = torch.softmax(torch.from_numpy(xs[r, :lim]).float() * 0.1, dim=-1).mul(127).round().numpy()
        assert np.abs(got[r, :lim] - p).max() <= 1 and np.all(got[r, lim:] == 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_quantize_per_token_absmax_vs_the_torch_steps(dtype):
    """The oracle against the five torch calls the reference helper makes
    (functional/quantization.py:61-67), executed by torch on the CPU in the tensor's dtype."""
    g = torch.Generator().manual_seed(4)
    t = (torch.randn((37, 300), generator=g) * torch.logspace(-3, 2, 37).unsqueeze(1)).to(dtype)
    t[5] = 0.25  # a constant row: every quotient is exactly 127
    t[6, 7] = 65504.0 if dtype == torch.float16 else 3.0e38
    x = t.clone()
    max_val = x.abs().max(dim=-1, keepdim=True)[0]
    max_val = torch.clamp(max_val, min=1e-8) / 127
    x.div_(max_val).round_().clamp_(-128, 127)
    want_q, want_s = x.to(torch.int8).numpy(), max_val.numpy()
    got_q, got_s = O.quantize_per_token_absmax(t.numpy())
    assert got_s.dtype == want_s.dtype and np.array_equal(got_s, want_s)
    assert np.array_equal(got_q, want_q)
    assert np.abs(got_q[5]).max() == 127 and set(np.unique(got_q[5])) == {127}


def test_round_fp_matches_torch_casts():
    g = torch.Generator().manual_seed(9)
    v = torch.randn(100000, generator=g) * torch.logspace(-6, 6, 100000)
    v[:4] = torch.tensor([0.0, -0.0, 1.00390625, 1.01171875])  # bf16 ties: to even both ways
    assert np.array_equal(O._round_fp(v.numpy(), "bf16"), v.bfloat16().float().numpy())
    assert np.array_equal(O._round_fp(v.numpy(), "f16"), v.half().float().numpy())


@pytest.mark.parametrize("cols", [5, 128, 768, 5120])
@pytest.mark.parametrize("kind,tdt", [("f32", torch.float32), ("f16", torch.float16), ("bf16", torch.bfloat16)])
def test_layer_norm_fp_vs_torch_layer_norm(cols, kind, tdt):
    """The floating-point LayerNorm restatement (kernels/fused.py:385-862) against torch's CPU
    layer_norm on the same (already rounded) inputs, the skip add against torch's add in the
    tensors' dtype, RMSNorm against its closed form in float64."""
    g = torch.Generator().manual_seed(cols)
    rows = 19
    x = (torch.randn((rows, cols), generator=g) * 1.7 + 0.3).to(tdt)
    sk = torch.randn((rows, cols), generator=g).to(tdt)
    w = (torch.randn(cols, generator=g) * 0.1 + 1.0).to(tdt)
    b = (torch.randn(cols, generator=g) * 0.1).to(tdt)
    eps = 1e-5
    xn, skn, wn, bn = (t.float().numpy() for t in (x, sk, w, b))
    out, skip_out = O.layer_norm_fp(xn, wn, bn, eps, skip=skn, kind=kind)
    ref32 = F.layer_norm(x.float(), (cols,), w.float(), b.float(), eps)
    want = ref32.to(tdt).float().numpy()
    ulp = {"f32": 2.0 ** -23, "f16": 2.0 ** -10, "bf16": 2.0 ** -7}[kind]
    # a different summation order moves the fp32 result by a few fp32 ulps: at most one step of the
    # output type, and only where the value sat on a rounding boundary
    err = np.abs(out - want)
    step = ulp * np.maximum(np.abs(want), 2.0 ** -14)
    assert np.all(err <= (8 if kind == "f32" else 1) * step + (1e-6 if kind == "f32" else 0))
    if kind != "f32":
        assert (err > 0).mean() < 5e-3
    # skip add: exact given `out`
    want_skip = (torch.from_numpy(out).to(tdt) + sk).float().numpy()
    assert np.array_equal(skip_out, want_skip)
    # no bias
    out_nb, none = O.layer_norm_fp(xn, wn, None, eps, kind=kind)
    assert none is None
    ref_nb = F.layer_norm(x.float(), (cols,), w.float(), None, eps).to(tdt).float().numpy()
    assert np.all(np.abs(out_nb - ref_nb) <= (8 if kind == "f32" else 1) * ulp * np.maximum(np.abs(ref_nb), 2.0 ** -14) + 1e-6)
    # RMSNorm closed form
    out_r, _ = O.layer_norm_fp(xn, wn, bn, eps, rms=True, kind=kind)
    x64 = xn.astype(np.float64)
    r64 = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps) * wn + bn
    assert np.all(np.abs(out_r - r64) <= 2 * ulp * np.maximum(np.abs(r64), 2.0 ** -14) + 1e-6)


def test_layer_norm_fp_invariants():
    """Constant rows hit the eps path (output = bias), a shifted row normalises to the same values."""
    x = np.full((3, 64), 2.5, np.float32)
    w = np.linspace(0.5, 1.5, 64).astype(np.float32)
    b = np.linspace(-1, 1, 64).astype(np.float32)
    out, _ = O.layer_norm_fp(x, w, b, 1e-5)
    assert np.array_equal(out, np.broadcast_to(b, out.shape))
    g = rng(3)
    y = g.standard_normal((4, 256)).astype(np.float32)
    o1, _ = O.layer_norm_fp(y, w.repeat(4), None, 1e-5)
    o2, _ = O.layer_norm_fp(y + np.float32(8.0), w.repeat(4), None, 1e-5)
    assert np.allclose(o1, o2, rtol=0, atol=2e-5)
