"""The nn modules and functional aliases: buffers, from_float algebra, shapes, and the attention
BMMs at the baseline's OPT-13B shapes (config 4)."""
import numpy as np
import pytest
import torch

import oracle as O
from tests.util import DEV, cpu, gpu, mismatch_report, rand_i8, rng

pytestmark = pytest.mark.gpu


def test_linear_modules_buffers_and_forward():
    from triton_int_amd.nn import linear as nnl
    g = rng(1)
    x = rand_i8(g, 2, 9, 128)
    for cls, bias_dtype in [(nnl.W8A8B8O8Linear, torch.int8), (nnl.W8A8B8O8LinearReLU, torch.int8),
                            (nnl.W8A8B32O32Linear, torch.int32), (nnl.W8A8BFP32OFP32Linear, torch.float32)]:
        m = cls(128, 96, alpha=0.004, beta=0.5)
        sd = m.state_dict()
        assert set(sd) == {"weight", "bias", "a", "b"} and sd["weight"].dtype == torch.int8
        assert sd["bias"].dtype == bias_dtype and sd["a"].ndim == 0
        m = m.to(DEV)
        y = m(gpu(x))
        assert y.shape == (2, 9, 96)
    m = nnl.W8A8BFP32OFP32Linear(128, 96, alpha=0.004, beta=7.0)
    assert float(m.b) == 1.0                       # beta is pinned to 1 (nn/linear.py:244)
    m = m.to(DEV).half()
    assert m.bias.dtype == torch.float32 and m.a.dtype == torch.float32   # stays fp32 under .half()
    m2 = nnl.W8A8B32O32LinearWithoutScaling(128, 96).to(DEV)
    w = cpu(m2.weight)
    assert np.array_equal(cpu(m2(gpu(x))), O.linear_a8_w8_b32_o32(x, w, np.zeros(96, np.int32)))


def test_from_float_scale_algebra():
    from triton_int_amd.nn.linear import W8A8B8O8Linear, W8A8BFP32OFP32Linear
    from triton_int_amd.nn.fused import W8A8BFP32OFP32_GeLu_Q, LayerNormQ
    torch.manual_seed(0)
    lin = torch.nn.Linear(64, 48)
    w0, b0 = lin.weight.detach().clone(), lin.bias.detach().clone()
    q = W8A8B8O8Linear.from_float(lin, input_scale=0.02, output_scale=0.05)
    ws, bs = w0.abs().max() / 127, b0.abs().max() / 127
    assert torch.equal(q.weight, (w0 / ws).round().to(torch.int8))
    assert torch.allclose(q.a, 0.02 * ws / 0.05) and torch.allclose(q.b, bs / 0.05)
    lin = torch.nn.Linear(64, 48)
    b0 = lin.bias.detach().clone(); ws = lin.weight.detach().abs().max() / 127
    q = W8A8BFP32OFP32Linear.from_float(lin, input_scale=0.02)
    assert torch.allclose(q.a, 0.02 * ws) and torch.equal(q.bias, b0) and float(q.b) == 1.0
    lin = torch.nn.Linear(64, 48); ws = lin.weight.detach().abs().max() / 127
    q = W8A8BFP32OFP32_GeLu_Q.from_float(lin, input_scale=0.02, out_scale=0.05)
    assert torch.allclose(q.a, 0.02 * ws) and torch.allclose(q.b, torch.tensor(20.0))
    ln = torch.nn.LayerNorm(64)
    with torch.no_grad():
        ln.weight.normal_(1, 0.1); ln.bias.normal_(0, 0.1)
    qn = LayerNormQ.from_float(ln, 0.05)
    assert torch.allclose(qn.weight, ln.weight / 0.05) and torch.allclose(qn.bias, ln.bias / 0.05)
    # end to end: the quantised pipeline tracks the float module
    x = torch.randn(32, 64)
    qn = qn.to(DEV)
    y8 = qn(x.to(DEV)).cpu().float() * 0.05
    assert (y8 - ln(x)).abs().max() < 0.05


def test_norm_and_gelu_linear_modules():
    from triton_int_amd.nn.fused import DQ_Add_LayerNorm_Q, LayerNormQ, W8A8BFP32OFP32_GeLu_Q, _LayerNormQ
    g = rng(4)
    H = 768
    x = g.standard_normal((2, 5, H), dtype=np.float32)
    w = (g.normal(1, 0.1, H) / 0.05).astype(np.float32); b = (g.normal(0, 0.1, H) / 0.05).astype(np.float32)
    m = LayerNormQ(H)
    m.weight, m.bias = torch.from_numpy(w), torch.from_numpy(b)
    m = m.to(DEV)
    mx, rate = mismatch_report(cpu(m(gpu(x))), O.layernorm_q(x, w, b, 1e-5))
    assert mx <= 1 and rate < 1e-3
    assert _LayerNormQ is LayerNormQ
    d = DQ_Add_LayerNorm_Q(H)
    d.weight, d.bias = torch.from_numpy(w), torch.from_numpy(b)
    d.input_scale = 2e-5
    d = d.to(DEV)
    acc = g.integers(-2**20, 2**20, size=(2, 5, H), dtype=np.int32)
    rout, q = d(gpu(x), gpu(acc))
    o_rout, o_q = O.dq_add_layernorm_q(acc, 2e-5, x, w, b, 1e-5)
    assert rout.shape == (2, 5, H) and np.array_equal(cpu(rout), o_rout)
    mx, rate = mismatch_report(cpu(q), o_q)
    assert mx <= 1 and rate < 1e-3
    fc1 = W8A8BFP32OFP32_GeLu_Q(H, 256, alpha=3.0 / (np.sqrt(H) * 127 * 127 / 3), beta=20.0)
    bias = g.standard_normal(256, dtype=np.float32)
    fc1.bias = torch.from_numpy(bias)
    fc1 = fc1.to(DEV)
    xi = rand_i8(g, 3, 7, H)
    got = cpu(fc1(gpu(xi)))
    want = O.linear_a8_w8_bfp32_ofp32_GeLu_Q(xi, cpu(fc1.weight), bias, np.float32(float(fc1.a)), np.float32(20.0))
    mx, rate = mismatch_report(got, want)
    assert got.shape == (3, 7, 256) and mx <= 1 and rate < 1e-3


def test_bmm_modules_and_functional_aliases():
    from triton_int_amd.nn import bmm as nnb
    from triton_int_amd.functional.bmm import bmm_i8_o8, bmm_i8_o32
    g = rng(6)
    a, b = rand_i8(g, 4, 48, 64), rand_i8(g, 4, 80, 64)
    ga, gb = gpu(a), gpu(b)
    m = nnb.BMM_S8T_S8N_S8T.from_scale(0.02, 0.03, 0.6).to(DEV)
    assert set(m.state_dict()) == {"a"} and abs(float(m.a) - 0.001) < 1e-9
    assert np.array_equal(cpu(m(ga, gb)), O.bmm_s8t_s8n_s8t(a, b, np.float32(float(m.a))))
    m = nnb.BMM_S8T_S8T_S8T(1e-3).to(DEV)
    assert np.array_equal(cpu(m(ga, gb.transpose(1, 2).contiguous())), O.bmm_s8t_s8n_s8t(a, b, np.float32(1e-3)))
    m = nnb.BMM_S8T_S8N_F32T.from_scale(1 / 127, 1 / 127).to(DEV)
    assert np.array_equal(cpu(m(ga, gb)), O.bmm_s8t_s8n_f32t(a, b, np.float32(float(m.a))))
    for cls, dt, odt in [(nnb.BMM_S8T_S8N_F16T, torch.float16, O.DT_F16), (nnb.BMM_S8T_S8N_BF16T, torch.bfloat16, O.DT_BF16)]:
        m = cls(1e-3).to(DEV)
        y = m(ga, gb)
        assert y.dtype == dt and np.array_equal(cpu(y), O.bmm_s8t_s8n_f32t(a, b, np.float32(1e-3), out_dtype=odt))
    assert np.array_equal(cpu(nnb.BMM_S8T_S8N_S32T()(ga, gb)), O.bmm_s8t_s8n_s32t(a, b))
    assert np.array_equal(cpu(bmm_i8_o8(ga, gb, 1e-3)), O.bmm_s8t_s8n_s8t(a, b, np.float32(1e-3)))
    assert np.array_equal(cpu(bmm_i8_o32(ga, gb)), O.bmm_s8t_s8n_s32t(a, b))


def test_baseline_config4_attention_bmms_opt13b_shapes():
    """160 batched matmuls, seq 2048, head_dim 128.  QK^T -> int8 with alpha 1e-3; P.V -> fp32 with
    alpha 1/127^2 and P in [0,127] from a seeded quantised softmax.  The oracle checks sampled
    (batch, row) slices; integer linearity covers the rest."""
    from triton_int_amd.nn.bmm import BMM_S8T_S8N_F32T, BMM_S8T_S8N_S8T
    g = rng(44)
    B, S, D = 160, 2048, 128
    q, k = rand_i8(g, B, S, D), rand_i8(g, B, S, D)
    gq, gk = gpu(q), gpu(k)
    qk = BMM_S8T_S8N_S8T(1e-3).to(DEV)
    scores = qk(gq, gk)
    assert scores.shape == (B, S, S) and scores.dtype == torch.int8
    bsel = [0, 57, 159]
    rsel = np.sort(g.choice(S, size=40, replace=False))
    for bi in bsel:
        want = O.bmm_s8t_s8n_s8t(q[bi:bi + 1, rsel], k[bi:bi + 1], np.float32(1e-3))
        assert np.array_equal(cpu(scores[bi])[rsel], want[0])
    # P.V: probabilities from a seeded fp32 softmax quantised to [0,127]
    gen = torch.Generator(device="cpu").manual_seed(45)
    vt = rand_i8(g, B, D, S)
    gvt = gpu(vt)
    pv = BMM_S8T_S8N_F32T(1.0 / (127 * 127)).to(DEV)
    logits = torch.randn((len(bsel), S, S), generator=gen) * 2.0
    p_small = torch.round(torch.softmax(logits, dim=-1) * 127).to(torch.int8).numpy()
    assert p_small.min() >= 0 and p_small.max() <= 127
    probs = torch.zeros((B, S, S), dtype=torch.int8, device=DEV)
    probs.copy_((torch.softmax(scores.float() * 0.05, dim=-1) * 127).round().to(torch.int8))  # filler for the other batches
    for j, bi in enumerate(bsel):
        probs[bi] = gpu(p_small[j])
    out = pv(probs, gvt)
    assert out.shape == (B, S, D) and out.dtype == torch.float32
    for j, bi in enumerate(bsel):
        want = O.bmm_s8t_s8n_f32t(p_small[j:j + 1, rsel], vt[bi:bi + 1], np.float32(1.0 / (127 * 127)))
        assert np.array_equal(cpu(out[bi])[rsel], want[0])
    # whole-output integer check: acc(P, V) summed over the batch equals a batch-1 product of sums?  No —
    # instead use linearity in V: acc(P, V1 + V2) == acc(P, V1) + acc(P, V2), exact in int32.
    from triton_int_amd.kernels.bmm import bmm_s8t_s8n_s32t
    v1 = rand_i8(g, B, D, S, lo=-60, hi=60); v2 = rand_i8(g, B, D, S, lo=-60, hi=60)
    s12 = bmm_s8t_s8n_s32t(probs, gpu((v1 + v2).astype(np.int8)))
    s1 = bmm_s8t_s8n_s32t(probs, gpu(v1)); s2 = bmm_s8t_s8n_s32t(probs, gpu(v2))
    assert torch.equal(s12, s1 + s2)


def test_registered_torch_ops_dispatch_and_trace():
    """torch.ops.triton_op.* run the same kernels as the launchers, and a function that calls them
    can be captured as one graph (torch.compile with the `eager` backend: tracing only)."""
    from triton_int_amd.kernels import linear
    g = rng(21)
    a, w, b = rand_i8(g, 48, 64), rand_i8(g, 32, 64), rand_i8(g, 32)
    ga, gw, gb = gpu(a), gpu(w), gpu(b)
    sa, sb = torch.tensor(0.003, device=DEV), torch.tensor(0.02, device=DEV)
    want = linear.linear_a8_w8_b8_o8(ga, gw, gb, sa, sb)
    assert torch.equal(torch.ops.triton_op.linear_a8_w8_b8_o8(ga, gw, gb, sa, sb), want)
    assert np.array_equal(cpu(want), O.linear_a8_w8_b8_o8(a, w, b, np.float32(0.003), np.float32(0.02)))

    def f(x):
        y = torch.ops.triton_op.linear_relu_a8_w8_b8_o8(x, gw, gb, sa, sb)
        return torch.ops.triton_op.gelu_q(y.float(), 2.0)

    compiled = torch.compile(f, backend="eager", fullgraph=True)
    assert torch.equal(compiled(ga), f(ga))


def test_dynamic_w8a8_linear_tracks_the_float_module():
    """The dynamically quantised linear (per-tensor absmax of the activation at every call): the
    int8 GEMM and its fp32 epilogue are checked against the oracle on the int8 activations the module
    itself formed from a numpy restatement of the helper, and the result tracks the float module."""
    from triton_int_amd.nn.linear import DanymicW8A8BFP32OFP32Linear, DynamicW8A8BFP32OFP32Linear
    assert DanymicW8A8BFP32OFP32Linear is DynamicW8A8BFP32OFP32Linear
    torch.manual_seed(3)
    lin = torch.nn.Linear(256, 192)
    x = torch.randn(3, 17, 256) * 2.5
    want_float = lin(x).detach()
    q = DynamicW8A8BFP32OFP32Linear.from_float(_clone_linear(lin)).to(DEV)
    gx = x.to(DEV)
    y = q(gx)
    assert y.shape == (3, 17, 192) and y.dtype == torch.float32 and torch.equal(gx.cpu(), x)  # x untouched
    xs = x.numpy().reshape(-1, 256)
    scale = np.float32(np.abs(xs).max()) / np.float32(127)
    x8 = np.rint(xs / scale).astype(np.int8)
    alpha = np.float32(scale * np.float32(float(q.weight_scale)))
    want = O.linear_a8_w8_bfp32_ofp32(x8, cpu(q.weight), cpu(q.bias), alpha, np.float32(1.0))
    assert np.allclose(cpu(y).reshape(-1, 192), want, rtol=1e-5, atol=1e-6)
    assert (y.cpu() - want_float).abs().max() < 0.15  # two 8-bit quantisations of a 256-term sum


def _clone_linear(lin):
    c = torch.nn.Linear(lin.in_features, lin.out_features)
    c.load_state_dict(lin.state_dict())
    return c


def test_reference_usage_through_the_triton_int_import_path():
    """A caller written against the reference runs unchanged: the imports, constructor, buffer
    assignment, `.to()` and forward of triton_int/nn/linear.py:18-54 and triton_int/nn/bmm.py:10-29,
    checked against the oracle."""
    from triton_int.nn.bmm import BMM_S8T_S8N_S8T
    from triton_int.nn.linear import W8A8B8O8Linear, W8A8BFP32OFP32Linear
    from triton_int.kernels.linear import linear_a8_w8_b8_o8
    from triton_int.functional.bmm import bmm_i8_o8
    g = rng(21)
    x = rand_i8(g, 4, 40, 256)
    w, b = rand_i8(g, 192, 256), rand_i8(g, 192)
    m = W8A8B8O8Linear(256, 192, alpha=0.0021, beta=0.013)
    m.weight, m.bias = torch.from_numpy(w), torch.from_numpy(b)
    m = m.to(DEV)
    y = m(gpu(x))
    want = O.linear_a8_w8_b8_o8(x.reshape(-1, 256), w, b, 0.0021, 0.013).reshape(4, 40, 192)
    assert y.shape == (4, 40, 192) and np.array_equal(cpu(y), want)
    assert np.array_equal(cpu(linear_a8_w8_b8_o8(gpu(x), gpu(w), gpu(b), m.a, m.b)), want)
    bf = g.standard_normal(192).astype(np.float32)
    m2 = W8A8BFP32OFP32Linear(256, 192, alpha=0.003)
    m2.weight, m2.bias = torch.from_numpy(w), torch.from_numpy(bf)
    m2 = m2.to(DEV)
    np.testing.assert_array_equal(cpu(m2(gpu(x))),
                                  O.linear_a8_w8_bfp32_ofp32(x.reshape(-1, 256), w, bf, 0.003, 1.0).reshape(4, 40, 192))
    q, k = rand_i8(g, 6, 48, 64), rand_i8(g, 6, 80, 64)
    bmm = BMM_S8T_S8N_S8T(1e-3).to(DEV)
    want_s = O.bmm_s8t_s8n_s8t(q, k, np.float32(1e-3))
    assert np.array_equal(cpu(bmm(gpu(q), gpu(k))), want_s)
    assert np.array_equal(cpu(bmm_i8_o8(gpu(q), gpu(k), 1e-3)), want_s)
