"""The W8A8 OPT-shaped decoder layer chained from the package's kernels.  Each stage is checked
against the oracle on the stage's actual GPU inputs (so a permitted 1-LSB difference in one stage
does not hide or amplify through the next), for a prefill pass and for a decode pass against an
int8 KV cache."""
import numpy as np
import pytest
import torch

import oracle as O
from tests.util import DEV, cpu, gpu, mismatch_report

pytestmark = pytest.mark.gpu


def _check_stages(layer, tr, hidden_np, B, S, causal_q_len):
    H, heads, D = layer.hidden, layer.heads, layer.head_dim
    f = lambda t: cpu(t)
    # LayerNormQ
    mx, rate = mismatch_report(f(tr["h8"]), O.layernorm_q(hidden_np, f(layer.ln1.weight), f(layer.ln1.bias), 1e-5))
    assert mx <= 1 and rate < 1e-3
    h8 = f(tr["h8"]).reshape(B * S, H)
    # q projection (bit-exact given the same int8 input), laid out per head
    q = O.linear_a8_w8_b8_o8(h8, f(layer.q_proj.weight), f(layer.q_proj.bias), np.float32(float(layer.q_proj.a)), np.float32(float(layer.q_proj.b)))
    q_heads = q.reshape(B, S, heads, D).transpose(0, 2, 1, 3).reshape(B * heads, S, D)
    assert np.array_equal(f(tr["q"]), q_heads)
    # new K / V rows land in the last S slots of the cache
    k = O.linear_a8_w8_b8_o8(h8, f(layer.k_proj.weight), f(layer.k_proj.bias), np.float32(float(layer.k_proj.a)), np.float32(float(layer.k_proj.b)))
    k_heads = k.reshape(B, S, heads, D).transpose(0, 2, 1, 3).reshape(B * heads, S, D)
    assert np.array_equal(f(tr["k_all"])[:, -S:, :], k_heads)
    v = O.linear_a8_w8_b8_o8(h8, f(layer.v_proj.weight), f(layer.v_proj.bias), np.float32(float(layer.v_proj.a)), np.float32(float(layer.v_proj.b)))
    v_heads = v.reshape(B, S, heads, D).transpose(0, 2, 1, 3).reshape(B * heads, S, D)
    assert np.array_equal(f(tr["vt_all"])[:, :, -S:], v_heads.transpose(0, 2, 1))
    # scores, probabilities, context
    assert np.array_equal(f(tr["scores"]), O.bmm_s8t_s8n_s8t(f(tr["q"]), f(tr["k_all"]), np.float32(layer.qk_alpha)))
    mx, rate = mismatch_report(f(tr["probs"]), O.softmax_q(f(tr["scores"]), layer.score_scale, causal_q_len=causal_q_len))
    assert mx <= 1 and rate < 2e-3
    ctx = O.bmm_s8t_s8n_s8t(f(tr["probs"]), f(tr["vt_all"]), np.float32(layer.pv_alpha))       # [B*heads, S, D]
    ctx_merged = ctx.reshape(B, heads, S, D).transpose(0, 2, 1, 3).reshape(B, S, H)
    assert np.array_equal(f(tr["ctx"]), ctx_merged)
    # out_proj -> int32, fused dequant + residual + LayerNormQ
    acc = O.linear_a8_w8_b32_o32(f(tr["ctx"]).reshape(B * S, H), f(layer.out_proj.weight), f(layer.out_proj.bias))
    assert np.array_equal(f(tr["acc"]).reshape(B * S, H), acc)
    rout, h8b = O.dq_add_layernorm_q(f(tr["acc"]), layer.ln2.input_scale, hidden_np, f(layer.ln2.weight), f(layer.ln2.bias), 1e-5)
    assert np.array_equal(f(tr["resid"]), rout)
    mx, rate = mismatch_report(f(tr["h8b"]), h8b)
    assert mx <= 1 and rate < 1e-3
    # fc1 + GELU-quant, fc2, residual
    f8 = O.linear_a8_w8_bfp32_ofp32_GeLu_Q(f(tr["h8b"]).reshape(B * S, H), f(layer.fc1.weight), f(layer.fc1.bias),
                                           np.float32(float(layer.fc1.a)), np.float32(float(layer.fc1.b)))
    mx, rate = mismatch_report(f(tr["f8"]).reshape(B * S, -1), f8)
    assert mx <= 1 and rate < 1e-3
    y = O.linear_a8_w8_bfp32_ofp32(f(tr["f8"]).reshape(B * S, -1), f(layer.fc2.weight), f(layer.fc2.bias), np.float32(float(layer.fc2.a)), np.float32(1.0))
    assert np.array_equal(f(tr["fc2"]).reshape(B * S, H), y)
    assert np.array_equal(f(tr["out"]), f(tr["fc2"]) + f(tr["resid"]))
    # the layer does something non-trivial: outputs are not saturated everywhere
    assert np.unique(f(tr["h8b"])).size > 50 and np.unique(f(tr["probs"])).size > 5


def test_decoder_layer_prefill_and_decode_small():
    from triton_int_amd.nn.opt import W8A8OPTDecoderLayer
    H, heads, ffn = 512, 4, 1024
    layer = W8A8OPTDecoderLayer(H, heads, ffn).randomize(seed=3).to(DEV)
    g = np.random.default_rng(5)
    B, S = 2, 48
    hidden = g.standard_normal((B, S, H), dtype=np.float32)
    tr = {}
    out = layer(gpu(hidden), _trace=tr)
    assert out.shape == (B, S, H) and out.dtype == torch.float32
    _check_stages(layer, tr, hidden, B, S, causal_q_len=S)
    # untraced, fc2 and the residual add are one library call: same bits
    assert torch.equal(layer(gpu(hidden)), out)
    # the one-kernel attention forced on for this small two-batch case: same context rows
    layer.fused_attention_min_queries = 1
    trf = {}
    layer(gpu(hidden), _trace=trf)
    assert trf["scores"] is None
    assert torch.equal(trf["ctx"], tr["ctx"]) and torch.equal(trf["q"], tr["q"])
    layer.fused_attention_min_queries = 128
    # decode: 16 new tokens against a cache of T = 80 slots (64 old + 16 new)
    T, Sd = 80, 16
    k_cache = torch.from_numpy(g.integers(-127, 128, size=(B * heads, T, H // heads), dtype=np.int8)).to(DEV)
    vt_cache = torch.from_numpy(g.integers(-127, 128, size=(B * heads, H // heads, T), dtype=np.int8)).to(DEV)
    k_old, vt_old = k_cache.clone(), vt_cache.clone()
    hidden_d = g.standard_normal((B, Sd, H), dtype=np.float32)
    tr = {}
    layer.fused_attention = False  # the three-launch chain first: its stages are checked one by one
    out = layer(gpu(hidden_d), kv_cache=(k_cache, vt_cache), _trace=tr)
    assert out.shape == (B, Sd, H)
    assert torch.equal(k_cache[:, :T - Sd], k_old[:, :T - Sd]) and torch.equal(vt_cache[:, :, :T - Sd], vt_old[:, :, :T - Sd])
    _check_stages(layer, tr, hidden_d, B, Sd, causal_q_len=Sd)
    k3, v3 = k_old.clone(), vt_old.clone()
    assert torch.equal(layer(gpu(hidden_d), kv_cache=(k3, v3)), out)  # decode: the GEMM kernel adds the residual
    # the same decode step through the one-kernel attention, the default for 16 or fewer query rows
    # (cache offset T - S in the causal mask)
    layer.fused_attention = True
    k2, v2 = k_old.clone(), vt_old.clone()
    trf = {}
    layer(gpu(hidden_d), kv_cache=(k2, v2), _trace=trf)
    assert trf["scores"] is None and torch.equal(trf["ctx"], tr["ctx"])   # the one-kernel attention is the chain, bit for bit


def test_decoder_layer_opt13b_shapes_run():
    """OPT-13B shapes (hidden 5120, 40 heads, FFN 20480): prefill 1x2048 and decode 16 tokens against
    a 2048-long int8 KV.  Spot checks through the oracle on sampled rows."""
    from triton_int_amd.nn.opt import W8A8OPTDecoderLayer
    layer = W8A8OPTDecoderLayer().randomize(seed=1).to(DEV)
    g = torch.Generator(device="cpu").manual_seed(2)
    hidden = torch.randn((1, 2048, 5120), generator=g)
    # one-kernel attention (the default at this size) against the three-launch chain
    trf = {}
    out_fused = layer(hidden.to(DEV), _trace=trf)
    assert trf["scores"] is None and trf["probs"] is None
    layer.fused_attention = False
    tr = {}
    out = layer(hidden.to(DEV), _trace=tr)
    assert out.shape == (1, 2048, 5120) and torch.isfinite(out).all()
    # The one-kernel attention sums a row's exponentials as integers, like the stand-alone softmax
    # kernel: same probabilities, same context, same layer output, bit for bit.
    assert torch.equal(trf["ctx"], tr["ctx"])
    assert torch.equal(trf["q"], tr["q"]) and torch.equal(trf["vt_all"], tr["vt_all"])
    assert torch.equal(out_fused, out)
    rows = [0, 777, 2047]
    h8 = cpu(tr["h8"])[0]
    q = O.linear_a8_w8_b8_o8(h8[rows], cpu(layer.q_proj.weight), cpu(layer.q_proj.bias), np.float32(float(layer.q_proj.a)), np.float32(float(layer.q_proj.b)))
    assert np.array_equal(cpu(tr["q"]).transpose(1, 0, 2).reshape(2048, 5120)[rows], q)
    sc = cpu(tr["scores"][7])
    assert np.array_equal(sc[rows], O.bmm_s8t_s8n_s8t(cpu(tr["q"][7:8])[:, rows], cpu(tr["k_all"][7:8]), np.float32(layer.qk_alpha))[0])
    mx, rate = mismatch_report(cpu(tr["probs"][7]), O.softmax_q(sc, layer.score_scale, causal_q_len=2048))
    assert mx <= 1 and rate < 2e-3
    y = O.linear_a8_w8_bfp32_ofp32(cpu(tr["f8"])[0][rows], cpu(layer.fc2.weight), cpu(layer.fc2.bias), np.float32(float(layer.fc2.a)), np.float32(1.0))
    assert np.array_equal(cpu(tr["fc2"])[0][rows], y)
    # decode
    k_cache = torch.randint(-127, 128, (40, 2048, 128), dtype=torch.int8, generator=g).to(DEV)
    vt_cache = torch.randint(-127, 128, (40, 128, 2048), dtype=torch.int8, generator=g).to(DEV)
    hd = torch.randn((1, 16, 5120), generator=g)
    tr = {}
    kc2, vc2 = k_cache.clone(), vt_cache.clone()
    out = layer(hd.to(DEV), kv_cache=(k_cache, vt_cache), _trace=tr)  # layer.fused_attention is off here: the chain
    assert out.shape == (1, 16, 5120) and torch.isfinite(out).all()
    assert np.array_equal(cpu(tr["scores"]), O.bmm_s8t_s8n_s8t(cpu(tr["q"]), cpu(tr["k_all"]), np.float32(layer.qk_alpha)))
    acc = O.linear_a8_w8_b32_o32(cpu(tr["ctx"])[0], cpu(layer.out_proj.weight), cpu(layer.out_proj.bias))
    assert np.array_equal(cpu(tr["acc"])[0], acc)
    # the default decode path (one attention kernel per step): same context, same layer output
    layer.fused_attention = True
    trf = {}
    out_f = layer(hd.to(DEV), kv_cache=(kc2, vc2), _trace=trf)
    assert trf["scores"] is None and torch.equal(kc2, k_cache) and torch.equal(vc2, vt_cache)
    assert torch.equal(trf["ctx"], tr["ctx"]) and torch.equal(out_f, out)


def test_layer_replayed_from_a_hip_graph_matches_eager():
    """The decode pass and a small prefill pass captured into a HIP graph: every replay (with the
    program's own eager launches and synchronisations in between) must reproduce the eager output
    bit for bit — the kernels keep no state between launches and the library records no memsets."""
    from triton_int_amd.nn.opt import W8A8OPTDecoderLayer

    layer = W8A8OPTDecoderLayer(hidden=1024, heads=8, ffn=4096).randomize(seed=5).to(DEV)
    g = torch.Generator(device="cpu").manual_seed(11)
    for S, T in ((16, 272), (192, 192)):
        x = torch.randn((1, S, 1024), generator=g).to(DEV)
        kc0 = torch.randint(-127, 128, (8, T, 128), dtype=torch.int8, generator=g).to(DEV)
        vc0 = torch.randint(-127, 128, (8, 128, T), dtype=torch.int8, generator=g).to(DEV)
        want = layer(x, kv_cache=(kc0.clone(), vc0.clone())).clone()
        kc, vc = kc0.clone(), vc0.clone()
        graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
        with torch.cuda.stream(side):
            layer(x, kv_cache=(kc, vc))  # warm-up on the capture stream (allocator, scale cache)
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                out = layer(x, kv_cache=(kc, vc))
        torch.cuda.synchronize()
        for rep in range(3):
            out.zero_()
            kc.copy_(kc0); vc.copy_(vc0)
            layer(torch.randn_like(x))  # unrelated eager work between replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want), f"S={S} replay {rep}"
