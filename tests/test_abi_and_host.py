"""CPU-side checks: the built library exports every function the public header declares, and the
host-side mirror of the reference interface (modules, buffers, scale algebra, argument checks)
behaves without a GPU.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "triton_int_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ti_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from triton_int_amd import _lib
    names = declared_functions()
    assert "ti_bmm_i8" in names and "ti_layernorm_q" in names and len(names) >= 10
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert set(names) == set(_lib.EXPORTS)
    assert _lib.lib().ti_version() == 2
    n = _lib.lib().ti_gemm_num_configs()
    assert n >= 5 and _lib.lib().ti_gemm_config_name(0).decode().startswith("gather")


def test_missing_library_raises(monkeypatch):
    from triton_int_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libtriton_int_hip.so")
    with pytest.raises(RuntimeError, match="no CPU or Triton fallback"):
        _lib.lib()


def test_cpu_tensors_are_refused_not_emulated():
    from triton_int_amd.kernels.linear import linear_a8_w8_b8_o8
    from triton_int_amd.kernels.fused import gelu_q, layer_norm_fwd_fused_single_pass_q
    a = torch.zeros((4, 16), dtype=torch.int8)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        linear_a8_w8_b8_o8(a, a, torch.zeros(4, dtype=torch.int8), 1.0, 1.0)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        gelu_q(torch.zeros(8), 1.0)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        layer_norm_fwd_fused_single_pass_q(torch.zeros(2, 8), torch.ones(8), torch.zeros(8), 1e-5)
    with pytest.raises(AssertionError, match="Incompatible dimensions"):
        linear_a8_w8_b8_o8(a, torch.zeros((4, 32), dtype=torch.int8), None, 1.0, 1.0)


def test_module_buffers_match_reference_names():
    from triton_int_amd.nn import bmm, fused, linear
    m = linear.W8A8B8O8Linear(32, 16, alpha=0.5, beta=0.25)
    sd = m.state_dict()
    assert list(sd) == ["weight", "bias", "a", "b"]
    assert sd["weight"].shape == (16, 32) and sd["weight"].dtype == torch.int8
    assert sd["bias"].dtype == torch.int8 and sd["a"].dtype == torch.float32 and sd["a"].ndim == 0
    assert int(sd["weight"].min()) >= -127 and int(sd["weight"].max()) <= 126
    assert linear.W8A8B32O32Linear(8, 8).bias.dtype == torch.int32
    assert list(linear.W8A8B32O32LinearWithoutScaling(8, 8).state_dict()) == ["weight", "bias"]
    assert linear.W8A8BFP32OFP32Linear(8, 8, alpha=3.0, beta=9.0).b.item() == 1.0
    assert list(bmm.BMM_S8T_S8N_S8T(0.5).state_dict()) == ["a"]
    ln = fused.LayerNormQ(24)
    assert list(ln.state_dict()) == ["weight", "bias"] and ln.eps == 1e-5 and ln.input_scale == 1.0
    assert fused.DQ_Add_LayerNorm_Q(24).input_scale == 1.0
    # state dicts interchange: load a dict with the reference's key names
    m2 = linear.W8A8B8O8Linear(32, 16)
    m2.load_state_dict(sd)
    assert torch.equal(m2.weight, m.weight) and float(m2.a) == 0.5


def test_from_float_algebra_on_cpu():
    from triton_int_amd.functional.quantization import (quantize_per_tensor_absmax,
                                                        quantize_weight_per_channel_absmax,
                                                        dynamic_quantize_activation_per_token_absmax)
    from triton_int_amd.nn.bmm import BMM_S8T_S8N_F32T, BMM_S8T_S8N_S8T
    from triton_int_amd.nn.linear import W8A8B32O32Linear
    torch.manual_seed(1)
    w = torch.randn(6, 10)
    q, s = quantize_per_tensor_absmax(w.clone())
    assert q.dtype == torch.int8 and torch.allclose(s, w.abs().max() / 127)
    assert torch.equal(q, (w / s).round().to(torch.int8)) and int(q.abs().max()) == 127
    qc, sc = quantize_weight_per_channel_absmax(w.clone())
    assert sc.shape == (6, 1) and torch.all(qc.abs().max(dim=1)[0] == 127)
    x = torch.randn(4, 10)
    qa, sa = dynamic_quantize_activation_per_token_absmax(x.clone())
    assert qa.dtype == torch.int8 and sa.shape == (4, 1)
    assert torch.allclose(qa.float() * sa, x, atol=float(sa.max()))
    lin = torch.nn.Linear(10, 6)
    b0 = lin.bias.detach().clone()
    m = W8A8B32O32Linear.from_float(lin, 0.02, 0.05)
    bs = b0.abs().max() / (2**31 - 1)
    assert m.bias.dtype == torch.int32 and torch.allclose(m.b, bs / 0.05)
    assert abs(float(BMM_S8T_S8N_S8T.from_scale(0.02, 0.03, 0.6).a) - 0.001) < 1e-9
    assert abs(float(BMM_S8T_S8N_F32T.from_scale(0.5, 0.25).a) - 0.125) < 1e-9


def test_torch_ops_are_registered_with_meta_implementations():
    """torch.ops.triton_op.* (the namespace the reference registers under, kernels/__init__.py:5)
    exist and propagate shapes and dtypes on meta tensors, which is what tracing needs."""
    import torch
    from triton_int_amd.kernels import _ops

    assert len(_ops.registered) == len(_ops._OPS)
    m = lambda shape, dt=torch.int8: torch.empty(shape, dtype=dt, device="meta")
    s = m((), torch.float32)
    ops = torch.ops.triton_op
    for name in ("linear_a8_w8_b8_o8", "linear_relu_a8_w8_b8_o8", "linear_a8_w8_bfp32_ofp32_GeLu_Q"):
        bias = m(32, torch.float32 if "GeLu" in name else torch.int8)
        y = getattr(ops, name)(m((3, 5, 64)), m((32, 64)), bias, s, s)
        assert y.shape == (3, 5, 32) and y.dtype == torch.int8 and y.device.type == "meta"
    assert ops.linear_a8_w8_b32_o32(m((7, 64)), m((32, 64)), None).dtype == torch.int32
    assert ops.linear_a8_w8_bfp32_ofp32(m((7, 64)), m((32, 64)), m(32, torch.float32), s, s).dtype == torch.float32
    assert ops.bmm_s8t_s8n_s8t(m((2, 3, 16)), m((2, 9, 16)), 0.5).shape == (2, 3, 9)
    assert ops.bmm_s8t_s8t_s32t(m((2, 3, 16)), m((2, 16, 9))).shape == (2, 3, 9)
    assert ops.bmm_s8t_s8n_f32t(m((2, 3, 16)), m((2, 9, 16)), 0.5).dtype == torch.float32
    assert ops.layer_norm_fwd_fused_single_pass_q(m((4, 8), torch.float32), m(8, torch.float32), None, 1e-5).dtype == torch.int8
    r, q = ops.dq_add_layernorm_q(m((4, 8), torch.int32), 0.1, m((4, 8), torch.float32), m(8, torch.float32), m(8, torch.float32), 1e-5)
    assert r.dtype == torch.float32 and q.dtype == torch.int8 and q.shape == (4, 8)
    assert ops.softmax_q(m((2, 4, 16)), 0.05).shape == (2, 4, 16)
    assert ops.attention_i8(m((2, 4, 128)), m((2, 16, 128)), m((2, 128, 16)), 1e-3, 0.05, 0.01, 4).shape == (2, 4, 128)
    q8, sc = ops.quantize_per_token_absmax(m((3, 5, 16), torch.float16))
    assert q8.shape == (3, 5, 16) and sc.shape == (3, 5, 1) and sc.dtype == torch.float16
    y = ops.layer_norm_fwd_fused_single_pass(m((4, 8), torch.bfloat16), m(8, torch.bfloat16), None, 1e-5)
    assert y.shape == (4, 8) and y.dtype == torch.bfloat16
    y = ops.skip_layer_norm_fwd_fused_single_pass(m((4, 8), torch.float16), m((4, 8), torch.float16), m(8, torch.float16), None, 1e-5)
    assert y.shape == (4, 8) and y.dtype == torch.float16
    o, so = ops.skip_layer_norm_fwd_fused_single_pass2(m((4, 8), torch.float32), m((4, 8), torch.float32), m(8, torch.float32),
                                                       m(8, torch.float32), 1e-5, True)
    assert o.shape == so.shape == (4, 8) and so.dtype == torch.float32


def test_reference_import_paths_resolve_to_this_package():
    """Code written against the reference imports triton_int.* (nn/linear.py:18, nn/bmm.py:10,
    functional/bmm.py:6); those paths are this package's modules, not copies."""
    import importlib

    import triton_int
    import triton_int_amd
    from triton_int.functional.bmm import bmm_i8_o8, bmm_i8_o32
    from triton_int.functional.fused import dq_add_layernorm_q_py
    from triton_int.kernels.bmm import bmm_s8t_s8n_f32t, bmm_s8t_s8n_s8t
    from triton_int.kernels.fused import layer_norm_fwd_fused_single_pass_q, linear_a8_w8_bfp32_ofp32_GeLu_Q
    from triton_int.kernels.linear import linear_a8_w8_b8_o8, linear_a8_w8_bfp32_ofp32
    from triton_int.nn.bmm import BMM_S8T_S8N_F32T, BMM_S8T_S8N_S8T
    from triton_int.nn.fused import DQ_Add_LayerNorm_Q, LayerNormQ, W8A8BFP32OFP32_GeLu_Q
    from triton_int.nn.linear import W8A8B8O8Linear, W8A8B8O8LinearReLU, W8A8BFP32OFP32Linear

    assert W8A8B8O8Linear is triton_int_amd.nn.linear.W8A8B8O8Linear
    assert BMM_S8T_S8N_S8T is triton_int_amd.nn.bmm.BMM_S8T_S8N_S8T
    assert LayerNormQ is triton_int_amd.nn.fused.LayerNormQ
    assert linear_a8_w8_b8_o8 is triton_int_amd.kernels.linear.linear_a8_w8_b8_o8
    assert bmm_i8_o8 is triton_int_amd.functional.bmm.bmm_i8_o8
    for rel in triton_int.ALIASES:
        assert importlib.import_module("triton_int." + rel) is importlib.import_module("triton_int_amd." + rel)
    assert triton_int.nn.linear is triton_int_amd.nn.linear
    for f in (bmm_i8_o32, dq_add_layernorm_q_py, bmm_s8t_s8n_f32t, bmm_s8t_s8n_s8t, layer_norm_fwd_fused_single_pass_q,
              linear_a8_w8_bfp32_ofp32_GeLu_Q, linear_a8_w8_bfp32_ofp32, BMM_S8T_S8N_F32T, DQ_Add_LayerNorm_Q,
              W8A8BFP32OFP32_GeLu_Q, W8A8B8O8LinearReLU, W8A8BFP32OFP32Linear):
        assert callable(f)


def test_c_abi_status_codes_with_raw_ctypes():
    """Argument errors come back as TI_E_* codes with a message in ti_last_error(), straight from the
    C ABI (no Python launcher in between).  Argument validation precedes any device access, so no
    kernel is launched and no GPU is needed."""
    from triton_int_amd import _lib as L
    lib = L.lib()
    TI_E_NULL, TI_E_SHAPE, TI_E_COMBO, TI_E_STRIDE = -1, -2, -3, -4
    P = 0x1000  # a non-NULL pointer value; never dereferenced on these paths

    def bmm(A=P, B=P, C=P, sC=(0, 64, 1), batch=1, M=32, N=64, K=64, bias=0, bias_kind=L.BIAS_NONE, alpha=P, beta=0,
            epi=L.EPI_SCALE_I8, dt=L.DT_I8, rnd=L.ROUND_RNE_CLAMP):
        return lib.ti_bmm_i8(A, 0, K, 1, B, 0, K, 1, C, sC[0], sC[1], sC[2], batch, M, N, K, bias, bias_kind, alpha, beta,
                             epi, dt, rnd, None)

    def err():
        return lib.ti_last_error().decode()

    assert bmm(A=0) == TI_E_NULL and "A is NULL" in err()
    assert bmm(B=0) == TI_E_NULL and "B is NULL" in err()
    assert bmm(C=0) == TI_E_NULL and "C is NULL" in err()
    assert bmm(alpha=0) == TI_E_NULL and "alpha" in err()
    assert bmm(bias=P, bias_kind=L.BIAS_I8, beta=0) == TI_E_NULL and "beta" in err()
    assert bmm(epi=L.EPI_GELU_I8, beta=0) == TI_E_NULL and "beta" in err()
    assert bmm(M=-1) == TI_E_SHAPE and "negative" in err()
    assert bmm(batch=70000) == TI_E_SHAPE and "batch" in err()
    assert bmm(dt=L.DT_F32) == TI_E_COMBO and "combination" in err()                       # int8 epilogue, fp32 output
    assert bmm(epi=L.EPI_SCALE_F, dt=L.DT_I8) == TI_E_COMBO
    assert bmm(bias=P, bias_kind=L.BIAS_F32, beta=P) == TI_E_COMBO                         # fp32 bias on the int8-bias epilogue
    assert bmm(epi=L.EPI_I32, dt=L.DT_I32, bias=P, bias_kind=L.BIAS_I8) == TI_E_COMBO
    assert bmm(epi=17) == TI_E_COMBO
    assert bmm(rnd=5) == TI_E_COMBO and "round mode" in err()
    assert bmm(sC=(0, 0, 1)) == TI_E_STRIDE and "row stride" in err()
    assert bmm(sC=(0, 64, 0)) == TI_E_STRIDE and "column stride" in err()
    # empty problems are no-ops whatever the pointers are
    assert bmm(A=0, B=0, C=0, M=0) == 0 and bmm(A=0, B=0, C=0, batch=0) == 0
    # grouped form: negative batch strides of bias / scales
    assert lib.ti_bmm_i8_grouped(P, 0, 64, 1, P, 0, 64, 1, P, 0, 64, 1, 1, 32, 64, 64, 0, L.BIAS_NONE, -1, P, 0, 0,
                                 L.EPI_SCALE_I8, L.DT_I8, 0, -1, None) == TI_E_STRIDE
    # row kernels
    assert lib.ti_layernorm_q(0, 8, P, P, 1e-5, P, 8, 4, 8, 0, 0, 0, 0, None) == TI_E_NULL
    assert lib.ti_layernorm_q(P, 8, P, P, 1e-5, P, 8, -4, 8, 0, 0, 0, 0, None) == TI_E_SHAPE
    assert lib.ti_layernorm_q(P, 8, P, P, 1e-5, P, 8, 4, 8, 0, 9, 0, 0, None) == TI_E_COMBO
    assert lib.ti_dq_add_layernorm_q(P, 8, 1.0, 0, P, 8, P, P, 1e-5, P, 8, 0, 8, 0, 8, 4, 8, 0, 0, 0, None) == TI_E_NULL  # neither y nor ln_out
    assert "y / ln_out_f32" in err()
    assert lib.ti_softmax_q(P, 16, 0.1, P, 16, 4, 16, 32, None) == TI_E_SHAPE               # causal_q_len > cols
    assert lib.ti_softmax_q(0, 16, 0.1, P, 16, 4, 16, 0, None) == TI_E_NULL
    assert lib.ti_softmax_q(P, 16, 100.0, P, 16, 4, 16, 0, None) == TI_E_COMBO and "scale" in err()   # beyond the exact range
    assert lib.ti_softmax_q(P, 16, -0.1, P, 16, 4, 16, 0, None) == TI_E_COMBO
    assert lib.ti_attention_i8(P, 2048, 128, P, 2048, 128, P, 2048, 16, P, 2048, 128, 1, 16, 16, 128, 1e-3, 100.0, 0.01, 0, None) == TI_E_COMBO
    assert lib.ti_attention_i8(P, 2048, 128, P, 2048, 128, P, 2048, 16, P, 2048, 128, 1, 16, 16, 128, 1e-3, 0.0, 0.01, 0, None) == TI_E_COMBO
    assert lib.ti_qkv_decode_i8(P, 64, P, 64, 0, P, P, P, 64, 32, 64, 2048, P, 64, P, 64, 16, None) == TI_E_COMBO  # M > 16
    assert lib.ti_mfma_i8_probe(-1, 0, None, None) == TI_E_SHAPE


def test_bench_reads_the_traffic_figure_from_the_committed_profile():
    """bench.py's roofline.traffic is parsed out of the counters summary it names: the row and the two scale
    factors must be there, and the figure must be what they multiply out to."""
    import bench

    kernel = "ws_256x128x128_w2x2_s1_p3_l4/int8"
    total, source = bench.traffic_from_profile(kernel)
    assert total is not None and source.startswith(bench.TRAFFIC_PROFILE[kernel][0])
    assert 2.0 * 48.65e6 < total < 3.0 * 48.65e6  # 2.5x the algorithmic bytes of an average launch of the step
    assert bench.traffic_from_profile("no such kernel") == (None, None)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr
