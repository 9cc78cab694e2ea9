"""CPU oracle for the triton_int INT8 hot path — TEST INFRASTRUCTURE ONLY.

Nothing under ``triton_int_amd/`` may import this package.  It is the checker used by
``tests/``, by the smoke check and by the benchmark's ``cpu_baseline`` leg.

``ti_oracle.c`` is the restatement itself (plain C, each fp32 operation rounded on its own);
this module loads it with ctypes and gives it numpy signatures that follow the reference's
launcher names (``kernels/linear.py``, ``kernels/bmm.py``, ``kernels/fused.py``,
``functional/fused.py`` of zhanglei1172/triton_int).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libti_oracle.so")

EPI_I32, EPI_SCALE_I32, EPI_SCALE_I8, EPI_SCALE_RELU_I8, EPI_SCALE_F, EPI_GELU_I8 = range(6)
DT_I8, DT_I32, DT_F32, DT_F16, DT_BF16 = range(5)
BIAS_NONE, BIAS_I8, BIAS_I32, BIAS_F32 = range(4)
RNE_CLAMP, TRUNC = 0, 1

_NP_OUT = {DT_I8: np.int8, DT_I32: np.int32, DT_F32: np.float32, DT_F16: np.uint16, DT_BF16: np.uint16}


def build(force: bool = False) -> str:
    """Compile ti_oracle.c with gcc (a few hundred ms).  Returns the path of the library."""
    src = os.path.join(_HERE, "ti_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE, "-B", "-s"], check=True)
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        for name in ("ti_oracle_bmm_i8", "ti_oracle_layernorm_q", "ti_oracle_dq_add_layernorm_q",
                     "ti_oracle_gelu_q", "ti_oracle_gelu_f32", "ti_oracle_softmax_q"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _f32p(v):
    if v is None:
        return None, ctypes.c_void_p(0)
    arr = np.asarray(v, dtype=np.float32).reshape(1).copy()
    return arr, ctypes.c_void_p(arr.ctypes.data)


def _bias_kind(bias):
    if bias is None:
        return BIAS_NONE
    return {np.dtype(np.int8): BIAS_I8, np.dtype(np.int32): BIAS_I32, np.dtype(np.float32): BIAS_F32}[bias.dtype]


def bmm_i8(a, b, *, epilogue, out_dtype, bias=None, alpha=None, beta=None, round_mode=RNE_CLAMP):
    """a [B,M,K] int8, b [B,N,K] int8 (logical indexing; any numpy strides) -> [B,M,N]."""
    assert a.dtype == np.int8 and b.dtype == np.int8 and a.ndim == 3 and b.ndim == 3
    B, M, K = a.shape
    Bb, N, Kb = b.shape
    assert B == Bb and K == Kb, "Incompatible dimensions"
    out = np.empty((B, M, N), dtype=_NP_OUT[out_dtype])
    if bias is not None:
        bias = np.ascontiguousarray(bias)
        assert bias.shape == (N,)
    ka, pa = _f32p(alpha)
    kb, pb = _f32p(beta)
    i64 = ctypes.c_int64
    sa = [s // a.itemsize for s in a.strides]
    sb = [s // b.itemsize for s in b.strides]
    sc = [s // out.itemsize for s in out.strides]
    rc = lib().ti_oracle_bmm_i8(
        _p(a), i64(sa[0]), i64(sa[1]), i64(sa[2]), _p(b), i64(sb[0]), i64(sb[1]), i64(sb[2]),
        _p(out), i64(sc[0]), i64(sc[1]), i64(sc[2]), B, M, N, K, _p(bias), _bias_kind(bias),
        pa, pb, int(epilogue), int(out_dtype), int(round_mode))
    assert rc == 0
    del ka, kb
    return out


def _lin(a, w, **kw):
    lead = a.shape[:-1]
    rows = int(np.prod(lead, dtype=np.int64))
    a2 = a.reshape(1, rows, a.shape[-1])
    return bmm_i8(a2, w[None], **kw).reshape(*lead, w.shape[0])


# ---- launcher-named wrappers (reference: kernels/linear.py, kernels/bmm.py, kernels/fused.py) ----

def linear_a8_w8_b8_o8(a, w, bias, alpha, beta, round_mode=RNE_CLAMP):
    return _lin(a, w, epilogue=EPI_SCALE_I8, out_dtype=DT_I8, bias=bias, alpha=alpha, beta=beta, round_mode=round_mode)


def linear_relu_a8_w8_b8_o8(a, w, bias, alpha, beta, round_mode=RNE_CLAMP):
    return _lin(a, w, epilogue=EPI_SCALE_RELU_I8, out_dtype=DT_I8, bias=bias, alpha=alpha, beta=beta, round_mode=round_mode)


def linear_a8_w8_b32_o32(a, w, bias):
    return _lin(a, w, epilogue=EPI_I32, out_dtype=DT_I32, bias=bias)


def linear_a8_w8_b32_o32_with_scaling(a, w, bias, alpha, beta, round_mode=TRUNC):
    return _lin(a, w, epilogue=EPI_SCALE_I32, out_dtype=DT_I32, bias=bias, alpha=alpha, beta=beta, round_mode=round_mode)


def linear_a8_w8_bfp32_ofp32(a, w, bias, alpha, beta, out_dtype=DT_F32):
    return _lin(a, w, epilogue=EPI_SCALE_F, out_dtype=out_dtype, bias=bias, alpha=alpha, beta=beta)


def linear_a8_w8_ofp32(a, w, alpha, out_dtype=DT_F32):
    return _lin(a, w, epilogue=EPI_SCALE_F, out_dtype=out_dtype, alpha=alpha)


def linear_a8_w8_bfp32_ofp32_GeLu_Q(a, w, bias, alpha, beta, round_mode=RNE_CLAMP):
    return _lin(a, w, epilogue=EPI_GELU_I8, out_dtype=DT_I8, bias=bias, alpha=alpha, beta=beta, round_mode=round_mode)


def bmm_s8t_s8n_s8t(a, b, alpha, round_mode=RNE_CLAMP):
    return bmm_i8(a, b, epilogue=EPI_SCALE_I8, out_dtype=DT_I8, alpha=alpha, round_mode=round_mode)


def bmm_s8t_s8n_f32t(a, b, alpha, out_dtype=DT_F32):
    return bmm_i8(a, b, epilogue=EPI_SCALE_F, out_dtype=out_dtype, alpha=alpha)


def bmm_s8t_s8n_s32t(a, b):
    return bmm_i8(a, b, epilogue=EPI_I32, out_dtype=DT_I32)


def bmm_s8t_s8t_s8t(a, b_kn, alpha, round_mode=RNE_CLAMP):
    """b_kn is [B,K,N] (kernels/bmm.py:732-734)."""
    return bmm_i8(a, b_kn.transpose(0, 2, 1), epilogue=EPI_SCALE_I8, out_dtype=DT_I8, alpha=alpha, round_mode=round_mode)


def bmm_s8t_s8t_s32t(a, b_kn):
    return bmm_i8(a, b_kn.transpose(0, 2, 1), epilogue=EPI_I32, out_dtype=DT_I32)


def layernorm_q(x, gamma, beta, eps, rms=False, round_mode=RNE_CLAMP, return_stats=False):
    """kernels/fused.py:336-382.  x [..., N] fp32 -> int8 same shape."""
    x2 = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, x.shape[-1])
    rows, cols = x2.shape
    gamma = np.ascontiguousarray(gamma, dtype=np.float32)
    beta = None if beta is None else np.ascontiguousarray(beta, dtype=np.float32)
    y = np.empty((rows, cols), np.int8)
    mean = np.empty(rows, np.float32)
    rstd = np.empty(rows, np.float32)
    i64 = ctypes.c_int64
    rc = lib().ti_oracle_layernorm_q(_p(x2), i64(cols), _p(gamma), _p(beta), ctypes.c_float(eps), _p(y),
                                     i64(cols), rows, cols, int(bool(rms)), int(round_mode), _p(mean), _p(rstd))
    assert rc == 0
    y = y.reshape(x.shape)
    return (y, mean, rstd) if return_stats else y


def dq_add_layernorm_q(acc_i32, in_scale, resid_in, gamma, beta, eps, round_mode=RNE_CLAMP, return_all=False):
    """functional/fused.py:6-15 -> (resid_out fp32, y int8); return_all adds (ln fp32, mean, rstd)."""
    shape = acc_i32.shape
    a2 = np.ascontiguousarray(acc_i32, dtype=np.int32).reshape(-1, shape[-1])
    r2 = np.ascontiguousarray(resid_in, dtype=np.float32).reshape(-1, shape[-1])
    rows, cols = a2.shape
    gamma = np.ascontiguousarray(gamma, dtype=np.float32)
    beta = None if beta is None else np.ascontiguousarray(beta, dtype=np.float32)
    rout = np.empty((rows, cols), np.float32)
    y = np.empty((rows, cols), np.int8)
    ln = np.empty((rows, cols), np.float32)
    mean = np.empty(rows, np.float32)
    rstd = np.empty(rows, np.float32)
    i64 = ctypes.c_int64
    rc = lib().ti_oracle_dq_add_layernorm_q(
        _p(a2), i64(cols), ctypes.c_float(in_scale), _p(r2), i64(cols), _p(gamma), _p(beta), ctypes.c_float(eps),
        _p(rout), i64(cols), _p(y), i64(cols), _p(ln), i64(cols), rows, cols, int(round_mode), _p(mean), _p(rstd))
    assert rc == 0
    if return_all:
        return rout.reshape(shape), y.reshape(shape), ln.reshape(shape), mean, rstd
    return rout.reshape(shape), y.reshape(shape)


def gelu_q(x, scale, round_mode=RNE_CLAMP):
    """kernels/fused.py:76-79 then q8."""
    x1 = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    y = np.empty(x1.shape, np.int8)
    ks, ps = _f32p(scale)
    rc = lib().ti_oracle_gelu_q(_p(x1), ps, _p(y), ctypes.c_int64(x1.size), int(round_mode))
    assert rc == 0
    return y.reshape(x.shape)


def gelu_f32(x, scale):
    x1 = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    y = np.empty(x1.shape, np.float32)
    ks, ps = _f32p(scale)
    rc = lib().ti_oracle_gelu_f32(_p(x1), ps, _p(y), ctypes.c_int64(x1.size))
    assert rc == 0
    return y.reshape(x.shape)


def softmax_q(x_i8, scale, causal_q_len=0):
    """int8 scores [..., cols] -> int8 probabilities round(softmax(x*scale)*127)."""
    x2 = np.ascontiguousarray(x_i8, dtype=np.int8).reshape(-1, x_i8.shape[-1])
    rows, cols = x2.shape
    y = np.empty((rows, cols), np.int8)
    i64 = ctypes.c_int64
    rc = lib().ti_oracle_softmax_q(_p(x2), i64(cols), ctypes.c_float(scale), _p(y), i64(cols), rows, cols, int(causal_q_len))
    assert rc == 0
    return y.reshape(x_i8.shape)


def attention_i8(q, k, vt, qk_alpha, score_scale, pv_alpha, causal_q_len=0, return_all=False):
    """The three steps an attention block chains (reference: nn/bmm.py:10-29 BMM_S8T_S8N_S8T for
    Q.K^T, the caller's softmax, nn/bmm.py:10-29 again for P.V), restated as that chain:
    int8 scores, int8 probabilities, int8 context.  q [BH,S,D], k [BH,T,D], vt [BH,D,T]."""
    scores = bmm_s8t_s8n_s8t(q, k, np.float32(qk_alpha))
    probs = softmax_q(scores, score_scale, causal_q_len=causal_q_len)
    ctx = bmm_s8t_s8n_s8t(probs, vt, np.float32(pv_alpha))
    return (scores, probs, ctx) if return_all else ctx


def quantize_per_token_absmax(t):
    """dynamic_quantize_activation_per_token_absmax (reference: functional/quantization.py:61-67)
    restated in numpy, every step in t's dtype (float32 or float16; numpy rounds each float16
    operation to float16 as torch's elementwise kernels do): returns (q int8, max_val [..., 1])."""
    dt = t.dtype
    assert dt in (np.float32, np.float16)
    max_val = np.abs(t).max(axis=-1, keepdims=True)
    max_val = np.maximum(max_val.astype(np.float32), np.float32(1e-8)).astype(dt)  # clamp(min=1e-8)
    max_val = (max_val / dt.type(127)).astype(dt)
    with np.errstate(divide="ignore", invalid="ignore"):
        d = (t / max_val).astype(dt)
    q = np.clip(np.rint(d.astype(np.float32)), -128, 127)
    return q.astype(np.int8), max_val


def _round_fp(v32, kind):
    """float32 values rounded (half to even) to `kind` in {"f32", "f16", "bf16"}, returned as float32."""
    v32 = np.asarray(v32, dtype=np.float32)
    if kind == "f32":
        return v32
    if kind == "f16":
        with np.errstate(over="ignore"):  # beyond 65504 -> inf, as the hardware conversion gives
            return v32.astype(np.float16).astype(np.float32)
    assert kind == "bf16"
    u = v32.view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    r = np.where(nan, (u | 0x400000) & 0xFFFF0000, r).astype(np.uint32)
    return r.view(np.float32)


def layer_norm_fp(x, weight, bias, eps, rms=False, skip=None, kind="f32"):
    """layer_norm_fwd_fused_single_pass / skip_layer_norm_fwd_fused_single_pass(2)
    (reference: kernels/fused.py:385-862).  All tensors are float32 arrays holding values
    representable in `kind` ("f32", "f16", "bf16"); returns (out, skip_out) the same way
    (skip_out is None without skip).  Statistics: the row's mean and biased variance evaluated in
    float64 and rounded to float32 (what any fp32 summation order approximates to a few ulps);
    normalisation: ((a - mean) * rstd) * w (+ b), each step rounded to float32
    (kernels/fused.py:473-477); out rounded to `kind`, skip_out = round(out + skip)
    (kernels/fused.py:630-640).  fp16 callers raise eps to 1.6e-5 first (kernels/fused.py:502-503)."""
    shape = x.shape
    a = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, shape[-1])
    w = np.asarray(weight, dtype=np.float32)
    a64 = a.astype(np.float64)
    if rms:
        mean = np.zeros((a.shape[0], 1), np.float32)
        var = (a64 * a64).mean(axis=1, keepdims=True).astype(np.float32)
    else:
        mean64 = a64.mean(axis=1, keepdims=True)
        mean = mean64.astype(np.float32)
        var = ((a64 - mean64) ** 2).mean(axis=1, keepdims=True).astype(np.float32)
    rstd = (np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)).astype(np.float32)
    o = ((a - mean) * rstd).astype(np.float32) * w
    if bias is not None:
        o = o + np.asarray(bias, dtype=np.float32)
    out = _round_fp(o.astype(np.float32), kind)
    skip_out = None
    if skip is not None:
        s = np.ascontiguousarray(skip, dtype=np.float32).reshape(a.shape)
        skip_out = _round_fp(out + s, kind).reshape(shape)
    return out.reshape(shape), skip_out
