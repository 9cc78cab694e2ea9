"""ctypes binding of libtriton_int_hip.so (declared in include/triton_int_hip.h).

torch is imported first on purpose: the library needs libamdhip64.so.7, and torch carries its
own copy with that SONAME; loading torch first makes both share one HIP runtime (one context,
interchangeable streams and device pointers).
"""
from __future__ import annotations

import ctypes
import os

import torch  # noqa: F401  (must precede the CDLL below)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtriton_int_hip.so")

# enum ti_epilogue / ti_dtype / ti_bias / ti_round
EPI_I32, EPI_SCALE_I32, EPI_SCALE_I8, EPI_SCALE_RELU_I8, EPI_SCALE_F, EPI_GELU_I8 = range(6)
DT_I8, DT_I32, DT_F32, DT_F16, DT_BF16 = range(5)
BIAS_NONE, BIAS_I8, BIAS_I32, BIAS_F32, BIAS_F16, BIAS_BF16 = range(6)
ROUND_RNE_CLAMP, ROUND_TRUNC = 0, 1

TORCH_TO_DT = {torch.int8: DT_I8, torch.int32: DT_I32, torch.float32: DT_F32, torch.float16: DT_F16,
               torch.bfloat16: DT_BF16}
TORCH_TO_BIAS = {torch.int8: BIAS_I8, torch.int32: BIAS_I32, torch.float32: BIAS_F32, torch.float16: BIAS_F16,
                 torch.bfloat16: BIAS_BF16}

EXPORTS = ("ti_version", "ti_last_error", "ti_mfma_i8_probe", "ti_bmm_i8", "ti_bmm_i8_config", "ti_bmm_i8_grouped", "ti_bmm_i8_static_scratch", "ti_gemm_num_configs",
           "ti_gemm_config_name", "ti_gemm_last_config", "ti_gemm_last_splits", "ti_gemm_plan", "ti_release_workspaces", "ti_layernorm_q", "ti_dq_add_layernorm_q", "ti_gelu_q", "ti_softmax_q", "ti_transpose_i8", "ti_attention_i8", "ti_quantize_per_token_absmax", "ti_kv_append_i8",
           "ti_layernorm_fp", "ti_linear_i8_residual_f32", "ti_qkv_decode_i8")

_lib = None

_vp, _i64, _int, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float


def _declare(lib):
    lib.ti_version.restype = _int
    lib.ti_version.argtypes = []
    lib.ti_last_error.restype = ctypes.c_char_p
    lib.ti_last_error.argtypes = []
    lib.ti_mfma_i8_probe.restype = _int
    lib.ti_mfma_i8_probe.argtypes = [_int, _int, _vp, ctypes.POINTER(ctypes.c_double)]
    bmm_args = [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64,
                _int, _int, _int, _int, _vp, _int, _vp, _vp, _int, _int, _int]
    lib.ti_bmm_i8.restype = _int
    lib.ti_bmm_i8.argtypes = bmm_args + [_vp]
    lib.ti_bmm_i8_config.restype = _int
    lib.ti_bmm_i8_config.argtypes = bmm_args + [_int, _vp]
    lib.ti_bmm_i8_static_scratch.restype = _int
    lib.ti_bmm_i8_static_scratch.argtypes = bmm_args + [_int, _vp]
    lib.ti_bmm_i8_grouped.restype = _int
    lib.ti_bmm_i8_grouped.argtypes = [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64,
                                      _int, _int, _int, _int, _vp, _int, _i64, _vp, _vp, _i64, _int, _int, _int,
                                      _int, _vp]
    lib.ti_gemm_plan.restype = _int
    lib.ti_gemm_plan.argtypes = bmm_args + [_int, _int, ctypes.POINTER(ctypes.c_int64)]
    lib.ti_release_workspaces.restype = _int
    lib.ti_release_workspaces.argtypes = [_vp, _int, ctypes.POINTER(ctypes.c_int64)]
    lib.ti_gemm_num_configs.restype = _int
    lib.ti_gemm_num_configs.argtypes = []
    lib.ti_gemm_last_config.restype = _int
    lib.ti_gemm_last_config.argtypes = []
    lib.ti_gemm_last_splits.restype = _int
    lib.ti_gemm_last_splits.argtypes = []
    lib.ti_gemm_config_name.restype = ctypes.c_char_p
    lib.ti_gemm_config_name.argtypes = [_int]
    lib.ti_layernorm_q.restype = _int
    lib.ti_layernorm_q.argtypes = [_vp, _i64, _vp, _vp, _f32, _vp, _i64, _int, _int, _int, _int, _vp, _vp, _vp]
    lib.ti_dq_add_layernorm_q.restype = _int
    lib.ti_dq_add_layernorm_q.argtypes = [_vp, _i64, _f32, _vp, _vp, _i64, _vp, _vp, _f32, _vp, _i64, _vp, _i64,
                                          _vp, _i64, _int, _int, _int, _vp, _vp, _vp]
    lib.ti_softmax_q.restype = _int
    lib.ti_softmax_q.argtypes = [_vp, _i64, _f32, _vp, _i64, _int, _int, _int, _vp]
    lib.ti_transpose_i8.restype = _int
    lib.ti_transpose_i8.argtypes = [_vp, _i64, _vp, _i64, _int, _int, _vp]
    lib.ti_kv_append_i8.restype = _int
    lib.ti_kv_append_i8.argtypes = [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _int, _int, _int, _vp]
    lib.ti_quantize_per_token_absmax.restype = _int
    lib.ti_quantize_per_token_absmax.argtypes = [_vp, _int, _i64, _vp, _i64, _vp, _int, _int, _vp]
    lib.ti_layernorm_fp.restype = _int
    lib.ti_layernorm_fp.argtypes = [_vp, _i64, _vp, _i64, _int, _vp, _vp, _f32, _int, _vp, _i64, _vp, _i64, _int, _int, _vp]
    lib.ti_attention_i8.restype = _int
    lib.ti_attention_i8.argtypes = [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64,
                                    _int, _int, _int, _int, _f32, _f32, _f32, _int, _vp]
    lib.ti_linear_i8_residual_f32.restype = _int
    lib.ti_linear_i8_residual_f32.argtypes = [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _i64, _int, _int, _int, _vp]
    lib.ti_qkv_decode_i8.restype = _int
    lib.ti_qkv_decode_i8.argtypes = [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _int, _int, _int,
                                     _vp, _i64, _vp, _i64, _int, _vp]
    lib.ti_gelu_q.restype = _int
    lib.ti_gelu_q.argtypes = [_vp, _vp, _vp, _i64, _int, _vp]


def lib() -> ctypes.CDLL:
    """The loaded library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m triton_int_amd.build` "
                "(hipcc, gfx950).  triton_int_amd has no CPU or Triton fallback.")
        handle = ctypes.CDLL(LIB_PATH)
        _declare(handle)
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc == 0:
        return
    msg = lib().ti_last_error().decode()
    if rc < 0:
        # invalid-argument codes surface like the reference's Python asserts
        raise AssertionError(f"{what}: {msg} (status {rc})")
    raise RuntimeError(f"{what}: {msg} (hipError {rc})")


def ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def current_stream(device) -> int:
    """Raw hipStream_t of torch's current stream on `device` (the short way: no Stream object)."""
    idx = device.index
    if idx is None:
        idx = torch.cuda.current_device()
    return torch._C._cuda_getCurrentRawStream(idx)


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def on_device(device):
    """Context manager that makes `device` current for the launch; free when it already is."""
    idx = device.index
    if idx is None or idx == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def require_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "triton_int_amd kernels run on the GPU only (got a tensor on "
                f"{t.device}); there is no CPU fallback")


_scalar_cache: dict = {}
_SCALAR_CACHE_MAX = 1024  # distinct (value, device) pairs kept; beyond it python-float scales are uploaded per call


def scale_tensor(v, device) -> torch.Tensor:
    """Scales are 0-dim fp32 device tensors read inside the kernel (the reference does
    tl.load(scale), kernels/linear.py:227,247).  Python floats, which the reference's own
    scripts also pass (kernels/bmm.py:777), are uploaded once and cached by value."""
    if torch.is_tensor(v):
        if v.device != device or v.dtype != torch.float32:
            v = v.to(device=device, dtype=torch.float32)
        return v
    key = (float(v), str(device))
    t = _scalar_cache.get(key)
    if t is None:
        # Entries are never evicted: a captured HIP graph keeps the device address of every scale it
        # was recorded with (4 bytes per distinct value and device).  The upload is a synchronous
        # host-to-device copy, which a capturing stream cannot record: pass the scale as a device
        # tensor, or call once with the same value before the capture.
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                f"scale {float(v)!r} was first seen during HIP graph capture; pass scales as fp32 device "
                "tensors, or run the call once before capturing")
        t = torch.tensor(float(v), dtype=torch.float32, device=device)
        # Bounded: a caller that passes a fresh python float on every call (a dynamic per-batch scale) would
        # otherwise grow the cache without end.  Past the bound the upload is simply not kept: the launcher
        # holds the tensor until the launch is enqueued, and the allocator hands its block only to later work
        # of the same stream.  Dynamic scales belong in device tensors, which take no upload at all.
        if len(_scalar_cache) < _SCALAR_CACHE_MAX:
            _scalar_cache[key] = t
    return t


def release_workspaces(stream=None, all_streams: bool = False) -> int:
    """Frees the split-K workspaces the library holds for `stream` (default: torch's current stream) on the
    current device, or for every stream; returns the bytes freed.  Waits for the streams' queued work."""
    freed = ctypes.c_int64(0)
    h = current_stream(torch.device("cuda", torch.cuda.current_device())) if stream is None else int(stream)
    check(lib().ti_release_workspaces(h, 1 if all_streams else 0, ctypes.byref(freed)), "ti_release_workspaces")
    return int(freed.value)
