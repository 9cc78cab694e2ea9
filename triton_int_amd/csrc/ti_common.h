// ti_common.h — shared host/device helpers for libtriton_int_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/triton_int_hip.h"

namespace ti {

// ---- host: error reporting ---------------------------------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
// Checks once per device that the current device is gfx950; returns TI_OK or TI_E_DEVICE.
int check_device();
int launch_status(const char* what);

// ---- device: quantisation helpers ----------------------------------------------------------

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

// clamp(round_half_even(v), -128, 127), NaN -> 0.  v_rndne_f32, v_cvt_i32_f32 (saturating,
// NaN -> 0), v_med3_i32.  TRUNC drops the rndne: the conversion itself truncates toward zero.
template <bool TRUNC>
__device__ __forceinline__ int q8(float v) {
  float r = TRUNC ? v : __builtin_rintf(v);
  int i = (int)r;
  return min(max(i, -128), 127);
}

__device__ __forceinline__ int q8(float v, int round_mode) {
  return round_mode == TI_ROUND_TRUNC ? q8<true>(v) : q8<false>(v);
}

// fp32 -> int32 with the same two modes; the hardware conversion saturates and maps NaN to 0.
__device__ __forceinline__ int q32(float v, int round_mode) {
  float r = round_mode == TI_ROUND_TRUNC ? v : __builtin_rintf(v);
  if (r >= 2147483648.0f) return 0x7fffffff;
  if (r <= -2147483648.0f) return (int)0x80000000;
  if (r != r) return 0;
  return (int)r;
}

__device__ __forceinline__ unsigned pack4(int a, int b, int c, int d) {
  return (unsigned)(a & 0xff) | ((unsigned)(b & 0xff) << 8) | ((unsigned)(c & 0xff) << 16) |
         ((unsigned)d << 24);
}

// tanh-GELU times scale, 0.5 * x * (1 + tanh(k * (x + 0.044715 * x^3))) * scale
// (kernels/fused.py:79), evaluated as (x * scale) / (1 + e^(-2u)) with
// -2u * log2(e) = x * (c0 + c1 * x^2), c0 = -2 k log2 e, c1 = 0.044715 * c0: 6 plain operations, one
// exp2 and one reciprocal per element instead of 15 + 2 in the literal order — in a GEMM epilogue
// this is time the matrix pipe waits.  Same function to within a few fp32 ulps (no cancellation at
// either end: e -> inf gives x * scale * 0, e -> 0 gives x * scale); after the int8 quantisation a
// value sitting on a rounding boundary can come out one step apart.
__device__ __forceinline__ float gelu_tanh_scaled(float x, float scale) {
  const float c0 = -2.30220819814f;            // -2 * sqrt(2/pi) * log2(e)
  const float c1 = -2.30220819814f * 0.044715f;
  const float p = __builtin_fmaf(x * x, c1, c0);
  const float e = __builtin_amdgcn_exp2f(x * p);
  const float r = __builtin_amdgcn_rcpf(1.0f + e);
  return (x * scale) * r;
}

// ---- softmax-quantise arithmetic -----------------------------------------------------------------
// int8 scores x -> int8 probabilities rne(127 * softmax(x * scale)) the same way in every kernel that
// forms them (the stand-alone softmax kernels and both attention kernels), so that their results
// agree bit for bit whatever the order in which they visit a row:
//   mx  = the row's largest visible score (an integer: exact in any order)
//   t   = fma(float(x), s2, c),  c = -(float(mx) * s2),  s2 = scale * log2(e)
//   e   = exp2(t)                                      (at the maximum t is the rounding residue of
//                                                       mx * s2, at most half an ulp of it, so e = 2^(+-d)
//                                                       with d <= 2^-12 for scales up to SM_MAX_SCALE: the
//                                                       steps below stay exact in that range.  Far beyond it
//                                                       (scale ~ 1000) e * r could pass 127.5 and wrap the
//                                                       byte; the entry points refuse such scales.)
//   u   = rne(e * 2^23), taken from the bit pattern of 1.0f + e
//   S   = sum of u over the row: an integer, so any order and any grouping give the same S
//   r   = 127 * 2^23 / float(S)                        (float(S) correctly rounded, IEEE division)
//   p   = rne(e * r): the low byte of the bit pattern of fma(e, r, 1.5 * 2^23)
constexpr float SM_MAX_SCALE = 64.0f;           // largest score scale the entry points accept (e^64 between neighbours: one-hot)
constexpr unsigned SM_ONE_BITS = 0x3f800000u;  // bit pattern of 1.0f: sm_unit_bits(e) - SM_ONE_BITS = u

__device__ __forceinline__ unsigned sm_unit_bits(float e) { return __float_as_uint(1.0f + e); }

// 127 * 2^23 / S for the exact row sum S (< 2^48)
__device__ __forceinline__ float sm_scale_from_sum(unsigned long long S) {
  const float hi = (float)(unsigned)(S >> 24), lo = (float)(unsigned)(S & 0xffffffu);  // both exact
  const float sf = __builtin_fmaf(hi, 16777216.0f, lo);                                // rounded once
  return 1065353216.0f / sf;
}

// byte n (0..3) of w as a signed int8, converted to float: one instruction (sub-dword source select
// with sign extension)
template <int N>
__device__ __forceinline__ float sbyte_to_float(unsigned w) {
  float f;
  if constexpr (N == 0) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_0" : "=v"(f) : "v"(w));
  else if constexpr (N == 1) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_1" : "=v"(f) : "v"(w));
  else if constexpr (N == 2) asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_2" : "=v"(f) : "v"(w));
  else asm("v_cvt_f32_i32_sdwa %0, sext(%1) dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_3" : "=v"(f) : "v"(w));
  return f;
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  __bf16 h = (__bf16)f;  // v_cvt_pk_bf16_f32, round-to-nearest-even
  return __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;  // v_cvt_f16_f32, round-to-nearest-even
  return __builtin_bit_cast(uint16_t, h);
}

}  // namespace ti
