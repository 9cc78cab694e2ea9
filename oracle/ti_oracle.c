/*
 * ti_oracle.c — CPU restatement of the triton_int INT8 hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker the HIP kernels are compared against.  Only tests/, the smoke
 * check and the benchmark's cpu_baseline leg may build, load or call it; the product
 * (triton_int_amd/) never does and has no CPU fallback.
 *
 * It restates, in plain scalar C with every fp32 operation separately rounded
 * (build with -ffp-contract=off, SSE2 fp32, no fast-math), the arithmetic of these files of
 * zhanglei1172/triton_int.  The reference holds no golden vectors or known-answer tests for
 * any of this (its only checks are GPU print-scripts, kernels/linear.py:856-957,
 * kernels/bmm.py:763-827), so each function is pinned by the independent checks listed
 * with it; they live in tests/test_oracle_*.py.
 *
 *   ti_oracle_bmm_i8            kernels/linear.py:224-254,396,505-534,644-674,786-817,107
 *                               kernels/bmm.py:398-426,551-562,700-710  kernels/fused.py:76-79,184-187
 *       pins: python-int brute force on tiny shapes; torch int32 matmul/bmm and float64 BLAS
 *       (exact for |acc| < 2^53) on mid shapes; alpha=1,beta=0 reduces to acc; ties k+0.5
 *       built with alpha=0.5; torch.round / torch.clamp; F.gelu(approximate="tanh").
 *   ti_oracle_layernorm_q       kernels/fused.py:276-333, nn/fused.py:8-32 (_LayerNormQ emulation)
 *       pins: F.layer_norm in fp32 and fp64; shift invariance; constant rows (var=0).
 *   ti_oracle_dq_add_layernorm_q functional/fused.py:6-24
 *       pins: torch.add(alpha=) + F.layer_norm (the emulation's own calls); resid_out - resid_in
 *       == s*x exactly where representable.
 *   ti_oracle_gelu_q            kernels/fused.py:13,76-79
 *       pins: F.gelu(approximate="tanh"); gelu(0)=0; gelu(x)-gelu(-x)=x; saturation.
 *   ti_oracle_softmax_q         (no reference function: the caller-side step between the two BMMs)
 *       pins: torch.softmax(x*scale).mul(127).round(); rows sum to ~127; one-hot and uniform rows.
 *
 * Rounding contract: q8 = clamp(round_half_even(v), -128, 127), NaN -> 0 (mode 0); mode 1 is
 * the literal Triton `.to(int8)` truncation toward zero, clamped, kept as a test-time switch.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { EPI_I32 = 0, EPI_SCALE_I32 = 1, EPI_SCALE_I8 = 2, EPI_SCALE_RELU_I8 = 3, EPI_SCALE_F = 4,
       EPI_GELU_I8 = 5 };
enum { DT_I8 = 0, DT_I32 = 1, DT_F32 = 2, DT_F16 = 3, DT_BF16 = 4 };
enum { BIAS_NONE = 0, BIAS_I8 = 1, BIAS_I32 = 2, BIAS_F32 = 3 };

/* ---- scalar helpers ------------------------------------------------------------------ */

static inline int8_t q8(float v, int mode) {
  if (v != v) return 0;
  float r = (mode == 1) ? truncf(v) : nearbyintf(v); /* default FP env: ties-to-even */
  if (r < -128.0f) r = -128.0f;
  if (r > 127.0f) r = 127.0f;
  return (int8_t)(int)r;
}

static inline int32_t q32(float v, int mode) {
  if (v != v) return 0;
  float r = (mode == 1) ? truncf(v) : nearbyintf(v);
  if (r <= -2147483648.0f) return INT32_MIN;
  if (r >= 2147483648.0f) return INT32_MAX;
  return (int32_t)r;
}

/* fp32 -> fp16 / bf16 bit patterns, round-to-nearest-even (what a device cvt does). */
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u); /* quiet NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return (uint16_t)(u >> 16);
}

static inline uint16_t f32_to_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 -> inf (65520 rounds up below) */
  if (a < 0x33000000u) return (uint16_t)sign;               /* < 2^-25 -> 0 */
  int e = (int)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  int shift = (e < -14) ? (13 + (-14 - e)) : 13; /* subnormal halves lose more bits */
  uint32_t half_m = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (half_m & 1u))) half_m++;
  uint32_t h;
  if (e < -14) h = half_m; /* subnormal (may carry into the smallest normal, which is right) */
  else h = ((uint32_t)(e + 15) << 10) + (half_m - 0x400u);
  if (h >= 0x7c00u) h = 0x7c00u;
  return (uint16_t)(sign | h);
}

/* tanh-GELU times scale, literal left-to-right evaluation order of kernels/fused.py:79 with the
 * constant of kernels/fused.py:13 rounded to fp32. */
static inline float gelu_tanh_scaled(float x, float scale) {
  const float k = 0.79788456080286535588f; /* sqrt(2/pi) */
  float cube = ((0.044715f * x) * x) * x;
  float inner = k * (x + cube);
  float t = tanhf(inner);
  return ((0.5f * x) * (1.0f + t)) * scale;
}

/* ---- GEMM / BMM ---------------------------------------------------------------------- */

/* Strides in elements.  Host pointers.  alpha/beta are host pointers to one float. */
int ti_oracle_bmm_i8(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk,
                     const int8_t* B, int64_t sBb, int64_t sBn, int64_t sBk,
                     void* C, int64_t sCb, int64_t sCm, int64_t sCn,
                     int batch, int M, int N, int K,
                     const void* bias, int bias_kind,
                     const float* alpha_p, const float* beta_p,
                     int epilogue, int out_dtype, int round_mode) {
  const float alpha = alpha_p ? *alpha_p : 1.0f;
  const float beta = beta_p ? *beta_p : 1.0f;
  if (bias == NULL) bias_kind = BIAS_NONE;
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < batch; ++b) {
    for (int m = 0; m < M; ++m) {
      const int8_t* a_row = A + b * sAb + m * sAm;
      for (int n = 0; n < N; ++n) {
        const int8_t* b_row = B + b * sBb + n * sBn;
        int32_t acc = 0;
        if (sAk == 1 && sBk == 1) {
          for (int k = 0; k < K; ++k) acc += (int32_t)a_row[k] * (int32_t)b_row[k];
        } else {
          for (int k = 0; k < K; ++k) acc += (int32_t)a_row[k * sAk] * (int32_t)b_row[k * sBk];
        }
        const int64_t off = b * sCb + m * sCm + n * sCn;
        float v = 0.0f;
        switch (epilogue) {
          case EPI_I32: {
            /* kernels/linear.py:505-507: bias is added to the int32 accumulator */
            int32_t r = acc;
            if (bias_kind == BIAS_I32) r = (int32_t)((uint32_t)r + (uint32_t)((const int32_t*)bias)[n]);
            ((int32_t*)C)[off] = r;
            continue;
          }
          case EPI_SCALE_I32:
          case EPI_SCALE_I8:
          case EPI_SCALE_RELU_I8:
          case EPI_SCALE_F: {
            /* kernels/linear.py:227,247: c = f(bias)*beta; c += f(acc)*alpha */
            v = (float)acc * alpha;
            if (bias_kind != BIAS_NONE) {
              float bf = bias_kind == BIAS_I8    ? (float)((const int8_t*)bias)[n]
                         : bias_kind == BIAS_I32 ? (float)((const int32_t*)bias)[n]
                                                 : ((const float*)bias)[n];
              float c0 = bf * beta;
              v = c0 + v;
            }
            break;
          }
          case EPI_GELU_I8: {
            /* kernels/fused.py:184-186: fast_geluQ(f(acc)*alpha + bias, beta) */
            float x = (float)acc * alpha;
            if (bias_kind == BIAS_F32) x = x + ((const float*)bias)[n];
            v = gelu_tanh_scaled(x, beta);
            break;
          }
          default:
            continue;
        }
        switch (epilogue) {
          case EPI_SCALE_I32: ((int32_t*)C)[off] = q32(v, round_mode); break;
          case EPI_SCALE_I8:
          case EPI_GELU_I8: ((int8_t*)C)[off] = q8(v, round_mode); break;
          case EPI_SCALE_RELU_I8: { /* kernels/linear.py:396: max(int8(c), 0) */
            int8_t q = q8(v, round_mode);
            ((int8_t*)C)[off] = q < 0 ? 0 : q;
            break;
          }
          case EPI_SCALE_F:
            if (out_dtype == DT_F32) ((float*)C)[off] = v;
            else if (out_dtype == DT_F16) ((uint16_t*)C)[off] = f32_to_f16(v);
            else ((uint16_t*)C)[off] = f32_to_bf16(v);
            break;
          default: break;
        }
      }
    }
  }
  return 0;
}

/* ---- LayerNorm -> int8 --------------------------------------------------------------- */

/* Row statistics are formed in float64 (the value every fp32 summation order approximates)
 * and rounded to fp32; the normalisation then follows kernels/fused.py:307-308,323-327 in fp32:
 * rstd = 1/sqrt(var + eps);  out = ((a - mean) * rstd) * w + b. */
static void row_stats(const float* x, int cols, int rms, float eps, float* mean_f, float* rstd_f) {
  double s = 0.0;
  if (!rms) {
    for (int i = 0; i < cols; ++i) s += (double)x[i];
  }
  const double mean = rms ? 0.0 : s / (double)cols;
  double m2 = 0.0;
  for (int i = 0; i < cols; ++i) {
    double d = (double)x[i] - mean;
    m2 += d * d;
  }
  const float var = (float)(m2 / (double)cols);
  *mean_f = (float)mean;
  *rstd_f = 1.0f / sqrtf(var + eps);
}

int ti_oracle_layernorm_q(const float* x, int64_t x_row_stride, const float* gamma,
                          const float* beta, float eps, int8_t* y, int64_t y_row_stride,
                          int rows, int cols, int rms, int round_mode, float* mean_out,
                          float* rstd_out) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < rows; ++r) {
    const float* xr = x + (int64_t)r * x_row_stride;
    float mean, rstd;
    row_stats(xr, cols, rms, eps, &mean, &rstd);
    if (mean_out) mean_out[r] = mean;
    if (rstd_out) rstd_out[r] = rstd;
    for (int i = 0; i < cols; ++i) {
      float a_hat = (xr[i] - mean) * rstd;
      float o = a_hat * gamma[i];
      if (beta) o = o + beta[i];
      y[(int64_t)r * y_row_stride + i] = q8(o, round_mode);
    }
  }
  return 0;
}

/* functional/fused.py:6-24.  resid_out = resid_in + s * f(x_i32) (product and sum separately
 * rounded); LayerNorm as above; y_i8 = round(clamp(ln, -128, 127)). */
int ti_oracle_dq_add_layernorm_q(const int32_t* acc, int64_t acc_row_stride, float in_scale,
                                 const float* resid_in, int64_t resid_in_row_stride,
                                 const float* gamma, const float* beta, float eps,
                                 float* resid_out, int64_t resid_out_row_stride, int8_t* y,
                                 int64_t y_row_stride, float* ln_out, int64_t ln_out_row_stride,
                                 int rows, int cols, int round_mode, float* mean_out,
                                 float* rstd_out) {
#pragma omp parallel for schedule(static)
  for (int r = 0; r < rows; ++r) {
    const int32_t* ar = acc + (int64_t)r * acc_row_stride;
    const float* rin = resid_in + (int64_t)r * resid_in_row_stride;
    float* rout = resid_out + (int64_t)r * resid_out_row_stride;
    for (int i = 0; i < cols; ++i) {
      float p = in_scale * (float)ar[i];
      rout[i] = rin[i] + p;
    }
    float mean, rstd;
    row_stats(rout, cols, 0, eps, &mean, &rstd);
    if (mean_out) mean_out[r] = mean;
    if (rstd_out) rstd_out[r] = rstd;
    for (int i = 0; i < cols; ++i) {
      float a_hat = (rout[i] - mean) * rstd;
      float o = a_hat * gamma[i];
      if (beta) o = o + beta[i];
      if (ln_out) ln_out[(int64_t)r * ln_out_row_stride + i] = o;
      if (y) y[(int64_t)r * y_row_stride + i] = q8(o, round_mode);
    }
  }
  return 0;
}

/* kernels/fused.py:76-79 applied element-wise, then q8. */
int ti_oracle_gelu_q(const float* x, const float* scale, int8_t* y, int64_t n, int round_mode) {
  const float s = *scale;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) y[i] = q8(gelu_tanh_scaled(x[i], s), round_mode);
  return 0;
}

/* int8 scores -> int8 probabilities round_half_even(127 * softmax(x * scale)) over the row, as
 * SmoothQuant-style callers of the BMM modules do between bmm_s8t_s8n_s8t (kernels/bmm.py:576-612)
 * and the P.V BMM (`softmax(...).mul(127).round()`); the reference tree itself has no such function,
 * so there is nothing of the reference's to follow line by line.  The fp32 steps are fixed so that
 * the row sum does not depend on the order of summation (the HIP kernels visit a row in different
 * orders and must agree with each other bit for bit):
 *     mx = largest visible score;  s2 = scale * log2(e)
 *     e_j = exp2f(fmaf((float)x_j, s2, -((float)mx * s2)))
 *     S   = sum_j rne(e_j * 2^23)     (integer; taken from the bit pattern of 1.0f + e_j)
 *     y_j = rne(e_j * (127 * 2^23 / (float)S))
 * Pins: torch.softmax on x*scale, mul(127), round (tests/test_oracle_rowops.py): the integer sum
 * differs from the real one by less than cols * 2^-24 relative, far inside the +-1 step the
 * comparison allows on rounding boundaries.  causal_q_len as in the HIP entry point. */
int ti_oracle_softmax_q(const int8_t* x, int64_t x_row_stride, float scale, int8_t* y, int64_t y_row_stride,
                        int rows, int cols, int causal_q_len) {
  if (!(scale >= 0.0f)) return -3;
  const float s2 = scale * 1.44269504088896340736f;
#pragma omp parallel for schedule(static)
  for (int r = 0; r < rows; ++r) {
    const int8_t* xr = x + (int64_t)r * x_row_stride;
    int8_t* yr = y + (int64_t)r * y_row_stride;
    int limit = cols;
    if (causal_q_len > 0) {
      limit = (r % causal_q_len) + (cols - causal_q_len) + 1;
      if (limit > cols) limit = cols;
    }
    int mx = -128;
    for (int j = 0; j < limit; ++j) if (xr[j] > mx) mx = xr[j];
    const float c = -((float)mx * s2);
    uint64_t S = 0;
    for (int j = 0; j < limit; ++j) {
      const float e = exp2f(fmaf((float)xr[j], s2, c));
      const float one_plus = 1.0f + e;
      uint32_t bits;
      memcpy(&bits, &one_plus, 4);
      S += bits - 0x3f800000u;
    }
    const float sf = fmaf((float)(uint32_t)(S >> 24), 16777216.0f, (float)(uint32_t)(S & 0xffffffu));
    const float rr = 1065353216.0f / sf;
    for (int j = 0; j < cols; ++j) {
      uint32_t bits = 0;
      if (j < limit) {
        /* e * rr <= 127: adding 1.5 * 2^23 inside the fma rounds the exact product to the nearest
         * integer (ties to even) and leaves it in the low byte of the sum's bit pattern */
        const float t = fmaf(exp2f(fmaf((float)xr[j], s2, c)), rr, 12582912.0f);
        memcpy(&bits, &t, 4);
      }
      yr[j] = (int8_t)(bits & 0xffu);
    }
  }
  return 0;
}

/* Un-quantised value of the GELU epilogue, for tests that want to look at near-ties. */
int ti_oracle_gelu_f32(const float* x, const float* scale, float* y, int64_t n) {
  const float s = *scale;
  for (int64_t i = 0; i < n; ++i) y[i] = gelu_tanh_scaled(x[i], s);
  return 0;
}
