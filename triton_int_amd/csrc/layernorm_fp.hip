// layernorm_fp.hip — floating-point LayerNorm / RMSNorm row kernels for gfx950, with the optional
// skip (residual) add of the output.  Replaces kernel_layer_norm_fwd_fused_single_pass,
// kernel_skip_layer_norm_fwd_fused_single_pass and kernel_skip_layer_norm_fwd_fused_single_pass_2
// (kernels/fused.py:385-862 of zhanglei1172/triton_int) for fp32, fp16 and bf16 tensors:
//     a    = f32(x)
//     mean = sum(a) / N (0 for RMSNorm), var = sum((a - mean)^2) / N, rstd = 1 / sqrt(var + eps)
//     out  = T( ((a - mean) * rstd) * f32(weight) [+ f32(bias)] )            (kernels/fused.py:473-481)
//     skip_out = T( f32(out) + f32(skip) )                                   (kernels/fused.py:630-640)
// The reference merges per-block Welford statistics; the statistics here are the exact two-pass
// ones of the whole row (the row sits in registers), which agree with it to fp32 rounding.
//
// One 256-thread workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ...; weight and bias stay
// in registers across rows.  A thread owns 16-byte vectors t, t + 256, ... of the row, so every load
// and store instruction of a wave covers one contiguous 1 KB run; x and skip are read once, each
// output is written once, all non-temporal.
#include "ti_common.h"

namespace ti {

constexpr int LF_THREADS = 256;
constexpr int LF_WAVES = LF_THREADS / 64;

struct bf16_t { uint16_t bits; };

template <typename T> __device__ __forceinline__ float lf_to_f32(unsigned raw_bits);
template <> __device__ __forceinline__ float lf_to_f32<float>(unsigned b) { return __uint_as_float(b); }
template <> __device__ __forceinline__ float lf_to_f32<_Float16>(unsigned b) { return (float)__builtin_bit_cast(_Float16, (uint16_t)b); }
template <> __device__ __forceinline__ float lf_to_f32<bf16_t>(unsigned b) { return __uint_as_float(b << 16); }

template <typename T> __device__ __forceinline__ unsigned lf_from_f32(float f);
template <> __device__ __forceinline__ unsigned lf_from_f32<float>(float f) { return __float_as_uint(f); }
template <> __device__ __forceinline__ unsigned lf_from_f32<_Float16>(float f) { return f32_to_f16_bits(f); }
template <> __device__ __forceinline__ unsigned lf_from_f32<bf16_t>(float f) { return f32_to_bf16_bits(f); }

// element e of a 16-byte vector of T held as four dwords
template <typename T>
__device__ __forceinline__ float lf_get(const v4u& raw, int e) {
  if constexpr (sizeof(T) == 4) return lf_to_f32<T>(raw[e]);
  else return lf_to_f32<T>((raw[e >> 1] >> (16 * (e & 1))) & 0xffffu);
}

// round N floats to T and pack them into a 16-byte vector; `rounded` receives the values as T holds them
template <typename T, int N>
__device__ __forceinline__ v4u lf_pack(const float (&v)[N], float (&rounded)[N]) {
  v4u raw = {0u, 0u, 0u, 0u};
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const unsigned b = lf_from_f32<T>(v[e]);
    rounded[e] = lf_to_f32<T>(b);
    if constexpr (sizeof(T) == 4) raw[e] = b;
    else raw[e >> 1] |= b << (16 * (e & 1));
  }
  return raw;
}

// `red` holds two sets of per-wave partial sums; consecutive reductions (counted by `k`) alternate between
// them, so one barrier per reduction is enough (a wave that runs ahead writes the set nobody reads any more)
__device__ __forceinline__ float lf_block_sum(float v, float* red, int tid, int& k) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  float* set = red + (k & 1) * LF_WAVES;
  ++k;
  if ((tid & 63) == 0) set[tid >> 6] = v;
  __syncthreads();
  float s = set[0];
#pragma unroll
  for (int w = 1; w < LF_WAVES; ++w) s += set[w];
  return s;
}

struct LnFpParams {
  const void* x;
  const void* skip;   // may be null
  const void* gamma;
  const void* beta;   // may be null
  void* out;          // may be null (skip_out only)
  void* skip_out;     // may be null
  int64_t x_rs, skip_rs, out_rs, sout_rs;  // row strides in elements
  float eps;
  int rows, cols, rms;
};

template <typename T, int VPT>
__global__ __launch_bounds__(LF_THREADS) void layernorm_fp_vec_kernel(LnFpParams p) {
  constexpr int N = 16 / (int)sizeof(T);
  __shared__ float red[2 * LF_WAVES];
  int red_k = 0;
  const int tid = threadIdx.x;
  const int nvec = p.cols / N;
  const bool has_b = p.beta != nullptr;
  const v4u zero = {0u, 0u, 0u, 0u};

  float w[VPT][N], b[VPT][N];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int v = tid + j * LF_THREADS;
    const v4u rw = v < nvec ? *((const v4u*)p.gamma + v) : zero;
    const v4u rb = (has_b && v < nvec) ? *((const v4u*)p.beta + v) : zero;
#pragma unroll
    for (int e = 0; e < N; ++e) {
      w[j][e] = lf_get<T>(rw, e);
      b[j][e] = lf_get<T>(rb, e);
    }
  }
  const float inv_n = 1.0f / (float)p.cols;

  for (int row = blockIdx.x; row < p.rows; row += gridDim.x) {
    const v4u* xr = (const v4u*)((const T*)p.x + (int64_t)row * p.x_rs);
    v4u rx[VPT], rs[VPT];
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int v = tid + j * LF_THREADS;
      rx[j] = v < nvec ? __builtin_nontemporal_load(xr + v) : zero;
    }
    if (p.skip) {
      const v4u* sr = (const v4u*)((const T*)p.skip + (int64_t)row * p.skip_rs);
#pragma unroll
      for (int j = 0; j < VPT; ++j) {
        const int v = tid + j * LF_THREADS;
        rs[j] = v < nvec ? __builtin_nontemporal_load(sr + v) : zero;
      }
    }
    float x[VPT][N];
#pragma unroll
    for (int j = 0; j < VPT; ++j)
#pragma unroll
      for (int e = 0; e < N; ++e) x[j][e] = lf_get<T>(rx[j], e);

    float mean = 0.0f;
    if (!p.rms) {
      float s = 0.0f;
#pragma unroll
      for (int j = 0; j < VPT; ++j)
#pragma unroll
        for (int e = 0; e < N; ++e) s += x[j][e];  // padding vectors hold zeros
      mean = lf_block_sum(s, red, tid, red_k) * inv_n;
    }
    float m2 = 0.0f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      if (tid + j * LF_THREADS < nvec) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
          const float d = x[j][e] - mean;
          m2 += d * d;
        }
      }
    }
    const float var = lf_block_sum(m2, red, tid, red_k) * inv_n;
    const float rstd = 1.0f / sqrtf(var + p.eps);

#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int v = tid + j * LF_THREADS;
      if (v < nvec) {
        float o[N], ot[N];
#pragma unroll
        for (int e = 0; e < N; ++e) {
          const float t = ((x[j][e] - mean) * rstd) * w[j][e];
          o[e] = has_b ? t + b[j][e] : t;
        }
        const v4u ro = lf_pack<T, N>(o, ot);
        if (p.out) __builtin_nontemporal_store(ro, (v4u*)((T*)p.out + (int64_t)row * p.out_rs) + v);
        if (p.skip_out) {
          float so[N], unused[N];
#pragma unroll
          for (int e = 0; e < N; ++e) so[e] = ot[e] + lf_get<T>(rs[j], e);
          __builtin_nontemporal_store(lf_pack<T, N>(so, unused), (v4u*)((T*)p.skip_out + (int64_t)row * p.sout_rs) + v);
        }
      }
    }
  }
}

template <typename T> __device__ __forceinline__ float lf_load1(const void* p, int64_t i);
template <> __device__ __forceinline__ float lf_load1<float>(const void* p, int64_t i) { return ((const float*)p)[i]; }
template <> __device__ __forceinline__ float lf_load1<_Float16>(const void* p, int64_t i) { return (float)((const _Float16*)p)[i]; }
template <> __device__ __forceinline__ float lf_load1<bf16_t>(const void* p, int64_t i) { return __uint_as_float((unsigned)((const uint16_t*)p)[i] << 16); }

template <typename T> __device__ __forceinline__ float lf_store1(void* p, int64_t i, float f);
template <> __device__ __forceinline__ float lf_store1<float>(void* p, int64_t i, float f) { ((float*)p)[i] = f; return f; }
template <> __device__ __forceinline__ float lf_store1<_Float16>(void* p, int64_t i, float f) {
  const _Float16 h = (_Float16)f;
  ((_Float16*)p)[i] = h;
  return (float)h;
}
template <> __device__ __forceinline__ float lf_store1<bf16_t>(void* p, int64_t i, float f) {
  const uint16_t h = f32_to_bf16_bits(f);
  ((uint16_t*)p)[i] = h;
  return __uint_as_float((unsigned)h << 16);
}

// Any column count / alignment: one row per workgroup, the row is read once per pass (it stays in L2).
template <typename T>
__global__ __launch_bounds__(LF_THREADS) void layernorm_fp_any_kernel(LnFpParams p) {
  __shared__ float red[2 * LF_WAVES];
  int red_k = 0;
  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  const int64_t xo = (int64_t)row * p.x_rs;
  const float inv_n = 1.0f / (float)p.cols;
  float mean = 0.0f;
  if (!p.rms) {
    float s = 0.0f;
    for (int i = tid; i < p.cols; i += LF_THREADS) s += lf_load1<T>(p.x, xo + i);
    mean = lf_block_sum(s, red, tid, red_k) * inv_n;
  }
  float m2 = 0.0f;
  for (int i = tid; i < p.cols; i += LF_THREADS) {
    const float d = lf_load1<T>(p.x, xo + i) - mean;
    m2 += d * d;
  }
  const float var = lf_block_sum(m2, red, tid, red_k) * inv_n;
  const float rstd = 1.0f / sqrtf(var + p.eps);
  for (int i = tid; i < p.cols; i += LF_THREADS) {
    const float t = ((lf_load1<T>(p.x, xo + i) - mean) * rstd) * lf_load1<T>(p.gamma, i);
    const float o = p.beta ? t + lf_load1<T>(p.beta, i) : t;
    float ot;
    if (p.out) ot = lf_store1<T>(p.out, (int64_t)row * p.out_rs + i, o);
    else ot = lf_to_f32<T>(lf_from_f32<T>(o));
    if (p.skip_out) lf_store1<T>(p.skip_out, (int64_t)row * p.sout_rs + i, ot + lf_load1<T>(p.skip, (int64_t)row * p.skip_rs + i));
  }
}

static bool lf_aligned(const void* ptr, int64_t row_stride_elems, int elem) {
  return !ptr || ((((uintptr_t)ptr) & 15) == 0 && ((row_stride_elems * elem) & 15) == 0);
}

template <typename T>
static int launch_layernorm_fp(const LnFpParams& p, hipStream_t stream) {
  constexpr int N = 16 / (int)sizeof(T);
  const int E = (int)sizeof(T);
  const bool vec = p.cols % N == 0 && p.cols <= LF_THREADS * N * 8 && lf_aligned(p.x, p.x_rs, E) &&
                   lf_aligned(p.skip, p.skip_rs, E) && lf_aligned(p.gamma, 0, E) && lf_aligned(p.beta, 0, E) &&
                   lf_aligned(p.out, p.out_rs, E) && lf_aligned(p.skip_out, p.sout_rs, E);
  if (!vec) {
    layernorm_fp_any_kernel<T><<<dim3((unsigned)p.rows), dim3(LF_THREADS), 0, stream>>>(p);
    return launch_status("layernorm_fp_any_kernel");
  }
  const int vpt = (p.cols / N + LF_THREADS - 1) / LF_THREADS;
  // persistent workgroups per CU for 3..5 vectors per thread, measured at 16384 rows of 5120 / 4096
  // columns with 4 / 3 / 2 of them: the skip variants (two or three streams per row) run best with 2
  // (fp16 122 / 114 / 113 us, bf16 122 / 117 / 110, fp32 244 / 246 / 232), plain fp32 with 3 at 5120
  // columns (118 / 113 / 113) and 2 at 4096 (94 / 93 / 88), plain 16-bit with 4 (56 / 60 / 80)
  // Two vectors per thread (16-bit rows of 2049 .. 4096 columns), 16384 x 4096 fp16 after 20 ms of the same
  // launches, 8 / 6 / 4 / 3 / 2 per CU: plain 49.5 / 45.8 / 45.3 / 48.6 / 67.5 us, skip with both outputs
  // 96.4 / 95.6 / 96.3 / 87.7 / 86.8 us.
  const unsigned mid = p.skip ? 2u : (sizeof(T) == 4 ? (vpt >= 5 ? 3u : 2u) : 4u);
  const unsigned slots = 256u * (vpt <= 1 ? 8u : (vpt == 2 ? (p.skip ? 2u : 4u) : (vpt <= 5 ? mid : 2u)));
  const dim3 grid((unsigned)p.rows < slots ? (unsigned)p.rows : slots), block(LF_THREADS);
#define TI_LF_LAUNCH(V) layernorm_fp_vec_kernel<T, V><<<grid, block, 0, stream>>>(p)
  if (vpt <= 1) TI_LF_LAUNCH(1);
  else if (vpt <= 2) TI_LF_LAUNCH(2);
  else if (vpt <= 3) TI_LF_LAUNCH(3);
  else if (vpt <= 4) TI_LF_LAUNCH(4);
  else if (vpt <= 5) TI_LF_LAUNCH(5);
  else if (vpt <= 6) TI_LF_LAUNCH(6);
  else TI_LF_LAUNCH(8);
#undef TI_LF_LAUNCH
  return launch_status("layernorm_fp_vec_kernel");
}

}  // namespace ti

extern "C" int ti_layernorm_fp(const void* x, int64_t x_row_stride, const void* skip, int64_t skip_row_stride, int dtype,
                               const void* gamma, const void* beta, float eps, int rms, void* out,
                               int64_t out_row_stride, void* skip_out, int64_t skip_out_row_stride, int rows, int cols,
                               void* stream) {
  using namespace ti;
  if (rows < 0 || cols < 0) return fail(TI_E_SHAPE, "negative size");
  if (rows == 0 || cols == 0) return TI_OK;
  if (!x || !gamma) return fail(TI_E_NULL, "x and gamma are required");
  if (!out && !skip_out) return fail(TI_E_NULL, "one of out / skip_out is required");
  if ((skip_out != nullptr) != (skip != nullptr)) return fail(TI_E_NULL, "skip and skip_out go together");
  if (dtype != TI_F32 && dtype != TI_F16 && dtype != TI_BF16) return fail(TI_E_COMBO, "dtype %d: fp32, fp16 or bf16", dtype);
  if (x_row_stride < cols || (skip && skip_row_stride < cols) || (out && out_row_stride < cols) ||
      (skip_out && skip_out_row_stride < cols))
    return fail(TI_E_STRIDE, "row strides must cover a row");
  int rc = check_device();
  if (rc != TI_OK) return rc;
  LnFpParams p = {};
  p.x = x; p.skip = skip; p.gamma = gamma; p.beta = beta; p.out = out; p.skip_out = skip_out;
  p.x_rs = x_row_stride; p.skip_rs = skip_row_stride; p.out_rs = out_row_stride; p.sout_rs = skip_out_row_stride;
  p.eps = eps; p.rows = rows; p.cols = cols; p.rms = rms;
  if (dtype == TI_F32) return launch_layernorm_fp<float>(p, (hipStream_t)stream);
  if (dtype == TI_F16) return launch_layernorm_fp<_Float16>(p, (hipStream_t)stream);
  return launch_layernorm_fp<bf16_t>(p, (hipStream_t)stream);
}
