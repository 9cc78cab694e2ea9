// rowops.hip — HBM-bound row kernels for gfx950: LayerNorm -> int8, dequant + residual add +
// LayerNorm -> int8, tanh-GELU -> int8, softmax -> int8 probabilities, int8 transpose and
// KV-cache append.
//
// Replaces kernel_layer_norm_fwd_fused_single_pass_q (kernels/fused.py:235-382 of
// zhanglei1172/triton_int), supplies the native dq_add_layernorm_q the reference only emulates
// (functional/fused.py:6-32) and a launchable form of fast_geluQ (kernels/fused.py:76-79).
//
// Row kernels: a 256-thread workgroup per row at a time.  The whole row sits in registers as float4
// vectors (thread t owns vectors t, t+256, ...: every load/store instruction of a wave is one
// contiguous 1 KB / 256 B run), so x is read from HBM exactly once; mean and the centred sum of
// squares are exact two-pass statistics reduced with wave shuffles and one LDS hop.
#include "ti_common.h"

namespace ti {

constexpr int RN_THREADS = 256;
constexpr int RN_WAVES = RN_THREADS / 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Sum over the workgroup; every thread returns the same bits (fixed combination order).  `red` holds two
// sets of per-wave partial sums and consecutive reductions (counted by `k`) alternate between them, so one
// barrier per reduction is enough: a wave that runs ahead writes the set the slower waves are not reading
// (they finished with it before the barrier in between).
__device__ __forceinline__ float block_sum(float v, float* red, int tid, int& k) {
  v = wave_sum(v);
  float* set = red + (k & 1) * RN_WAVES;
  ++k;
  if ((tid & 63) == 0) set[tid >> 6] = v;
  __syncthreads();
  float s = set[0];
#pragma unroll
  for (int w = 1; w < RN_WAVES; ++w) s += set[w];
  return s;
}

struct RowNormParams {
  const float* x;        // LN input (DQ = false)
  const int32_t* acc;    // DQ: int32 accumulator
  const float* resid_in; // DQ
  float* resid_out;      // DQ
  int64_t x_rs, acc_rs, rin_rs, rout_rs, y_rs, ln_rs;
  float in_scale;
  const float* in_scale_dev;  // when given, the dequantisation scale is read from device memory
  const float* gamma;
  const float* beta;
  float eps;
  int8_t* y;
  float* ln_out;
  float* mean_out;
  float* rstd_out;
  int rows, cols, rms, round_mode;
};

__device__ __forceinline__ float norm_one(float x, float mean, float rstd, float w, float b, bool has_b) {
  // kernels/fused.py:323-327: a_hat = (a - mean) * rstd; out = a_hat * weight (+ bias)
  float o = ((x - mean) * rstd) * w;
  return has_b ? o + b : o;
}

// Persistent: a workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ...  gamma and beta are
// row-invariant and stay in registers for all of them (re-reading them per row would triple the
// bytes that cross the L2 -> CU path), and for the plain LayerNorm the next row's loads are issued
// before the current row's reductions so that they are in flight during the two block-wide sums.
//
// Every access to a row goes through a buffer descriptor of that row (range-checked: vectors past the
// row's end load zeros and store nothing), so the loop has no branch around a memory instruction.  That
// matters for more than the branches: with straight-line code the compiler can count the memory
// operations between a load and its use, and the wait at the top of an iteration becomes "all but the
// stores issued since" instead of "everything", i.e. the next row's reductions no longer wait for the
// previous row's stores to be acknowledged by the L2.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_rsrc(const void* row_ptr, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)row_ptr, 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ v4f row_load_f4(__amdgpu_buffer_rsrc_t r, int vec) {
  return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, vec * 16, 0, 2));  // 2: non-temporal
}
__device__ __forceinline__ void row_store_f4(__amdgpu_buffer_rsrc_t r, int vec, v4f v) {
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, v), r, vec * 16, 0, 2);
}

template <int VPT, bool DQ>
__global__ __launch_bounds__(RN_THREADS) void rownorm_vec_kernel(RowNormParams p) {
  __shared__ float red[2 * RN_WAVES];
  int red_k = 0;
  const int tid = threadIdx.x;
  const int nvec = p.cols >> 2;
  const bool has_b = p.beta != nullptr;
  const v4f zero4 = {0.f, 0.f, 0.f, 0.f};
  const unsigned row_bytes = (unsigned)p.cols * 4u;

  v4f w[VPT], b[VPT];
  {
    const __amdgpu_buffer_rsrc_t rg = row_rsrc(p.gamma, row_bytes), rb = row_rsrc(p.beta, has_b ? row_bytes : 0u);
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      w[j] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rg, (tid + j * RN_THREADS) * 16, 0, 0));
      b[j] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(rb, (tid + j * RN_THREADS) * 16, 0, 0));
    }
  }

  // a row at or past p.rows gets an empty descriptor: its loads touch no memory
  auto load_x = [&](int row, v4f (&dst)[VPT]) {
    const bool in = row < p.rows;
    const __amdgpu_buffer_rsrc_t rx = row_rsrc(p.x + (int64_t)(in ? row : 0) * p.x_rs, in ? row_bytes : 0u);
#pragma unroll
    for (int j = 0; j < VPT; ++j) dst[j] = row_load_f4(rx, tid + j * RN_THREADS);
  };

  v4f x[VPT], xn[VPT];
  int row = blockIdx.x;
  if constexpr (!DQ) load_x(row, xn);
  const float inv_n = 1.0f / (float)p.cols;
  const bool y_vec = p.y && ((p.y_rs & 3) == 0) && ((((uintptr_t)p.y) & 3) == 0);
  float in_scale = p.in_scale;
  if constexpr (DQ) {
    if (p.in_scale_dev) in_scale = *p.in_scale_dev;
  }

  for (; row < p.rows; row += gridDim.x) {
    if constexpr (DQ) {
      const __amdgpu_buffer_rsrc_t ra = row_rsrc(p.acc + (int64_t)row * p.acc_rs, row_bytes);
      const __amdgpu_buffer_rsrc_t rr = row_rsrc(p.resid_in + (int64_t)row * p.rin_rs, row_bytes);
      const __amdgpu_buffer_rsrc_t ro = row_rsrc(p.resid_out + (int64_t)row * p.rout_rs, row_bytes);
      v4i a[VPT];
      v4f r[VPT];
#pragma unroll
      for (int j = 0; j < VPT; ++j) {
        a[j] = __builtin_amdgcn_raw_buffer_load_b128(ra, (tid + j * RN_THREADS) * 16, 0, 2);
        r[j] = row_load_f4(rr, tid + j * RN_THREADS);
      }
#pragma unroll
      for (int j = 0; j < VPT; ++j) {
        v4f o;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          // functional/fused.py:9: residual + alpha * int32 (product and sum rounded separately)
          const float prod = in_scale * (float)a[j][t];
          o[t] = r[j][t] + prod;
        }
        x[j] = o;  // vectors past the row's end: 0 + scale * 0
        row_store_f4(ro, tid + j * RN_THREADS, o);
      }
    } else {
#pragma unroll
      for (int j = 0; j < VPT; ++j) x[j] = xn[j];
      load_x(row + (int)gridDim.x, xn);
    }

    float mean = 0.0f;
    if (!p.rms) {
      float s = 0.0f;
#pragma unroll
      for (int j = 0; j < VPT; ++j) s += (x[j][0] + x[j][1]) + (x[j][2] + x[j][3]);
      mean = block_sum(s, red, tid, red_k) * inv_n;
    }
    float m2 = 0.0f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int v = tid + j * RN_THREADS;
      if (v < nvec) {
        const float d0 = x[j][0] - mean, d1 = x[j][1] - mean, d2 = x[j][2] - mean, d3 = x[j][3] - mean;
        m2 += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
      }
    }
    const float var = block_sum(m2, red, tid, red_k) * inv_n;
    const float rstd = 1.0f / sqrtf(var + p.eps);
    if (tid == 0) {
      if (p.mean_out) p.mean_out[row] = mean;
      if (p.rstd_out) p.rstd_out[row] = rstd;
    }

    const __amdgpu_buffer_rsrc_t rl = row_rsrc(p.ln_out ? p.ln_out + (int64_t)row * p.ln_rs : nullptr, p.ln_out ? row_bytes : 0u);
    const __amdgpu_buffer_rsrc_t ry = row_rsrc(p.y ? p.y + (int64_t)row * p.y_rs : nullptr, y_vec ? (unsigned)p.cols : 0u);
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int v = tid + j * RN_THREADS;
      v4f o;
#pragma unroll
      for (int t = 0; t < 4; ++t) o[t] = norm_one(x[j][t], mean, rstd, w[j][t], b[j][t], has_b);
      row_store_f4(rl, v, o);  // an empty descriptor when there is no fp32 output
      const int q0 = q8(o[0], p.round_mode), q1 = q8(o[1], p.round_mode), q2 = q8(o[2], p.round_mode),
                q3 = q8(o[3], p.round_mode);
      __builtin_amdgcn_raw_buffer_store_b32((int)pack4(q0, q1, q2, q3), ry, v * 4, 0, 2);
      if (p.y && !y_vec && v < nvec) {  // int8 rows that are not 4-byte aligned
        int8_t* dst = p.y + (int64_t)row * p.y_rs + v * 4;
        dst[0] = (int8_t)q0; dst[1] = (int8_t)q1; dst[2] = (int8_t)q2; dst[3] = (int8_t)q3;
      }
    }
  }
}

// Any column count / alignment: the row is re-read from memory for each pass (it stays in L2).
template <bool DQ>
__global__ __launch_bounds__(RN_THREADS) void rownorm_any_kernel(RowNormParams p) {
  __shared__ float red[2 * RN_WAVES];
  int red_k = 0;
  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  const float* xr;
  if constexpr (DQ) {
    const int32_t* ar = p.acc + (int64_t)row * p.acc_rs;
    const float* rin = p.resid_in + (int64_t)row * p.rin_rs;
    float* rout = p.resid_out + (int64_t)row * p.rout_rs;
    const float in_scale = p.in_scale_dev ? *p.in_scale_dev : p.in_scale;
    for (int i = tid; i < p.cols; i += RN_THREADS) {
      const float prod = in_scale * (float)ar[i];
      rout[i] = rin[i] + prod;
    }
    __threadfence_block();
    __syncthreads();
    xr = rout;
  } else {
    xr = p.x + (int64_t)row * p.x_rs;
  }
  const float inv_n = 1.0f / (float)p.cols;
  float mean = 0.0f;
  if (!p.rms) {
    float s = 0.0f;
    for (int i = tid; i < p.cols; i += RN_THREADS) s += xr[i];
    mean = block_sum(s, red, tid, red_k) * inv_n;
  }
  float m2 = 0.0f;
  for (int i = tid; i < p.cols; i += RN_THREADS) {
    const float d = xr[i] - mean;
    m2 += d * d;
  }
  const float var = block_sum(m2, red, tid, red_k) * inv_n;
  const float rstd = 1.0f / sqrtf(var + p.eps);
  if (tid == 0) {
    if (p.mean_out) p.mean_out[row] = mean;
    if (p.rstd_out) p.rstd_out[row] = rstd;
  }
  const bool has_b = p.beta != nullptr;
  for (int i = tid; i < p.cols; i += RN_THREADS) {
    const float o = norm_one(xr[i], mean, rstd, p.gamma[i], has_b ? p.beta[i] : 0.0f, has_b);
    if (p.ln_out) p.ln_out[(int64_t)row * p.ln_rs + i] = o;
    if (p.y) p.y[(int64_t)row * p.y_rs + i] = (int8_t)q8(o, p.round_mode);
  }
}

static bool aligned16(const void* ptr, int64_t row_stride_elems, int elem) {
  return (((uintptr_t)ptr) & 15) == 0 && ((row_stride_elems * elem) & 15) == 0;
}

template <bool DQ>
static int launch_rownorm(const RowNormParams& p, hipStream_t stream) {
  if (p.rows == 0 || p.cols == 0) return TI_OK;
  int rc = check_device();
  if (rc != TI_OK) return rc;
  bool vec = (p.cols & 3) == 0 && p.cols <= RN_THREADS * 4 * 8 && aligned16(p.gamma, 0, 4) &&
             (!p.beta || aligned16(p.beta, 0, 4)) && (!p.ln_out || aligned16(p.ln_out, p.ln_rs, 4));
  if (DQ) vec = vec && aligned16(p.acc, p.acc_rs, 4) && aligned16(p.resid_in, p.rin_rs, 4) && aligned16(p.resid_out, p.rout_rs, 4);
  else vec = vec && aligned16(p.x, p.x_rs, 4);
  dim3 grid((unsigned)p.rows), block(RN_THREADS);
  if (!vec) {
    rownorm_any_kernel<DQ><<<grid, block, 0, stream>>>(p);
    return launch_status("rownorm_any_kernel");
  }
  const int vpt = (p.cols / 4 + RN_THREADS - 1) / RN_THREADS;
  // persistent workgroups: a few per CU, each walking several rows.  Measured at 8192 rows with 2 / 3 / 4 / 8
  // workgroups per CU, each figure after 20 ms of the same launches (us): plain LayerNormQ of 5120 columns
  // 35.7 / 37.5 / 39.0 / 38.6, of 4096 columns 30.9 / 30.6 / 31.1 / 31.0, of 3072 columns 27.3 / 24.2 / 24.1 / 25.3,
  // of 2048 columns 22.8 / 18.8 / 17.8 / 17.5 (16384 rows: 41.7 / 34.1 / 31.0 / 33.7), of 8192 columns
  // 57.1 / 63.7 / 59.0 / 62.3; the dq + add variant of 5120 columns 89.8 / 95.8 / 96.5 / 95.4, of 4096 columns
  // 71.2 / 73.8 / 74.8 / 73.7, of 3072 columns 54.5 / 55.5 / 57.4 / 57.9, of 2048 columns 41.4 / 36.4 / 38.2 / 39.8.
  // (In the first milliseconds of a burst, while the chip's power management settles, 2 per CU is the variant
  // that suffers most: 36-45 us for the first of these where 3 per CU stay at 37-40.)
  const unsigned ln_per_cu = vpt <= 2 ? 4u : (vpt <= 4 ? 3u : 2u);
  const unsigned per_cu = DQ ? (vpt <= 2 ? 3u : 2u) : ln_per_cu;
  const unsigned slots = 256u * per_cu;
  if (grid.x > slots) grid.x = slots;
  if (vpt <= 1) rownorm_vec_kernel<1, DQ><<<grid, block, 0, stream>>>(p);
  else if (vpt <= 2) rownorm_vec_kernel<2, DQ><<<grid, block, 0, stream>>>(p);
  else if (vpt <= 3) rownorm_vec_kernel<3, DQ><<<grid, block, 0, stream>>>(p);
  else if (vpt <= 4) rownorm_vec_kernel<4, DQ><<<grid, block, 0, stream>>>(p);
  else if (vpt <= 5) rownorm_vec_kernel<5, DQ><<<grid, block, 0, stream>>>(p);
  else if (vpt <= 6) rownorm_vec_kernel<6, DQ><<<grid, block, 0, stream>>>(p);
  else rownorm_vec_kernel<8, DQ><<<grid, block, 0, stream>>>(p);
  return launch_status("rownorm_vec_kernel");
}

// ---- softmax -> int8 probabilities -------------------------------------------------------------
// y = round_half_even(softmax(x_int8 * scale) * 127), the step between the two attention BMMs of a
// W8A8 decoder layer (int8 scores in, int8 probabilities in [0,127] out).  One wavefront per row:
// a lane holds VPT x 16 consecutive int8 scores, the row maximum is exact (integers), the
// exponentials are kept in registers, and max / sum are wave reductions — no LDS, no barrier.
// With causal_q_len > 0 the rows form groups of that many query positions and position i sees
// columns 0 .. i + (cols - causal_q_len); masked columns get probability 0.
constexpr int SM_WAVES = 4;

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// exact sum over the 64 lanes of values below 2^31: the low and high 16 bits are summed separately
__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned v) {
  unsigned lo = v & 0xffffu, hi = v >> 16;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    lo += (unsigned)__shfl_xor((int)lo, off, 64);
    hi += (unsigned)__shfl_xor((int)hi, off, 64);
  }
  return ((unsigned long long)hi << 16) + lo;
}

// Rows whose start and length are multiples of 16 bytes.  Every load of a row is issued before the
// first use: buffer loads whose offset is pushed out of range for chunks beyond the causal limit
// (they return 0 without touching memory), then masking in registers.  Stores are range-checked
// buffer stores, so neither phase branches around a memory instruction.
template <int VPT>
__global__ __launch_bounds__(SM_WAVES * 64) void softmax_q_kernel(const int8_t* __restrict__ x, int64_t x_rs,
                                                                  float scale, int8_t* __restrict__ y, int64_t y_rs,
                                                                  int rows, int cols, int causal_q_len) {
  const int lane = threadIdx.x & 63;
  const int row = __builtin_amdgcn_readfirstlane(blockIdx.x * SM_WAVES + (threadIdx.x >> 6));
  if (row >= rows) return;
  const int limit = causal_q_len > 0 ? min(cols, (row % causal_q_len) + (cols - causal_q_len) + 1) : cols;
  const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc((void*)(x + (int64_t)row * x_rs), 0, cols, 0x00020000);
  const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc((void*)(y + (int64_t)row * y_rs), 0, cols, 0x00020000);
  // masked elements are -inf: they drop out of the maximum, and with scale > 0 their exponential
  // is exactly 0, so neither the sum nor the output phase has to look at the mask again
  const float NEG = -__builtin_inff();
  const int OOB = 0x7ffffff0;

  v4i w[VPT];
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (j * 64 + lane) * 16;
    w[j] = __builtin_amdgcn_raw_buffer_load_b128(rx, c0 < limit ? c0 : OOB, 0, 2);
  }
  float f[VPT][16];
  float mx = NEG;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (j * 64 + lane) * 16;
    if (c0 >= limit) continue;  // whole 1 KB pieces beyond the limit cost no VALU work
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const unsigned u = (unsigned)w[j][g];
      f[j][4 * g + 0] = sbyte_to_float<0>(u);
      f[j][4 * g + 1] = sbyte_to_float<1>(u);
      f[j][4 * g + 2] = sbyte_to_float<2>(u);
      f[j][4 * g + 3] = sbyte_to_float<3>(u);
    }
    if (c0 + 16 > limit) {  // the chunk that straddles the limit
#pragma unroll
      for (int t = 0; t < 16; ++t) f[j][t] = c0 + t < limit ? f[j][t] : NEG;
    }
#pragma unroll
    for (int t = 0; t < 16; t += 2) mx = fmaxf(fmaxf(mx, f[j][t]), f[j][t + 1]);  // v_max3_f32
  }
  mx = wave_max(mx);
  const float s2 = scale * 1.44269504088896340736f;  // exp(v) = exp2(v * log2 e)
  const float c = -(mx * s2);
  // exponentials and their exact integer sum (see ti_common.h); a lane's partial sum stays below 2^31
  unsigned bits = 0;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (j * 64 + lane) * 16;
    if (c0 >= limit) continue;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      f[j][t] = __builtin_amdgcn_exp2f(__builtin_fmaf(f[j][t], s2, c));
      bits += sm_unit_bits(f[j][t]);
    }
    bits -= 16u * SM_ONE_BITS;  // modulo 2^32, like the additions: what is left is the chunk's sum of u
  }
  const float r = sm_scale_from_sum(wave_sum_u64(bits));
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (j * 64 + lane) * 16;
    v4i o = {0, 0, 0, 0};
    if (c0 < limit) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const unsigned b0 = __float_as_uint(__builtin_fmaf(f[j][4 * g + 0], r, 12582912.0f));
        const unsigned b1 = __float_as_uint(__builtin_fmaf(f[j][4 * g + 1], r, 12582912.0f));
        const unsigned b2 = __float_as_uint(__builtin_fmaf(f[j][4 * g + 2], r, 12582912.0f));
        const unsigned b3 = __float_as_uint(__builtin_fmaf(f[j][4 * g + 3], r, 12582912.0f));
        o[g] = (int)(__builtin_amdgcn_perm(b1, b0, 0x0c0c0400u) | __builtin_amdgcn_perm(b3, b2, 0x04000c0cu));
      }
    }
    __builtin_amdgcn_raw_buffer_store_b128(o, ry, c0, 0, 2);  // dropped beyond the row's end
  }
}
template <int VPT>
__global__ __launch_bounds__(SM_WAVES * 64) void softmax_q_any_kernel(const int8_t* __restrict__ x, int64_t x_rs,
                                                                  float scale, int8_t* __restrict__ y, int64_t y_rs,
                                                                  int rows, int cols, int causal_q_len) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * SM_WAVES + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int limit = causal_q_len > 0 ? min(cols, (row % causal_q_len) + (cols - causal_q_len) + 1) : cols;
  const int8_t* xr = x + (int64_t)row * x_rs;
  int8_t* yr = y + (int64_t)row * y_rs;
  const bool vec = ((((uintptr_t)xr) | ((uintptr_t)yr)) & 15) == 0;
  const float NEG = -__builtin_inff();  // drops out of the maximum; its exponential is 0 (scale > 0) or masked below

  // f[j][t] = the score as a float, or NEG for masked / out-of-row elements
  float f[VPT][16];
  float mx = NEG;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (j * 64 + lane) * 16;
    if (c0 >= limit) {
#pragma unroll
      for (int t = 0; t < 16; ++t) f[j][t] = NEG;
    } else if (vec && c0 + 16 <= cols) {
      // a chunk that straddles the causal limit is still inside the row: load it whole and mask
      // in registers, so that no wave waits for a second, dependent round of byte loads
      v4u w = __builtin_nontemporal_load((const v4u*)(xr + c0));
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        f[j][4 * g + 0] = sbyte_to_float<0>(w[g]);
        f[j][4 * g + 1] = sbyte_to_float<1>(w[g]);
        f[j][4 * g + 2] = sbyte_to_float<2>(w[g]);
        f[j][4 * g + 3] = sbyte_to_float<3>(w[g]);
      }
      if (c0 + 16 > limit) {
#pragma unroll
        for (int t = 0; t < 16; ++t) f[j][t] = c0 + t < limit ? f[j][t] : NEG;
      }
#pragma unroll
      for (int t = 0; t < 16; t += 2) mx = fmaxf(fmaxf(mx, f[j][t]), f[j][t + 1]);  // v_max3_f32
    } else {
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        f[j][t] = c0 + t < limit ? (float)(int)xr[c0 + t] : NEG;
        mx = fmaxf(mx, f[j][t]);
      }
    }
  }
  mx = wave_max(mx);
  const float s2 = scale * 1.44269504088896340736f;  // exp(v) = exp2(v * log2 e)
  const float c = -(mx * s2);
  unsigned bits = 0;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (j * 64 + lane) * 16;
    if (c0 >= limit) continue;
#pragma unroll
    for (int t = 0; t < 16; ++t) f[j][t] = __builtin_amdgcn_exp2f(__builtin_fmaf(f[j][t], s2, c));
    if (c0 + 16 > limit) {  // the chunk that straddles the limit (or the end of the row): with scale 0 its NEG elements gave NaN
#pragma unroll
      for (int t = 0; t < 16; ++t) f[j][t] = c0 + t < limit ? f[j][t] : 0.0f;
    }
#pragma unroll
    for (int t = 0; t < 16; ++t) bits += sm_unit_bits(f[j][t]);
    bits -= 16u * SM_ONE_BITS;
  }
  const float r = sm_scale_from_sum(wave_sum_u64(bits));
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c0 = (j * 64 + lane) * 16;
    if (c0 >= cols) continue;
    v4u w = {0u, 0u, 0u, 0u};
    if (c0 < limit) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const unsigned b0 = __float_as_uint(__builtin_fmaf(f[j][4 * g + 0], r, 12582912.0f));
        const unsigned b1 = __float_as_uint(__builtin_fmaf(f[j][4 * g + 1], r, 12582912.0f));
        const unsigned b2 = __float_as_uint(__builtin_fmaf(f[j][4 * g + 2], r, 12582912.0f));
        const unsigned b3 = __float_as_uint(__builtin_fmaf(f[j][4 * g + 3], r, 12582912.0f));
        w[g] = __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u) | __builtin_amdgcn_perm(b3, b2, 0x04000c0cu);
      }
    }
    if (vec && c0 + 16 <= cols) {
      __builtin_nontemporal_store(w, (v4u*)(yr + c0));
    } else {
#pragma unroll
      for (int t = 0; t < 16; ++t)
        if (c0 + t < cols) yr[c0 + t] = (int8_t)(w[t >> 2] >> ((t & 3) * 8));
    }
  }
}

// ---- GELU -> int8 ---------------------------------------------------------------------------

constexpr int GQ_THREADS = 256;
constexpr int GQ_UNROLL = 4;

// Each workgroup converts one contiguous run of GQ_UNROLL * 256 float4 vectors (16 KB in, 4 KB
// out): every load instruction of a wave covers 1 KB, every store 256 B, all loads are issued
// before the first use, and the streams bypass the caches (non-temporal).
__global__ __launch_bounds__(GQ_THREADS) void gelu_q_vec_kernel(const float* __restrict__ x, const float* scale,
                                                                int8_t* __restrict__ y, int64_t nvec,
                                                                int round_mode) {
  const float s = *scale;
  const int64_t base = (int64_t)blockIdx.x * (GQ_THREADS * GQ_UNROLL) + threadIdx.x;
  v4f in[GQ_UNROLL];
#pragma unroll
  for (int u = 0; u < GQ_UNROLL; ++u) {
    const int64_t v = base + u * GQ_THREADS;
    if (v < nvec) in[u] = __builtin_nontemporal_load((const v4f*)x + v);
  }
#pragma unroll
  for (int u = 0; u < GQ_UNROLL; ++u) {
    const int64_t v = base + u * GQ_THREADS;
    if (v < nvec) {
      const unsigned w = pack4(q8(gelu_tanh_scaled(in[u][0], s), round_mode), q8(gelu_tanh_scaled(in[u][1], s), round_mode),
                               q8(gelu_tanh_scaled(in[u][2], s), round_mode), q8(gelu_tanh_scaled(in[u][3], s), round_mode));
      __builtin_nontemporal_store(w, (unsigned*)y + v);
    }
  }
}

__global__ __launch_bounds__(GQ_THREADS) void gelu_q_any_kernel(const float* x, const float* scale, int8_t* y,
                                                                int64_t start, int64_t n, int round_mode) {
  const float s = *scale;
  const int64_t stride = (int64_t)gridDim.x * GQ_THREADS;
  for (int64_t i = start + (int64_t)blockIdx.x * GQ_THREADS + threadIdx.x; i < n; i += stride)
    y[i] = (int8_t)q8(gelu_tanh_scaled(x[i], s), round_mode);
}

// ---- int8 2-D transpose ------------------------------------------------------------------------
// dst[c, r] = src[r, c].  64 x 64-byte tiles through LDS: 16-byte loads along the source rows,
// 16-byte stores along the destination rows (4 lanes cover a 64-byte run on both sides).
constexpr int TR_TILE = 64, TR_PITCH = TR_TILE + 4;

__global__ __launch_bounds__(256) void transpose_i8_kernel(const int8_t* __restrict__ src, int64_t src_rs,
                                                           int8_t* __restrict__ dst, int64_t dst_rs, int rows, int cols,
                                                           int vec_src, int vec_dst) {
  __shared__ __attribute__((aligned(16))) int8_t tile[TR_TILE][TR_PITCH];
  const int t = threadIdx.x;
  const int r0 = blockIdx.y * TR_TILE, c0 = blockIdx.x * TR_TILE;
  {
    const int r = t >> 2, cc = (t & 3) * 16;  // source row, first column of this thread's 16 bytes
    unsigned w[4] = {0u, 0u, 0u, 0u};
    if (r0 + r < rows) {
      const int8_t* sp = src + (int64_t)(r0 + r) * src_rs + c0 + cc;
      if (vec_src && c0 + cc + 16 <= cols) {
        const v4u v = *(const v4u*)sp;
        w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
      } else {
        for (int i = 0; i < 16; ++i)
          if (c0 + cc + i < cols) w[i >> 2] |= (unsigned)(uint8_t)sp[i] << ((i & 3) * 8);
      }
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) *(unsigned*)&tile[r][cc + 4 * g] = w[g];
  }
  __syncthreads();
  {
    const int c = t >> 2, rr = (t & 3) * 16;  // destination row (source column), first of 16 source rows
    if (c0 + c >= cols) return;
    unsigned w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 16; ++i) w[i >> 2] |= (unsigned)(uint8_t)tile[rr + i][c] << ((i & 3) * 8);
    int8_t* dp = dst + (int64_t)(c0 + c) * dst_rs + r0 + rr;
    if (vec_dst && r0 + rr + 16 <= rows) {
      *(v4u*)dp = (v4u){w[0], w[1], w[2], w[3]};
    } else {
      for (int i = 0; i < 16; ++i)
        if (r0 + rr + i < rows) dp[i] = (int8_t)(w[i >> 2] >> ((i & 3) * 8));
    }
  }
}

// KV-cache append of S new positions in one launch: blockIdx.z == 0 transposes V [S, heads*D] into
// columns of V^T [heads*D, T] (the kernel above), blockIdx.z == 1 copies K [S, heads*D] into the
// head-major cache [heads, T, D], 16 bytes per thread (D % 16 == 0).
__global__ __launch_bounds__(256) void kv_append_i8_kernel(const int8_t* __restrict__ k_src, int64_t k_rs,
                                                           const int8_t* __restrict__ v_src, int64_t v_rs,
                                                           int8_t* __restrict__ k_dst, int64_t k_head_stride,
                                                           int8_t* __restrict__ vt_dst, int64_t vt_rs, int S, int H, int D,
                                                           int vec) {
  if (blockIdx.z == 0) {
    __shared__ __attribute__((aligned(16))) int8_t tile[TR_TILE][TR_PITCH];
    const int t = threadIdx.x;
    const int r0 = blockIdx.y * TR_TILE, c0 = blockIdx.x * TR_TILE;
    {
      const int r = t >> 2, cc = (t & 3) * 16;
      unsigned w[4] = {0u, 0u, 0u, 0u};
      if (r0 + r < S && c0 + cc < H) {  // H % 16 == 0: a chunk is inside or outside
        const int8_t* sp = v_src + (int64_t)(r0 + r) * v_rs + c0 + cc;
        if (vec) {
          const v4u v = *(const v4u*)sp;
          w[0] = v[0]; w[1] = v[1]; w[2] = v[2]; w[3] = v[3];
        } else {
          for (int i = 0; i < 16; ++i) w[i >> 2] |= (unsigned)(uint8_t)sp[i] << ((i & 3) * 8);
        }
      }
#pragma unroll
      for (int g = 0; g < 4; ++g) *(unsigned*)&tile[r][cc + 4 * g] = w[g];
    }
    __syncthreads();
    const int c = t >> 2, rr = (t & 3) * 16;
    if (c0 + c >= H) return;
    unsigned w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 16; ++i) w[i >> 2] |= (unsigned)(uint8_t)tile[rr + i][c] << ((i & 3) * 8);
    int8_t* dp = vt_dst + (int64_t)(c0 + c) * vt_rs + r0 + rr;
    if (vec && r0 + rr + 16 <= S) {
      *(v4u*)dp = (v4u){w[0], w[1], w[2], w[3]};
    } else {
      for (int i = 0; i < 16; ++i)
        if (r0 + rr + i < S) dp[i] = (int8_t)(w[i >> 2] >> ((i & 3) * 8));
    }
  } else {
    const int t = threadIdx.x;
    const int r = blockIdx.y * TR_TILE + (t >> 2), c = blockIdx.x * TR_TILE + (t & 3) * 16;
    if (r >= S || c >= H) return;
    const int8_t* sp = k_src + (int64_t)r * k_rs + c;
    int8_t* dp = k_dst + (int64_t)(c / D) * k_head_stride + (int64_t)r * D + (c % D);
    if (vec) {
      *(v4u*)dp = *(const v4u*)sp;
    } else {
      for (int i = 0; i < 16; ++i) dp[i] = sp[i];
    }
  }
}

}  // namespace ti

extern "C" {

int ti_layernorm_q(const float* x, int64_t x_row_stride, const float* gamma, const float* beta, float eps,
                   int8_t* y, int64_t y_row_stride, int rows, int cols, int rms, int round_mode, float* mean_out,
                   float* rstd_out, void* stream) {
  if (rows < 0 || cols < 0) return ti::fail(TI_E_SHAPE, "negative size");
  if (rows == 0 || cols == 0) return TI_OK;
  if (!x || !gamma || !y) return ti::fail(TI_E_NULL, "x, gamma and y are required");
  if (round_mode != TI_ROUND_RNE_CLAMP && round_mode != TI_ROUND_TRUNC) return ti::fail(TI_E_COMBO, "round mode %d", round_mode);
  ti::RowNormParams p = {};
  p.x = x; p.x_rs = x_row_stride;
  p.gamma = gamma; p.beta = beta; p.eps = eps;
  p.y = y; p.y_rs = y_row_stride;
  p.rows = rows; p.cols = cols; p.rms = rms; p.round_mode = round_mode;
  p.mean_out = mean_out; p.rstd_out = rstd_out;
  return ti::launch_rownorm<false>(p, (hipStream_t)stream);
}

int ti_dq_add_layernorm_q(const int32_t* acc, int64_t acc_row_stride, float in_scale, const float* in_scale_dev,
                          const float* resid_in, int64_t resid_in_row_stride, const float* gamma, const float* beta, float eps,
                          float* resid_out, int64_t resid_out_row_stride, int8_t* y, int64_t y_row_stride,
                          float* ln_out_f32, int64_t ln_out_row_stride, int rows, int cols, int round_mode,
                          float* mean_out, float* rstd_out, void* stream) {
  if (rows < 0 || cols < 0) return ti::fail(TI_E_SHAPE, "negative size");
  if (rows == 0 || cols == 0) return TI_OK;
  if (!acc || !resid_in || !resid_out || !gamma) return ti::fail(TI_E_NULL, "acc, resid_in, resid_out and gamma are required");
  if (!y && !ln_out_f32) return ti::fail(TI_E_NULL, "one of y / ln_out_f32 is required");
  if (round_mode != TI_ROUND_RNE_CLAMP && round_mode != TI_ROUND_TRUNC) return ti::fail(TI_E_COMBO, "round mode %d", round_mode);
  ti::RowNormParams p = {};
  p.acc = acc; p.acc_rs = acc_row_stride; p.in_scale = in_scale; p.in_scale_dev = in_scale_dev;
  p.resid_in = resid_in; p.rin_rs = resid_in_row_stride;
  p.resid_out = resid_out; p.rout_rs = resid_out_row_stride;
  p.gamma = gamma; p.beta = beta; p.eps = eps;
  p.y = y; p.y_rs = y_row_stride;
  p.ln_out = ln_out_f32; p.ln_rs = ln_out_row_stride;
  p.rows = rows; p.cols = cols; p.rms = 0; p.round_mode = round_mode;
  p.mean_out = mean_out; p.rstd_out = rstd_out;
  return ti::launch_rownorm<true>(p, (hipStream_t)stream);
}

int ti_softmax_q(const int8_t* x, int64_t x_row_stride, float scale, int8_t* y, int64_t y_row_stride, int rows,
                 int cols, int causal_q_len, void* stream) {
  if (rows < 0 || cols < 0 || causal_q_len < 0) return ti::fail(TI_E_SHAPE, "negative size");
  if (rows == 0 || cols == 0) return TI_OK;
  if (!x || !y) return ti::fail(TI_E_NULL, "x and y are required");
  if (causal_q_len > cols) return ti::fail(TI_E_SHAPE, "causal_q_len %d > cols %d", causal_q_len, cols);
  if (causal_q_len > 0 && rows % causal_q_len) return ti::fail(TI_E_SHAPE, "rows %d not a multiple of causal_q_len %d", rows, causal_q_len);
  if (cols > 64 * 16 * 8) return ti::fail(TI_E_SHAPE, "softmax rows longer than 8192 are not supported");
  if (!(scale >= 0.0f)) return ti::fail(TI_E_COMBO, "the score scale must be >= 0 (the exponent is taken against the row's largest score)");
  if (scale > ti::SM_MAX_SCALE) return ti::fail(TI_E_COMBO, "score scale %g above %g: the quantised softmax is exact up to that scale only", (double)scale, (double)ti::SM_MAX_SCALE);
  int rc = ti::check_device();
  if (rc != TI_OK) return rc;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)((rows + ti::SM_WAVES - 1) / ti::SM_WAVES)), block(ti::SM_WAVES * 64);
  const int vpt = (cols + 1023) / 1024;
  const bool aligned = ((((uintptr_t)x) | ((uintptr_t)y) | (uintptr_t)x_row_stride | (uintptr_t)y_row_stride | (uintptr_t)cols) & 15) == 0;
#define TI_SOFTMAX_LAUNCH(KERNEL)                                                                          \
  do {                                                                                                     \
    if (vpt <= 1) KERNEL<1><<<grid, block, 0, s>>>(x, x_row_stride, scale, y, y_row_stride, rows, cols, causal_q_len);      \
    else if (vpt <= 2) KERNEL<2><<<grid, block, 0, s>>>(x, x_row_stride, scale, y, y_row_stride, rows, cols, causal_q_len); \
    else if (vpt <= 4) KERNEL<4><<<grid, block, 0, s>>>(x, x_row_stride, scale, y, y_row_stride, rows, cols, causal_q_len); \
    else KERNEL<8><<<grid, block, 0, s>>>(x, x_row_stride, scale, y, y_row_stride, rows, cols, causal_q_len);               \
  } while (0)
  if (aligned && scale > 0.0f) TI_SOFTMAX_LAUNCH(ti::softmax_q_kernel);
  else TI_SOFTMAX_LAUNCH(ti::softmax_q_any_kernel);
#undef TI_SOFTMAX_LAUNCH
  return ti::launch_status("softmax_q_kernel");
}

int ti_gelu_q(const float* x, const float* scale, int8_t* y, int64_t n, int round_mode, void* stream) {
  if (n < 0) return ti::fail(TI_E_SHAPE, "negative size");
  if (n == 0) return TI_OK;
  if (!x || !scale || !y) return ti::fail(TI_E_NULL, "x, scale and y are required");
  if (round_mode != TI_ROUND_RNE_CLAMP && round_mode != TI_ROUND_TRUNC) return ti::fail(TI_E_COMBO, "round mode %d", round_mode);
  int rc = ti::check_device();
  if (rc != TI_OK) return rc;
  hipStream_t s = (hipStream_t)stream;
  int64_t done = 0;
  if ((((uintptr_t)x) & 15) == 0 && (((uintptr_t)y) & 3) == 0 && n >= 4) {
    const int64_t nvec = n / 4;
    const int64_t blocks = (nvec + ti::GQ_THREADS * ti::GQ_UNROLL - 1) / (ti::GQ_THREADS * ti::GQ_UNROLL);
    if (blocks > 0x7fffffff) return ti::fail(TI_E_SHAPE, "n too large");
    ti::gelu_q_vec_kernel<<<dim3((unsigned)blocks), dim3(ti::GQ_THREADS), 0, s>>>(x, scale, y, nvec, round_mode);
    rc = ti::launch_status("gelu_q_vec_kernel");
    if (rc != TI_OK) return rc;
    done = nvec * 4;
  }
  if (done < n) {
    int64_t blocks = (n - done + ti::GQ_THREADS - 1) / ti::GQ_THREADS;
    if (blocks > 256 * 16) blocks = 256 * 16;
    ti::gelu_q_any_kernel<<<dim3((unsigned)blocks), dim3(ti::GQ_THREADS), 0, s>>>(x, scale, y, done, n, round_mode);
    rc = ti::launch_status("gelu_q_any_kernel");
  }
  return rc;
}

int ti_transpose_i8(const int8_t* src, int64_t src_row_stride, int8_t* dst, int64_t dst_row_stride, int rows,
                    int cols, void* stream) {
  if (rows < 0 || cols < 0) return ti::fail(TI_E_SHAPE, "negative size");
  if (rows == 0 || cols == 0) return TI_OK;
  if (!src || !dst) return ti::fail(TI_E_NULL, "src and dst are required");
  int rc = ti::check_device();
  if (rc != TI_OK) return rc;
  const int vec_src = ((((uintptr_t)src) | (uintptr_t)(src_row_stride)) & 15) == 0;
  const int vec_dst = ((((uintptr_t)dst) | (uintptr_t)(dst_row_stride)) & 15) == 0;
  dim3 grid((unsigned)((cols + ti::TR_TILE - 1) / ti::TR_TILE), (unsigned)((rows + ti::TR_TILE - 1) / ti::TR_TILE));
  if (grid.y > 65535) return ti::fail(TI_E_SHAPE, "more than 65535 * 64 rows");
  ti::transpose_i8_kernel<<<grid, dim3(256), 0, (hipStream_t)stream>>>(src, src_row_stride, dst, dst_row_stride, rows,
                                                                    cols, vec_src, vec_dst);
  return ti::launch_status("transpose_i8_kernel");
}

int ti_kv_append_i8(const int8_t* k_src, int64_t k_src_row_stride, const int8_t* v_src, int64_t v_src_row_stride,
                    int8_t* k_dst, int64_t k_head_stride, int8_t* vt_dst, int64_t vt_row_stride, int S, int heads, int D,
                    void* stream) {
  if (S < 0 || heads < 0 || D < 0) return ti::fail(TI_E_SHAPE, "negative size");
  if (S == 0 || heads == 0 || D == 0) return TI_OK;
  if (!k_src || !v_src || !k_dst || !vt_dst) return ti::fail(TI_E_NULL, "k_src, v_src, k_dst and vt_dst are required");
  if (D & 15) return ti::fail(TI_E_SHAPE, "head dimension %d must be a multiple of 16", D);
  const int64_t H = (int64_t)heads * D;
  if (H > 0x7fffffff) return ti::fail(TI_E_SHAPE, "heads * D too large");
  if (k_src_row_stride < H || v_src_row_stride < H || vt_row_stride < S || k_head_stride < (int64_t)S * D)
    return ti::fail(TI_E_STRIDE, "strides must cover the rows they step over");
  int rc = ti::check_device();
  if (rc != TI_OK) return rc;
  const int vec = ((((uintptr_t)k_src) | ((uintptr_t)v_src) | ((uintptr_t)k_dst) | ((uintptr_t)vt_dst) |
                    (uintptr_t)k_src_row_stride | (uintptr_t)v_src_row_stride | (uintptr_t)k_head_stride |
                    (uintptr_t)vt_row_stride) & 15) == 0;
  dim3 grid((unsigned)((H + ti::TR_TILE - 1) / ti::TR_TILE), (unsigned)((S + ti::TR_TILE - 1) / ti::TR_TILE), 2);
  if (grid.y > 65535) return ti::fail(TI_E_SHAPE, "more than 65535 * 64 positions");
  ti::kv_append_i8_kernel<<<grid, dim3(256), 0, (hipStream_t)stream>>>(k_src, k_src_row_stride, v_src, v_src_row_stride, k_dst,
                                                                    k_head_stride, vt_dst, vt_row_stride, S, (int)H, D, vec);
  return ti::launch_status("kv_append_i8_kernel");
}

}  // extern "C"
