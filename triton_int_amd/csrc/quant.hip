// quant.hip — dynamic per-token activation quantisation (functional/quantization.py:61-67):
//     max_val = clamp(max_j |t[r, j]|, min = 1e-8) / 127        (in t's dtype)
//     q[r, j] = clamp(round_half_even(t[r, j] / max_val[r]), -128, 127) -> int8
// for fp32 and fp16 activations.  Every step is rounded to the tensor's dtype as torch's elementwise
// kernels do (fp16: computed in fp32, rounded to fp16 after the clamp, after the division by 127 and
// after the division of each element), so the int8 result and the scale are bit-identical to the
// reference helper's.  One workgroup per row.  Aligned rows of up to 32768 elements are
// held in registers between the maximum and the quantisation (one read: 5 bytes of HBM traffic per
// fp32 element, 3 per fp16 element); other rows are read twice.
#include <type_traits>

#include "ti_common.h"

namespace ti {

constexpr int QT_THREADS = 256;

template <typename T>
struct QtVec;
template <>
struct QtVec<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <>
struct QtVec<_Float16> { typedef _Float16 type __attribute__((ext_vector_type(4))); };

// `red` holds two sets of per-wave maxima that consecutive rows (counted by `k`) alternate between, so one
// barrier per row is enough: a wave that runs ahead writes the set the slower waves are not reading
__device__ __forceinline__ float block_max(float v, float* red, int tid, int& k) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  float* set = red + (k & 1) * (QT_THREADS / 64);
  ++k;
  if ((tid & 63) == 0) set[tid >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(set[0], set[1]), fmaxf(set[2], set[3]));
}

// x / s for a whole row of x, correctly rounded like the division instruction sequence the compiler emits
// for `x / s`, at half its cost per element.  That sequence is: scale both operands into a safe range,
// r = refined reciprocal of the divisor (v_rcp_f32 and one Newton step: two fma), then for the dividend
// q0 = n * r, two residual corrections (four fma, the last one carrying the range scaling back), and a
// fix-up of the special cases.  The reciprocal part depends on the divisor only, so a row computes it once;
// with the divisor in [2^-100, 2^100] and |n| not far above it (here |n / s| <= 127) no operand needs the
// range scaling and no special case arises, and the five per-element operations below are the same five,
// on the same values: the same bits.  Divisors outside that range (an all-zero row in fp16, infinities) take
// the ordinary division.
struct RowDivisor {
  float s, r;
  bool direct;
  __device__ __forceinline__ explicit RowDivisor(float s_) : s(s_) {
    direct = s_ >= 0x1p-100f && s_ <= 0x1p100f;
    const float r0 = __builtin_amdgcn_rcpf(s_);
    const float e0 = __builtin_fmaf(-s_, r0, 1.0f);
    r = __builtin_fmaf(e0, r0, r0);
  }
  template <bool DIRECT>
  __device__ __forceinline__ float divide(float n) const {
    if constexpr (!DIRECT) return n / s;
    const float q0 = n * r;
    const float e1 = __builtin_fmaf(-s, q0, n);
    const float q1 = __builtin_fmaf(e1, r, q0);
    const float e2 = __builtin_fmaf(-s, q1, n);
    return __builtin_fmaf(e2, r, q1);
  }
};

// t.div_(max_val) rounded to T, round_() (half to even, exact in T), clamp_(-128, 127), to int8.  For fp16 the
// rounding and the clamp run on the half itself (no trip back to fp32).  A NaN quotient gives -128; finite
// rows never produce one.
template <typename T, bool DIRECT>
__device__ __forceinline__ int quant_one(const RowDivisor& by_scale, T v) {
  const T d = (T)by_scale.template divide<DIRECT>((float)v);
  if constexpr (std::is_same<T, _Float16>::value) {
    const _Float16 r = __builtin_rintf16(d);
    const _Float16 c = __builtin_fminf16(__builtin_fmaxf16(r, (_Float16)-128.0f), (_Float16)127.0f);
    return (int)(short)c;
  } else {
    const float r = __builtin_rintf((float)d);
    return (int)fminf(fmaxf(r, -128.0f), 127.0f);
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(QT_THREADS) void quant_per_token_kernel(const T* __restrict__ x, int64_t x_rs,
                                                                     int8_t* __restrict__ q, int64_t q_rs,
                                                                     T* __restrict__ scale_out, int rows, int cols) {
  typedef typename QtVec<T>::type V4;
  __shared__ float red[2 * (QT_THREADS / 64)];
  int red_k = 0;
  const int tid = threadIdx.x;
  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
    const T* xr = x + (int64_t)row * x_rs;
    int8_t* qr = q + (int64_t)row * q_rs;
    float m = 0.0f;
    if constexpr (VEC) {
      for (int c = tid * 4; c < cols; c += QT_THREADS * 4) {
        const V4 v = *(const V4*)(xr + c);
        m = fmaxf(fmaxf(m, fabsf((float)v[0])), fmaxf(fabsf((float)v[1]), fmaxf(fabsf((float)v[2]), fabsf((float)v[3]))));
      }
    } else {
      for (int c = tid; c < cols; c += QT_THREADS) m = fmaxf(m, fabsf((float)xr[c]));
    }
    m = block_max(m, red, tid, red_k);
    // clamp(min = 1e-8) and the division by 127, each rounded to T
    const T clamped = (T)fmaxf(m, 1e-8f);
    const T scale = (T)((float)clamped / 127.0f);
    if (tid == 0 && scale_out) scale_out[row] = scale;
    const RowDivisor by_scale((float)scale);
    // the choice of the division is the row's, not the element's: one branch per row, two copies of the loop
    auto quantise_row = [&](auto direct_tag) {
      constexpr bool DIRECT = decltype(direct_tag)::value;
      auto one = [&](T v) -> int { return quant_one<T, DIRECT>(by_scale, v); };
      if constexpr (VEC) {
        for (int c = tid * 4; c < cols; c += QT_THREADS * 4) {
          const V4 v = *(const V4*)(xr + c);
          *(unsigned*)(qr + c) = pack4(one(v[0]), one(v[1]), one(v[2]), one(v[3]));
        }
      } else {
        for (int c = tid; c < cols; c += QT_THREADS) qr[c] = (int8_t)one(xr[c]);
      }
    };
    if (by_scale.direct) quantise_row(std::true_type{});
    else quantise_row(std::false_type{});
  }
}

// Rows of up to 256 * 4 * VPT elements whose 4-element groups are aligned: the row is read once
// into registers (all loads issued before the first use), reduced, and quantised from there.
template <typename T, int VPT>
__global__ __launch_bounds__(QT_THREADS) void quant_per_token_reg_kernel(const T* __restrict__ x, int64_t x_rs,
                                                                         int8_t* __restrict__ q, int64_t q_rs,
                                                                         T* __restrict__ scale_out, int rows, int cols) {
  typedef typename QtVec<T>::type V4;
  __shared__ float red[2 * (QT_THREADS / 64)];
  int red_k = 0;
  const int tid = threadIdx.x;
  const int nvec = cols >> 2;
  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
    const V4* xr = (const V4*)(x + (int64_t)row * x_rs);
    unsigned* qr = (unsigned*)(q + (int64_t)row * q_rs);
    V4 xv[VPT];
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
      const int v = tid + j * QT_THREADS;
      if (v < nvec) xv[j] = __builtin_nontemporal_load(xr + v);
      else xv[j] = (V4){(T)0, (T)0, (T)0, (T)0};
    }
    float m = 0.0f;
#pragma unroll
    for (int j = 0; j < VPT; ++j)
      m = fmaxf(fmaxf(m, fabsf((float)xv[j][0])), fmaxf(fabsf((float)xv[j][1]), fmaxf(fabsf((float)xv[j][2]), fabsf((float)xv[j][3]))));
    m = block_max(m, red, tid, red_k);
    const T clamped = (T)fmaxf(m, 1e-8f);
    const T scale = (T)((float)clamped / 127.0f);
    if (tid == 0 && scale_out) scale_out[row] = scale;
    const RowDivisor by_scale((float)scale);
    auto quantise_row = [&](auto direct_tag) {
      constexpr bool DIRECT = decltype(direct_tag)::value;
      auto one = [&](T v) -> int { return quant_one<T, DIRECT>(by_scale, v); };
#pragma unroll
      for (int j = 0; j < VPT; ++j) {
        const int v = tid + j * QT_THREADS;
        if (v < nvec) __builtin_nontemporal_store(pack4(one(xv[j][0]), one(xv[j][1]), one(xv[j][2]), one(xv[j][3])), qr + v);
      }
    };
    if (by_scale.direct) quantise_row(std::true_type{});
    else quantise_row(std::false_type{});
  }
}

template <typename T>
static int launch_quant(const void* x, int64_t x_rs, int8_t* q, int64_t q_rs, void* scale_out, int rows, int cols,
                        hipStream_t stream) {
  // one workgroup per row: workgroups that retire after their row leave the balancing to the dispatcher and never
  // wait for their own stores (8192 x 20480: fp16 85 us against 100-110 us for 8 persistent workgroups per CU, fp32
  // 139 against 145 us); the loops below only matter beyond 2^20 rows
  const unsigned grid = (unsigned)(rows < (1 << 20) ? rows : (1 << 20));
  const bool vec = (cols & 3) == 0 && (x_rs & 3) == 0 && (q_rs & 3) == 0 && (((uintptr_t)x) & (4 * sizeof(T) - 1)) == 0 &&
                   (((uintptr_t)q) & 3) == 0;
  const int vpt = (cols / 4 + QT_THREADS - 1) / QT_THREADS;
  if (vec && vpt <= 32) {
#define TI_QT_LAUNCH(V) quant_per_token_reg_kernel<T, V><<<dim3(grid), dim3(QT_THREADS), 0, stream>>>((const T*)x, x_rs, q, q_rs, (T*)scale_out, rows, cols)
    if (vpt <= 1) TI_QT_LAUNCH(1);
    else if (vpt <= 2) TI_QT_LAUNCH(2);
    else if (vpt <= 4) TI_QT_LAUNCH(4);
    else if (vpt <= 5) TI_QT_LAUNCH(5);
    else if (vpt <= 8) TI_QT_LAUNCH(8);
    else if (vpt <= 12) TI_QT_LAUNCH(12);
    else if (vpt <= 16) TI_QT_LAUNCH(16);
    else if (vpt <= 20) TI_QT_LAUNCH(20);
    else if (vpt <= 24) TI_QT_LAUNCH(24);
    else TI_QT_LAUNCH(32);
#undef TI_QT_LAUNCH
    return launch_status("quant_per_token_reg_kernel");
  }
  if (vec)
    quant_per_token_kernel<T, true><<<dim3(grid), dim3(QT_THREADS), 0, stream>>>((const T*)x, x_rs, q, q_rs, (T*)scale_out, rows, cols);
  else
    quant_per_token_kernel<T, false><<<dim3(grid), dim3(QT_THREADS), 0, stream>>>((const T*)x, x_rs, q, q_rs, (T*)scale_out, rows, cols);
  return launch_status("quant_per_token_kernel");
}

}  // namespace ti

extern "C" int ti_quantize_per_token_absmax(const void* x, int x_dtype, int64_t x_row_stride, int8_t* q,
                                            int64_t q_row_stride, void* scale_out, int rows, int cols, void* stream) {
  using namespace ti;
  if (rows < 0 || cols < 0) return fail(TI_E_SHAPE, "negative size");
  if (rows == 0 || cols == 0) return TI_OK;
  if (!x || !q) return fail(TI_E_NULL, "x and q are required");
  if (x_dtype != TI_F32 && x_dtype != TI_F16) return fail(TI_E_COMBO, "activation dtype %d: fp32 or fp16", x_dtype);
  if (x_row_stride < cols || q_row_stride < cols) return fail(TI_E_STRIDE, "row strides must cover a row");
  int rc = check_device();
  if (rc != TI_OK) return rc;
  if (x_dtype == TI_F32) return launch_quant<float>(x, x_row_stride, q, q_row_stride, scale_out, rows, cols, (hipStream_t)stream);
  return launch_quant<_Float16>(x, x_row_stride, q, q_row_stride, scale_out, rows, cols, (hipStream_t)stream);
}
