/*
 * triton_int_hip.h — C ABI of libtriton_int_hip.so (gfx950 / MI355X only).
 *
 * Every entry point takes raw device pointers, element strides, sizes and a HIP
 * stream handle (passed as void*; NULL = the null stream).  Nothing here knows
 * about torch.  All calls only enqueue work on `stream` and return; there is no
 * host synchronisation.  Return value: 0 = ok, <0 = invalid argument (TI_E_*),
 * >0 = a hipError_t from the launch.  ti_last_error() returns a thread-local
 * message for the last non-zero return.
 *
 * Each entry point names the reference interface (file:line in
 * zhanglei1172/triton_int) whose Triton launch it replaces.
 *
 * Arithmetic contract shared by all GEMM/BMM epilogues:
 *   acc      exact int32  sum_k a[m,k] * b[n,k]
 *   f(.)     int32 -> fp32 conversion, round-to-nearest-even
 *   all fp32 products and sums are separately rounded (no FMA contraction)
 *   q8(v)    TI_ROUND_RNE_CLAMP: clamp(round_half_even(v), -128, 127)
 *            TI_ROUND_TRUNC    : clamp(trunc(v), -128, 127)  (literal Triton `.to(int8)`
 *                                on in-range values; test-time switch only, always served by
 *                                the slow gather kernel)
 *            The result for a NaN v (possible only with non-finite scales) is unspecified.
 */
#ifndef TRITON_INT_HIP_H
#define TRITON_INT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- enums (plain ints in the ABI) ------------------------------------------------- */

enum ti_epilogue {
  /* C_i32 = acc (+ bias_i32[n])
   *   kernels/linear.py:433-566 (linear_a8_w8_b32_o32), kernels/bmm.py:163-311
   *   (bmm_s8t_s8n_s32t), kernels/bmm.py:12-160 (bmm_s8t_s8t_s32t) */
  TI_EPI_I32 = 0,
  /* C_i32 = cvt_i32(alpha*f(acc) + beta*f(bias_i32[n]))
   *   kernels/linear.py:569-708 (linear_a8_w8_b32_o32_with_scaling) */
  TI_EPI_SCALE_I32 = 1,
  /* C_i8 = q8(alpha*f(acc) + beta*f(bias_i8[n]))   (bias optional)
   *   kernels/linear.py:150-288 (linear_a8_w8_b8_o8), kernels/bmm.py:467-612
   *   (bmm_s8t_s8n_s8t), kernels/bmm.py:615-760 (bmm_s8t_s8t_s8t) */
  TI_EPI_SCALE_I8 = 2,
  /* C_i8 = max(q8(...), 0)   kernels/linear.py:291-430 (linear_relu_a8_w8_b8_o8) */
  TI_EPI_SCALE_RELU_I8 = 3,
  /* C_f = alpha*f(acc) + beta*bias_f32[n]  -> f32 / f16 / bf16   (bias optional)
   *   kernels/linear.py:711-853 (linear_a8_w8_bfp32_ofp32), kernels/linear.py:24-147
   *   (linear_a8_w8_ofp32), kernels/bmm.py:314-464 (bmm_s8t_s8n_f32t) */
  TI_EPI_SCALE_F = 4,
  /* x = alpha*f(acc) + bias_f32[n];  C_i8 = q8(0.5*x*(1+tanh(sqrt(2/pi)*(x+0.044715*x^3)))*beta)
   *   kernels/fused.py:76-79,88-231 (linear_a8_w8_bfp32_ofp32_GeLu_Q) */
  TI_EPI_GELU_I8 = 5,
  TI_EPI_COUNT_ = 6
};

enum ti_dtype { TI_I8 = 0, TI_I32 = 1, TI_F32 = 2, TI_F16 = 3, TI_BF16 = 4 };
/* TI_BIAS_F16 / TI_BIAS_BF16: TI_EPI_SCALE_F only; the elements are widened to fp32 exactly, i.e. the
 * result is that of passing bias.float() (the reference's launcher takes the bias in the output's
 * dtype, kernels/linear.py:830-832, and its kernel widens it on load, :786-790). */
enum ti_bias { TI_BIAS_NONE = 0, TI_BIAS_I8 = 1, TI_BIAS_I32 = 2, TI_BIAS_F32 = 3, TI_BIAS_F16 = 4, TI_BIAS_BF16 = 5 };
enum ti_round { TI_ROUND_RNE_CLAMP = 0, TI_ROUND_TRUNC = 1 };

enum ti_status {
  TI_OK = 0,
  TI_E_NULL = -1,      /* a required pointer is NULL */
  TI_E_SHAPE = -2,     /* negative size, or size beyond what the kernels index with int32 */
  TI_E_COMBO = -3,     /* epilogue / out dtype / bias kind combination not defined */
  TI_E_STRIDE = -4,    /* stride not usable (zero/negative stride on an output, ...) */
  TI_E_DEVICE = -5     /* current device is not gfx950 */
};

/* ---- library ----------------------------------------------------------------------- */

/* ABI version, bumped when a signature changes. */
int ti_version(void);
/* Message for the last non-zero status returned on the calling thread ("" if none). */
const char* ti_last_error(void);

/*
 * Measurement aid, no counterpart in the reference: enqueues a kernel that issues `iters` x 8
 * independent v_mfma_i32_32x32x32_i8 per wavefront on register operands (constant bytes, or
 * pseudo-random bytes when random_operands != 0) with no memory traffic.  *ops_out (host, may be
 * NULL) receives the int8 ops of the launch (2*M*N*K convention); the caller times it.  Gives
 * the matrix-pipe rate at the clock the chip actually sustains, which a benchmark reports beside
 * the nominal peak.
 */
int ti_mfma_i8_probe(int iters, int random_operands, void* stream, double* ops_out);

/* ---- int8 GEMM / BMM --------------------------------------------------------------- */

/*
 * Batched C[b,m,n] = epilogue( sum_k A[b,m,k] * B[b,n,k] ).
 *
 * Replaces every int8 Triton launcher in kernels/linear.py:117-853, kernels/bmm.py:125-760
 * and kernels/fused.py:197-231.  A linear is batch = 1.  All strides are in ELEMENTS and
 * arbitrary (the reference forwards tensor strides, kernels/linear.py:281-286,
 * kernels/bmm.py:139-151); the "[B,K,N]" operand of bmm_s8t_s8t_* is expressed by
 * sBn = 1, sBk = N.  The fastest kernels are used when sAk == sBk == 1, K % 16 == 0,
 * row/batch strides are multiples of 16 and base pointers are 16-byte aligned; any other
 * stride pattern runs a slower byte-gather kernel with identical results.
 *
 * alpha, beta: DEVICE pointers to one fp32 each (the reference loads its 0-dim scale
 * tensors inside the kernel, kernels/linear.py:227,247).  beta may be NULL when bias is
 * TI_BIAS_NONE; alpha may be NULL for TI_EPI_I32.
 * bias: device pointer to N contiguous elements of `bias_kind`, or NULL/TI_BIAS_NONE.
 * M, N or batch equal to 0 is a no-op; K == 0 gives acc = 0.
 */
int ti_bmm_i8(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk,
              const int8_t* B, int64_t sBb, int64_t sBn, int64_t sBk,
              void* C, int64_t sCb, int64_t sCm, int64_t sCn,
              int batch, int M, int N, int K,
              const void* bias, int bias_kind,
              const float* alpha, const float* beta,
              int epilogue, int out_dtype, int round_mode,
              void* stream);

/*
 * Same as ti_bmm_i8 but forces one kernel configuration (index into the library's tile
 * table; see ti_gemm_num_configs / ti_gemm_config_name).  Used by the tuner and the
 * parity tests so that every configuration is checked, not only the one the dispatcher
 * would pick.  config = -1 selects automatically.  Bits 8..15 of a non-negative config force
 * the number of K splits of a wave-specialised ("ws_") configuration (0 = choose; bits 0..7 equal
 * to 0xff = choose the configuration): K is dealt to that many work items per tile, whose int32
 * partial sums meet in a workspace the library keeps per device and stream (allocated on first
 * use, up to 96 MiB; never during a graph capture, where an unsplit launch is used if there is
 * none yet).  Integer sums: the result does not depend on the split.  For the M <= 16
 * weight-streaming configuration ("rows4_m16") the same bits select its wave layout instead: low
 * nibble the number of waves that share a unit of weight rows along K (1, 2, 4, 8), high nibble
 * the number of streaming waves (4, 6, 8); 0 = choose.  Returns TI_E_COMBO if the configuration
 * cannot run the given shape or stride pattern (e.g. "shortk_..." takes 16 <= K <= 128 and, for
 * int8 outputs, neither bias nor GELU) or cannot split K that way.
 */
int ti_bmm_i8_config(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk,
                     const int8_t* B, int64_t sBb, int64_t sBn, int64_t sBk,
                     void* C, int64_t sCb, int64_t sCm, int64_t sCn,
                     int batch, int M, int N, int K,
                     const void* bias, int bias_kind,
                     const float* alpha, const float* beta,
                     int epilogue, int out_dtype, int round_mode,
                     int config, void* stream);
/*
 * Grouped form: the batches are different projections rather than slices of one operand.  Batch b
 * adds bias elements [b * bias_batch_stride, b * bias_batch_stride + N) and scales with
 * alpha[b * scale_batch_stride], beta[b * scale_batch_stride]; everything else is ti_bmm_i8_config.
 * With sAb = 0 (one shared activation matrix), B = the projections' [N,K] weights stacked along N
 * (sBb = N * sBn) and sCb = N (batch b writes columns b*N .. of a [M, batch*N] row-major output)
 * this is the q/k/v projection of an attention block as one launch: each projection alone is
 * too small to fill the chip (W8A8B8O8Linear x3, nn/linear.py:18-67; the reference launches them
 * one by one).  No counterpart in the reference's kernels.
 */
int ti_bmm_i8_grouped(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk,
                      const int8_t* B, int64_t sBb, int64_t sBn, int64_t sBk,
                      void* C, int64_t sCb, int64_t sCm, int64_t sCn,
                      int batch, int M, int N, int K,
                      const void* bias, int bias_kind, int64_t bias_batch_stride,
                      const float* alpha, const float* beta, int64_t scale_batch_stride,
                      int epilogue, int out_dtype, int round_mode,
                      int config, void* stream);
/*
 * ti_bmm_i8_config for callers that cannot allocate device memory (a stream under HIP graph capture
 * before any workspace exists, a serving loop or harness that forbids hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, same arithmetic, same kernels and the same choice
 * of configuration and K split as ti_bmm_i8_config; the difference is where a split-K launch keeps
 * its ticket counters and int32 partial sums: in a fixed array in the library's device image
 * (16384 counters + 32 MiB of partial sums, held by every GPU the library runs on until the process
 * ends) instead of the per-stream workspace ti_bmm_i8 allocates.  The call allocates and frees
 * nothing, on the host side of the device or through any library.  A K split the caller forces
 * (bits 8..15 of config) whose partial sums would not fit (tiles x splits x tile bytes > 32 MiB, or
 * tiles x 4 > 16384) returns TI_E_SHAPE and launches nothing; a split the library would choose itself
 * gives way to the unsplit launch in that case (same result; it uses no scratch and always fits).  All calls on one
 * GPU share that GPU's array: two calls that may run at the same time on one GPU (different
 * streams, different host threads) race on it and must be serialised by the caller.  Kernels leave
 * the counters at zero; the partial sums are overwritten before they are read.
 */
int ti_bmm_i8_static_scratch(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk,
                             const int8_t* B, int64_t sBb, int64_t sBn, int64_t sBk,
                             void* C, int64_t sCb, int64_t sCm, int64_t sCn,
                             int batch, int M, int N, int K,
                             const void* bias, int bias_kind,
                             const float* alpha, const float* beta,
                             int epilogue, int out_dtype, int round_mode,
                             int config, void* stream);
/*
 * Frees the split-K workspaces (ticket counters + partial sums, including blocks a workspace has outgrown)
 * that ti_bmm_i8* allocated on the current device for `stream`, or for every stream when all_streams != 0,
 * after waiting for the work queued on those streams.  *freed_bytes (host, may be NULL) receives the bytes
 * of the current blocks released.  A caller that creates streams per request calls this before destroying
 * a stream; otherwise each stream that ever ran a split-K launch keeps up to 96 MiB until the process ends.
 * A graph that captured a split-K launch on such a stream must not be replayed afterwards.  The next
 * split-K launch allocates a new workspace.  No counterpart in the reference (Triton's autotuner
 * allocates and frees through torch).
 */
int ti_release_workspaces(void* stream, int all_streams, int64_t* freed_bytes);
int ti_gemm_num_configs(void);
const char* ti_gemm_config_name(int config);
/* Index of the configuration the calling thread's most recent ti_bmm_i8* launch used (-1 if
 * none); lets a benchmark attribute time to the kernel that actually ran. */
int ti_gemm_last_config(void);
/* Number of K splits that launch used (1 = K not split). */
int ti_gemm_last_splits(void);
/*
 * Dry run of ti_bmm_i8_config (static_scratch != 0: of ti_bmm_i8_static_scratch): takes every decision
 * the launch would take, through the same host code (validation, choice of configuration, K split, tile
 * order, grid), touches no device, allocates and launches nothing, dereferences no pointer (pointer
 * values matter only for their alignment), and writes what would be launched to plan[0..TI_PLAN_INTS):
 *   [0] configuration index  [1] K splits  [2] k-tiles per split  [3] row tiles  [4] column tiles
 *   [5] row tiles per group of the tile order  [6] grid x  [7] grid y  [8] threads per workgroup
 *   [9] waves that split K inside a workgroup (skinny / rows4 kernels)  [10] streaming waves (rows4)
 *   [11] bytes of split-K partial sums the launch needs
 * Runs without a GPU.  The autotuner of the reference (kernels/utils.py:6-558) answers the same
 * question -- which tile for which (M, N, K) -- by timing; this reports the static choice.  Used by the
 * host-side bounds tests, which replay the kernels' address arithmetic for the planned launch.
 */
#define TI_PLAN_INTS 12
int ti_gemm_plan(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk,
                 const int8_t* B, int64_t sBb, int64_t sBn, int64_t sBk,
                 void* C, int64_t sCb, int64_t sCm, int64_t sCn,
                 int batch, int M, int N, int K,
                 const void* bias, int bias_kind,
                 const float* alpha, const float* beta,
                 int epilogue, int out_dtype, int round_mode,
                 int config, int static_scratch, int64_t* plan);

/* ---- row kernels ------------------------------------------------------------------- */

/*
 * y_i8[r,:] = q8( ((x[r,:] - mean_r) * rstd_r) * gamma + beta ),  rstd = 1/sqrt(var + eps),
 * biased variance; rms != 0 selects the RMSNorm branch (mean = 0, var = mean(x^2)).
 * Replaces layer_norm_fwd_fused_single_pass_q, kernels/fused.py:235-382 (module LayerNormQ,
 * nn/fused.py:34-57).  x is fp32 with unit column stride and row stride `x_row_stride`
 * elements; y has row stride `y_row_stride`.  beta may be NULL (HAS_BIAS = False,
 * kernels/fused.py:324-326).  mean_out / rstd_out (fp32[rows], may be NULL) receive the row
 * statistics for tests.
 */
int ti_layernorm_q(const float* x, int64_t x_row_stride,
                   const float* gamma, const float* beta, float eps,
                   int8_t* y, int64_t y_row_stride,
                   int rows, int cols, int rms, int round_mode,
                   float* mean_out, float* rstd_out, void* stream);

/*
 * resid_out = resid_in + in_scale * f(acc_i32);  y_i8 = q8(LayerNorm(resid_out; gamma, beta, eps)).
 * The native op the reference intends at functional/fused.py:27-32 (module
 * DQ_Add_LayerNorm_Q, nn/fused.py:59-78) and defines only as the PyTorch emulation
 * functional/fused.py:6-15.  in_scale is a host float (nn/fused.py:62,73); when in_scale_dev is not
 * NULL the scale is read from that DEVICE fp32 instead and in_scale is ignored (a caller that holds
 * the scale as a device tensor need not synchronise to fetch it).  All row-major
 * with unit column stride; row strides in elements.  resid_out may alias resid_in.
 * ln_out_f32 (may be NULL) additionally receives the fp32 LayerNorm output, which is what
 * the un-quantised variant returns (functional/fused.py:18-24, dq_add_layernorm); y may be
 * NULL when only that variant is wanted.  At least one of y / ln_out_f32 must be given.
 */
int ti_dq_add_layernorm_q(const int32_t* acc, int64_t acc_row_stride, float in_scale, const float* in_scale_dev,
                          const float* resid_in, int64_t resid_in_row_stride,
                          const float* gamma, const float* beta, float eps,
                          float* resid_out, int64_t resid_out_row_stride,
                          int8_t* y, int64_t y_row_stride,
                          float* ln_out_f32, int64_t ln_out_row_stride,
                          int rows, int cols, int round_mode,
                          float* mean_out, float* rstd_out, void* stream);

/*
 * y_i8[i] = q8( 0.5*x*(1+tanh(sqrt(2/pi)*(x+0.044715*x^3))) * scale ),  i < n, contiguous.
 * Stand-alone form of fast_geluQ, kernels/fused.py:76-79 (module GeLu_Q, nn/fused.py:81-87).
 * scale: DEVICE pointer to one fp32.
 */
int ti_gelu_q(const float* x, const float* scale, int8_t* y, int64_t n,
              int round_mode, void* stream);

/*
 * y_i8[r,j] = round_half_even( softmax_j(x_i8[r,:] * scale)[j] * 127 ), values in [0,127].
 * The link between the two attention BMMs of a W8A8 decoder layer: int8 scores from
 * bmm_s8t_s8n_s8t (kernels/bmm.py:576-612) in, int8 probabilities for the P.V BMM out.  The
 * reference tree has no kernel for it (its modules stop at the BMMs); the arithmetic is the
 * fp32 softmax followed by `mul(127).round()` that SmoothQuant-style callers of these modules do,
 * fixed as follows so that every kernel that forms these probabilities (this one and
 * ti_attention_i8) gives the same bits whatever order it visits a row in:
 *     mx = largest visible score of the row;  s2 = scale * log2(e)  (fp32)
 *     e_j = exp2(fma(float(x_j), s2, -(float(mx) * s2)))
 *     S   = sum_j round_half_even(e_j * 2^23)              an integer: exact in any order
 *     y_j = round_half_even(e_j * (127 * 2^23 / float(S)))     float(S) correctly rounded, IEEE division
 * scale is a host float (score scale), 0 <= scale <= 64 (TI_E_COMBO otherwise).  causal_q_len > 0: rows come in groups of that many query
 * positions, position i attends to columns 0 .. i + (cols - causal_q_len); 0 = no mask.
 * cols <= 8192.  Row strides in elements, unit column stride.
 */
int ti_softmax_q(const int8_t* x, int64_t x_row_stride, float scale,
                 int8_t* y, int64_t y_row_stride, int rows, int cols, int causal_q_len, void* stream);

/*
 * dst[c, r] = src[r, c] for an int8 matrix of `rows` x `cols` (row strides in elements, unit column
 * stride on both sides).  The P.V BMM wants V^T with the sequence as its contiguous dimension
 * (bmm_s8t_s8n_*, kernels/bmm.py:428-464 takes b as [B, N, K]); callers of the reference's modules
 * build it with `v.transpose(1, 2).contiguous()` in torch.  With src = V [S, heads*D] and
 * dst = V^T viewed as [heads*D, T] (dst pointing at column T - S) this writes every head's V^T, or
 * appends S positions to a KV cache, in one launch.
 */
int ti_transpose_i8(const int8_t* src, int64_t src_row_stride, int8_t* dst, int64_t dst_row_stride,
                    int rows, int cols, void* stream);

/*
 * W8A8BFP32OFP32Linear (nn/linear.py:222-278) followed by the residual add its caller performs
 * (`fc2(x) + residual` in a decoder layer):
 *     C[m][n] = (alpha * f(acc[m][n]) + beta * bias[n]) + residual[m][n]        fp32, rounded per step
 * A [M,K], W [N,K] int8 with unit column stride, bias fp32 [N] or NULL, residual and C fp32 with unit
 * column stride (row strides in elements).  With M <= 16 the weight-streaming decode kernel adds the
 * residual as it stores, and the persistent kernels that serve large outputs add it in their epilogue (one
 * launch instead of two); otherwise the GEMM is followed by an add kernel.
 * Same bits as the linear followed by an fp32 add.  C must not overlap the residual.
 */
int ti_linear_i8_residual_f32(const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw, const float* bias,
                              const float* alpha, const float* beta, const float* residual, int64_t ldr,
                              float* C, int64_t ldc, int M, int N, int K, void* stream);

/*
 * A decode step's q / k / v projections (three W8A8B8O8Linear of one input, nn/linear.py:18-67) with the
 * KV-cache append folded in: one launch of the weight-streaming kernel instead of ti_bmm_i8_grouped
 * followed by ti_kv_append_i8.  A [M,K] (M <= 16, K >= 1024), W [3N,K] the stacked weights, bias int8
 * [3N] or NULL, alpha3 / beta3 fp32 [3], C [M,3N] int8 (row stride ldc) receives q | k | v as
 * ti_bmm_i8_grouped writes them; in addition k goes to k_dst[h * k_head_stride + m * D + d] and v to
 * vt_dst[(h * D + d) * vt_row_stride + m] (k_dst / vt_dst point at the first new slot / column, as for
 * ti_kv_append_i8; N = heads * D, D % 16 == 0).  TI_E_COMBO when the operands do not fit the kernel
 * (the caller then makes the two calls).
 */
int ti_qkv_decode_i8(const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw, const int8_t* bias,
                     const float* alpha3, const float* beta3, int8_t* C, int64_t ldc, int M, int N, int K,
                     int8_t* k_dst, int64_t k_head_stride, int8_t* vt_dst, int64_t vt_row_stride, int D,
                     void* stream);

/*
 * Appends S new positions to an int8 KV cache in one launch: K [S, heads*D] (row stride
 * k_src_row_stride) is copied to k_dst[h][s][d] = k_dst + h * k_head_stride + s * D + d (k_dst points at
 * the first new slot of head 0 in a [heads, T, D] cache, k_head_stride = T * D), and V [S, heads*D]
 * is transposed into vt_dst[(h*D + d) * vt_row_stride + s] (vt_dst points at the first new column
 * of a [heads*D, T] cache, vt_row_stride = T).  D % 16 == 0.  The reference's callers do both
 * steps with torch indexing; ti_transpose_i8 alone covers the prefill case without a cache.
 */
int ti_kv_append_i8(const int8_t* k_src, int64_t k_src_row_stride, const int8_t* v_src, int64_t v_src_row_stride,
                    int8_t* k_dst, int64_t k_head_stride, int8_t* vt_dst, int64_t vt_row_stride,
                    int S, int heads, int D, void* stream);

/*
 * One attention block without the score round trip through memory:
 *     scores = q8(qk_alpha * (q . k^T))                    (bmm_s8t_s8n_s8t, kernels/bmm.py:576-612)
 *     probs  = round_half_even(127 * softmax(scores * score_scale)), causal mask as ti_softmax_q
 *     out    = q8(pv_alpha * (probs . v))                  (bmm_s8t_s8n_s8t again, b = V^T)
 * q [batch, S, D], k [batch, T, D], vt [batch, D, T] (V^T, as the P.V BMM takes it), out
 * [batch, S, D]; int8, unit stride along the last dimension, batch and row strides in elements
 * (all multiples of 16, like the pointers); D = 128; T a multiple of 16; 0 < score_scale <= 64.
 * The scalars are host floats.  The int8 scores are the BMM's and the probabilities ti_softmax_q's
 * bit for bit (a row's exponentials are summed as integers, so the order in which the keys are
 * visited does not matter): the output equals the three-launch chain's exactly.
 * With S <= 16 and T <= 4096 (decode) a one-pass kernel runs instead, one to four workgroups per
 * batch entry.
 * The reference has no fused form (its modules stop at the BMMs, nn/bmm.py:10-74); the
 * three-launch chain remains available and is what this is tested against.
 */
int ti_attention_i8(const int8_t* q, int64_t q_batch_stride, int64_t q_row_stride,
                    const int8_t* k, int64_t k_batch_stride, int64_t k_row_stride,
                    const int8_t* vt, int64_t vt_batch_stride, int64_t vt_row_stride,
                    int8_t* out, int64_t out_batch_stride, int64_t out_row_stride,
                    int batch, int S, int T, int D,
                    float qk_alpha, float score_scale, float pv_alpha, int causal_q_len, void* stream);

/*
 * Dynamic per-token activation quantisation, dynamic_quantize_activation_per_token_absmax
 * (functional/quantization.py:61-67): per row r of x [rows, cols] (fp32 or fp16: x_dtype TI_F32 /
 * TI_F16, unit column stride, row strides in elements)
 *     scale[r] = clamp(max_j |x[r,j]|, min = 1e-8) / 127           (rounded to x's dtype per step)
 *     q[r,j]   = clamp(round_half_even(x[r,j] / scale[r]), -128, 127)
 * scale_out (rows elements of x's dtype, may be NULL) receives the scales.  x is not modified
 * (the reference helper overwrites it with the rounded quotients as a side effect).
 */
int ti_quantize_per_token_absmax(const void* x, int x_dtype, int64_t x_row_stride,
                                 int8_t* q, int64_t q_row_stride, void* scale_out,
                                 int rows, int cols, void* stream);

/*
 * Floating-point LayerNorm / RMSNorm over the rows of x [rows, cols], with the optional skip
 * (residual) add: layer_norm_fwd_fused_single_pass (kernels/fused.py:385-532),
 * skip_layer_norm_fwd_fused_single_pass (kernels/fused.py:535-693) and
 * skip_layer_norm_fwd_fused_single_pass2 (kernels/fused.py:696-862).  All tensors share one dtype
 * (TI_F32 / TI_F16 / TI_BF16), unit column stride, row strides in elements.
 *     a = f32(x); mean = sum(a)/cols (0 when rms != 0); var = sum((a-mean)^2)/cols
 *     out      = T( ((a - mean) / sqrt(var + eps)) * f32(gamma) [+ f32(beta)] )      (beta may be NULL)
 *     skip_out = T( f32(out) + f32(skip) )
 * out alone: the plain LayerNorm; skip + skip_out alone: the first skip variant; all three: the
 * second.  skip and skip_out are both NULL or both given.
 */
int ti_layernorm_fp(const void* x, int64_t x_row_stride, const void* skip, int64_t skip_row_stride, int dtype,
                    const void* gamma, const void* beta, float eps, int rms,
                    void* out, int64_t out_row_stride, void* skip_out, int64_t skip_out_row_stride,
                    int rows, int cols, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRITON_INT_HIP_H */
