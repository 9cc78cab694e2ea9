// gemm_i8.hip — int8 x int8 -> int32 GEMM / batched GEMM for gfx950 (MI355X) with fused epilogues.
//
// Replaces the Triton kernels of zhanglei1172/triton_int kernels/linear.py:24-853,
// kernels/bmm.py:12-760 and kernels/fused.py:88-231 (one tl.dot K loop + per-kernel epilogue).
//
// Kernels (all v_mfma_i32_*_i8, int32 accumulators in registers):
//   gemm_mfma_ws_kernel      persistent, wave-specialised: producer waves issue the global -> LDS
//                            loads, consumer waves read fragments and issue MFMAs.  The large GEMMs.
//   gemm_mfma_stream_kernel  persistent, loads issued by the MFMA waves (256x256 tiles, short K).
//   gemm_mfma_kernel         one tile per workgroup; any output layout the fast loads allow.
//   gemm_rows4_kernel        M <= 16: weights streamed as whole 1 KB row pieces (decode linears).
//   gemm_skinny_kernel       M <= 64: 16-row weight slabs in MFMA layout, K split over waves.
//   gemm_gather_kernel       any strides / alignment / K (byte gathers).
// The first five need both operands K-contiguous and 16-byte aligned: 128-bit buffer loads
// straight into XOR-swizzled LDS tiles, several stages deep.
//
// C = epilogue(sum_k A[m,k] * B[n,k]); A is [M,K], B is [N,K] (the reference's "N" operand,
// kernels/linear.py:217), the "T" operand [K,N] arrives as strides (sBn = 1, sBk = N).
#include <mutex>
#include <type_traits>
#include <vector>

#include "ti_common.h"

namespace ti {

#ifdef TI_GEMM_TIMELINE
// experiment builds only: per workgroup, the constant-rate clock (100 MHz) at a few points of the
// wave-specialised kernel, read back by ti_debug_timeline
__device__ unsigned long long g_timeline[1024 * 8];
#define TI_TL(slot) do { if ((threadIdx.x & 63) == 0) g_timeline[blockIdx.x * 8 + (slot)] = wall_clock64(); } while (0)
#else
#define TI_TL(slot) do { } while (0)
#endif

struct GemmParams {
  const int8_t* A;
  const int8_t* B;
  void* C;
  int64_t sAb, sAm, sAk, sBb, sBn, sBk, sCb, sCm, sCn;
  int batch, M, N, K;
  const void* bias;
  int bias_kind;
  const float* alpha;
  const float* beta;
  int epilogue, out_dtype, round_mode;
  int tiles_m, tiles_n, group_m;
  int ksplit;  // skinny kernel: waves of a workgroup that share one 16-row slab and split K
  // grouped launches (several projections of one input as the batches of one launch): batch b uses
  // bias elements [b * bias_bs, b * bias_bs + N) and the scalars alpha[b * scale_bs], beta[b * scale_bs]
  int64_t bias_bs;
  int64_t scale_bs;
  // fp32 outputs of gemm_rows4_kernel and of the persistent kernels' fp32 epilogue: C = epilogue value + resid[m * resid_rs + n]
  const float* resid;
  int64_t resid_rs;
  // int8 outputs of a grouped q/k/v launch of gemm_rows4_kernel only: batch 1 (k) also goes to
  // kv_k[head * kv_k_hs + m * kv_D + d], batch 2 (v) to kv_vt[(head * kv_D + d) * kv_vt_rs + m]
  int8_t* kv_k;
  int8_t* kv_vt;
  int64_t kv_k_hs, kv_vt_rs;
  int kv_D;
  // split K (gemm_mfma_ws_kernel, batch == 1): a tile's k-tiles are dealt to `splits` work items of
  // kt_split k-tiles each (the last takes what is left); the items leave their int32 sums in
  // sk_partial, and the item of a tile that finishes last adds them up and stores the tile.
  int splits, kt_split;
  int* sk_partial;   // [tile][split][consumer wave][accumulator dword][lane]
  int* sk_counter;   // [tile][consumer wave], zero between launches
};

enum OutClass { OUT8 = 0, OUT32 = 1, OUT16 = 2 };


// ---- tile -> (m, n) mapping ----------------------------------------------------------------
// Workgroups are dealt round-robin to the 8 XCDs (each with a private L2), so consecutive
// block ids are first folded into 8 contiguous ranges (one per XCD) and each range then walks
// the tile grid in column-major groups of `group_m` row-tiles so that a range re-uses few
// distinct A and B panels.
__device__ __forceinline__ void tile_from_rank(const GemmParams& p, int lid, int& tm, int& tn) {
  const int gsz = p.group_m * p.tiles_n;
  const int gid = lid / gsz;
  const int first_m = gid * p.group_m;
  const int gm = min(p.tiles_m - first_m, p.group_m);
  const int r = lid - gid * gsz;
  tm = first_m + r % gm;
  tn = r / gm;
}

__device__ __forceinline__ void tile_coords(const GemmParams& p, int pid, int& tm, int& tn) {
  const int T = p.tiles_m * p.tiles_n;
  const int xcd = pid & 7, local = pid >> 3;
  const int per = T >> 3, rem = T & 7;
  tile_from_rank(p, xcd * per + min(xcd, rem) + local, tm, tn);
}

// Batched launches (grid = tiles x batch): the same folding applied to the whole tiles*batch
// sequence, so that one XCD works through whole batches and its L2 fetches every operand panel of
// a batch once instead of all 8 L2s fetching most of every batch.
__device__ __forceinline__ void batch_tile_coords(const GemmParams& p, int pid, int by, int nbatch, int& bz, int& tm,
                                                  int& tn) {
  const int T = p.tiles_m * p.tiles_n;
  const int W = T * nbatch;
  const int lin = by * T + pid;
  const int xcd = lin & 7, local = lin >> 3;
  const int per = W >> 3, rem = W & 7;
  const int g = xcd * per + min(xcd, rem) + local;
  bz = g / T;
  tile_from_rank(p, g - bz * T, tm, tn);
}

// ---- epilogue (shared by both kernel families) ------------------------------------------------
// One fp32 value per accumulator, in the operation order the contract fixes:
//   v = f(acc) * alpha;  c0 = f(bias) * beta;  v = c0 + v        (no FMA contraction)
struct EpiCtx {
  float alpha, beta;
  int epilogue, round_mode, bias_kind;
  const void* bias;
  const float* safe;  // always-readable 4 bytes (the A operand), target of the no-bias dummy loads
};

// Per-column term that is added to alpha*f(acc): beta*f(bias) for the scale epilogues, the raw
// fp32 bias for GELU-Q (kernels/fused.py:184-186 adds the bias un-scaled), 0 without a bias.
// KIND is the bias element type the caller has already branched on; without a bias the load is
// redirected to element 0 of a valid buffer and the result replaced by 0, so there is no branch.
template <int KIND>
__device__ __forceinline__ float column_term_t(const EpiCtx& e, int n, bool gelu) {
  const bool has = e.bias_kind != TI_BIAS_NONE;
  const void* base = has ? e.bias : (const void*)e.safe;
  const int idx = has ? n : 0;
  float b;
  if constexpr (KIND == TI_BIAS_I8) b = (float)((const int8_t*)base)[idx];
  else if constexpr (KIND == TI_BIAS_I32) b = (float)((const int32_t*)base)[idx];
  else {
    // the floating-point family: fp32, or fp16 / bf16 widened exactly (what bias.float() gives)
    if (e.bias_kind == TI_BIAS_F16) b = has ? (float)((const _Float16*)base)[idx] : 0.0f;
    else if (e.bias_kind == TI_BIAS_BF16) b = has ? __uint_as_float((unsigned)((const uint16_t*)base)[idx] << 16) : 0.0f;
    else b = ((const float*)base)[idx];
  }
  const float scaled = gelu ? b : b * e.beta;
  return has ? scaled : 0.0f;
}

__device__ __forceinline__ float column_term(const EpiCtx& e, int n) {
  const bool gelu = e.epilogue == TI_EPI_GELU_I8;
  switch (e.bias_kind) {
    case TI_BIAS_I8: return column_term_t<TI_BIAS_I8>(e, n, gelu);
    case TI_BIAS_I32: return column_term_t<TI_BIAS_I32>(e, n, gelu);
    case TI_BIAS_F32:
    case TI_BIAS_F16:
    case TI_BIAS_BF16: return column_term_t<TI_BIAS_F32>(e, n, gelu);
    default: return 0.0f;
  }
}

__device__ __forceinline__ float epi_value(const EpiCtx& e, int acc, float col) {
  float v = (float)acc * e.alpha;
  if (e.bias_kind != TI_BIAS_NONE) v = col + v;
  if (e.epilogue == TI_EPI_GELU_I8) v = gelu_tanh_scaled(v, e.beta);
  return v;
}

__device__ __forceinline__ int epi_q8(const EpiCtx& e, int acc, float col) {
  int q = q8(epi_value(e, acc, col), e.round_mode);
  if (e.epilogue == TI_EPI_SCALE_RELU_I8) q = max(q, 0);
  return q;
}

template <int OUTCLS>
__device__ __forceinline__ void store_one(const EpiCtx& e, void* C, int64_t off, int acc, float col,
                                          int bias_i32, int out_dtype) {
  if constexpr (OUTCLS == OUT8) {
    ((int8_t*)C)[off] = (int8_t)epi_q8(e, acc, col);
  } else if constexpr (OUTCLS == OUT32) {
    if (e.epilogue == TI_EPI_I32) {
      ((int*)C)[off] = (int)((unsigned)acc + (unsigned)bias_i32);
    } else if (e.epilogue == TI_EPI_SCALE_I32) {
      ((int*)C)[off] = q32(epi_value(e, acc, col), e.round_mode);
    } else {
      ((float*)C)[off] = epi_value(e, acc, col);
    }
  } else {
    float v = epi_value(e, acc, col);
    ((uint16_t*)C)[off] = out_dtype == TI_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
  }
}

// the same conversions, returned as the output element's bits (for callers that pack several
// elements into one store)
template <int OUTCLS>
__device__ __forceinline__ unsigned convert_one(const EpiCtx& e, int acc, float col, int bias_i32, int out_dtype) {
  if constexpr (OUTCLS == OUT8) {
    return (unsigned)epi_q8(e, acc, col) & 0xffu;
  } else if constexpr (OUTCLS == OUT32) {
    if (e.epilogue == TI_EPI_I32) return (unsigned)acc + (unsigned)bias_i32;
    if (e.epilogue == TI_EPI_SCALE_I32) return (unsigned)q32(epi_value(e, acc, col), e.round_mode);
    return __float_as_uint(epi_value(e, acc, col));
  } else {
    const float v = epi_value(e, acc, col);
    return out_dtype == TI_F16 ? f32_to_f16_bits(v) : f32_to_bf16_bits(v);
  }
}

__device__ __forceinline__ EpiCtx make_epi(const GemmParams& p, int bz) {
  EpiCtx e;
  const int64_t si = (int64_t)bz * p.scale_bs;
  e.alpha = p.alpha ? p.alpha[si] : 1.0f;
  e.beta = p.beta ? p.beta[si] : 1.0f;
  e.epilogue = p.epilogue;
  e.round_mode = p.round_mode;
  e.bias_kind = p.bias ? p.bias_kind : TI_BIAS_NONE;
  const int bias_esz = p.bias_kind == TI_BIAS_I8 ? 1 : ((p.bias_kind == TI_BIAS_F16 || p.bias_kind == TI_BIAS_BF16) ? 2 : 4);
  e.bias = p.bias ? (const void*)((const char*)p.bias + (int64_t)bz * p.bias_bs * bias_esz) : nullptr;
  e.safe = (const float*)p.A;
  return e;
}

// ---- int8 quantisation of 16 clamped fp32 values into 4 dwords --------------------------------
// v + 1.5 * 2^23 rounds v to the nearest integer (ties to even) and leaves the two's-complement
// int8 in the low byte of the sum's bit pattern (|v| <= 128 after the clamp).  The adds write that
// byte straight into byte t of dword g (sub-dword destination select, the other bytes preserved),
// so there is no separate packing step: 4 instead of 4.75 vector instructions per output.  The
// four dwords are interleaved because a partial write must not be read by the very next
// instruction; the trailing s_nop covers whatever instruction follows the block.
__device__ __forceinline__ void pack16_q8(const float (&f)[4][4], unsigned (&X)[4]) {
  const float magic = 12582912.0f;
#define TI_SDWA_ADD(G, T, B) "v_add_f32_sdwa %" #G ", %4, %" #T " dst_sel:" B " dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
  asm("v_add_f32_e32 %0, %4, %5\n\t"
      "v_add_f32_e32 %1, %4, %9\n\t"
      "v_add_f32_e32 %2, %4, %13\n\t"
      "v_add_f32_e32 %3, %4, %17\n\t"
      TI_SDWA_ADD(0, 6, "BYTE_1") TI_SDWA_ADD(1, 10, "BYTE_1") TI_SDWA_ADD(2, 14, "BYTE_1") TI_SDWA_ADD(3, 18, "BYTE_1")
      TI_SDWA_ADD(0, 7, "BYTE_2") TI_SDWA_ADD(1, 11, "BYTE_2") TI_SDWA_ADD(2, 15, "BYTE_2") TI_SDWA_ADD(3, 19, "BYTE_2")
      TI_SDWA_ADD(0, 8, "BYTE_3") TI_SDWA_ADD(1, 12, "BYTE_3") TI_SDWA_ADD(2, 16, "BYTE_3") TI_SDWA_ADD(3, 20, "BYTE_3")
      "s_nop 0"
      : "=&v"(X[0]), "=&v"(X[1]), "=&v"(X[2]), "=&v"(X[3])
      : "v"(magic), "v"(f[0][0]), "v"(f[0][1]), "v"(f[0][2]), "v"(f[0][3]), "v"(f[1][0]), "v"(f[1][1]), "v"(f[1][2]),
        "v"(f[1][3]), "v"(f[2][0]), "v"(f[2][1]), "v"(f[2][2]), "v"(f[2][3]), "v"(f[3][0]), "v"(f[3][1]), "v"(f[3][2]),
        "v"(f[3][3]));
#undef TI_SDWA_ADD
}

// ---- fast family -----------------------------------------------------------------------------
//
// LDS stage = A tile (BM x BK bytes) + B tile (BN x BK bytes), each viewed as 16-byte chunks;
// chunk c of row r lives at chunk slot c ^ ((r >> SWZ) & (CH-1)) of that row, which spreads the
// 16-byte reads of the 32 lanes that share a chunk index (one MFMA operand column) over the banks.
//
// Global -> LDS: chunk slot q = it*NT + tid of a tile is filled by thread tid with
// buffer_load_dwordx4 ... lds (lane i of a wave lands at M0-base + 16*i, no VGPR round trip).
// The buffer descriptors bound the loads: rows past M/N and the K tail read as zero.
//
// Pipeline: NSTAGE LDS stages, NSTAGE-1 k-tiles of loads in flight.  Per k-tile one barrier,
// placed before the last MFMA k-step so that the first operand fragments of the next k-tile are
// fetched from LDS while the matrix pipe is still busy; inside a k-tile the fragments of k-step
// s+1 are read while the MFMAs of k-step s issue (two register sets).

template <int ROWS, int BK, int NT, int SWZ>
struct TileLoader {
  static constexpr int CH = BK / 16;
  static constexpr int IT = ROWS * CH / NT;
  static_assert(ROWS * CH % NT == 0, "tile must split evenly over the threads");
  int voff[IT];  // byte offset of this thread's chunk in k-tile 0 (the k offset is added as a scalar)
  int klim[IT];  // the chunk is inside K while k0 < klim

  __device__ __forceinline__ void init(int tid, int row0, int ld, int K) {
#pragma unroll
    for (int it = 0; it < IT; ++it) {
      const int q = it * NT + tid;
      const int row = q / CH;
      const int cphys = q % CH;
      const int clog = cphys ^ ((row >> SWZ) & (CH - 1));
      voff[it] = (row0 + row) * ld + clog * 16;
      klim[it] = K - clog * 16;
    }
  }
};

// The global -> LDS loads and the waits on them are written as inline assembly on purpose.  For
// the builtin form the compiler tracks "LDS written by a buffer load" conservatively: every
// workgroup barrier, and every LDS read that might alias, gets an s_waitcnt vmcnt(0) in front of
// it, which drains the load pipeline once per k-tile and defeats multi-stage prefetching.  With
// the loads invisible to that tracking, the kernel counts them itself (vmcnt retires in order).
// M0 carries the LDS destination of a wave's 64 x 16 bytes; nothing else in these kernels uses M0.
// Hazard the compiler cannot see: a VMEM instruction must not read an SGPR (descriptor, scalar
// offset) within 5 wait states of a VALU instruction writing it (v_readfirstlane, the tail of a
// uniform division), or it reads the register's previous contents -- and the scalar offset is added
// AFTER the descriptor's range check, so a stale one addresses base + garbage.  The compiler inserts
// those wait states for instructions it emits itself, not for the text of an asm block, so the
// helpers carry them: s_mov m0 (1) + s_nop 3 (4) = 5 wait states between whatever precedes the block
// and the load, wherever the operands come from.  (The s_nop also covers the one wait state a
// buffer load to LDS needs after a write of M0.)
__device__ __forceinline__ v4i make_rsrc(const void* base, int bytes) {
  const uint64_t a = (uint64_t)base;
  v4i r;
  r[0] = (int)(uint32_t)a;
  r[1] = (int)((uint32_t)(a >> 32) & 0xffffu);  // stride 0: raw buffer
  r[2] = bytes;                                 // num_records: loads at or past it return 0
  r[3] = 0x00020000;                            // 32-bit data format word of gfx9-family raw buffers
  return r;
}

__device__ __forceinline__ void dma16_to_lds(v4i rsrc, int voff, int soff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}

// the same, non-temporal, for data that is read exactly once (the decode kernel's weight stream:
// 7 % shorter launches than with the default cache policy)
__device__ __forceinline__ void dma16_to_lds_stream(v4i rsrc, int voff, int soff, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}

// wait until at most N of this wave's buffer loads are outstanding and its LDS reads are done,
// then meet the other waves of the workgroup
template <int N>
__device__ __forceinline__ void wait_loads_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// OCC = workgroups the register allocation must allow per CU (short-K batched shapes want two or
// three co-resident workgroups so that one's epilogue overlaps another's loads).
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int SWZ, int NSTAGE, int OUTCLS, int OCC = 1>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, (WAVES_M * WAVES_N * OCC + 3) / 4) void gemm_mfma_kernel(GemmParams p) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int CH = BK / 16;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int KS = BK / 32;  // MFMA k-steps per k-tile
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  constexpr int STAGE = A_BYTES + B_BYTES;
  constexpr int LDS_BYTES = NSTAGE * STAGE;
  constexpr int DEPTH = NSTAGE - 1;  // k-tiles of loads in flight
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 64 == 0, "tile shape");
  static_assert(NSTAGE >= 3 && LDS_BYTES <= 160 * 1024, "LDS budget");

  __shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  int tile_m, tile_n, bz = 0;
  if (gridDim.y == 1) tile_coords(p, blockIdx.x, tile_m, tile_n);
  else batch_tile_coords(p, blockIdx.x, blockIdx.y, gridDim.y, bz, tile_m, tile_n);
  // the divisions above run on the vector unit; the results are uniform and feed scalar operands
  bz = __builtin_amdgcn_readfirstlane(bz);
  tile_m = __builtin_amdgcn_readfirstlane(tile_m);
  tile_n = __builtin_amdgcn_readfirstlane(tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int8_t* Ab = p.A + (int64_t)bz * p.sAb;
  const int8_t* Bb = p.B + (int64_t)bz * p.sBb;
  const int lda = (int)p.sAm, ldb = (int)p.sBn;
  // bytes addressable from the batch base: rows past the end and the K tail read as zero
  const int a_extent = (p.M - 1) * lda + p.K;
  const int b_extent = (p.N - 1) * ldb + p.K;
  const v4i rA = make_rsrc(Ab, a_extent);
  const v4i rB = make_rsrc(Bb, b_extent);
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  // LDS byte address of this wave's 1 KB slot in chunk-slot group 0 of stage 0
  const unsigned wave_slot = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);

  TileLoader<BM, BK, NT, SWZ> la;
  TileLoader<BN, BK, NT, SWZ> lb;
  la.init(tid, m0, lda, p.K);
  lb.init(tid, n0, ldb, p.K);
  constexpr int A_IT = decltype(la)::IT, B_IT = decltype(lb)::IT;
  constexpr int LOADS = A_IT + B_IT;  // buffer loads per thread per k-tile
  const int KT = (p.K + BK - 1) / BK;
  const int OOB = (int)0x80000000;

  // One global -> LDS load of the k-tile being fetched (k offset k_issue, LDS stage st_issue):
  // load number d of the LOADS this thread owns per k-tile.  The address is the thread's constant
  // byte offset plus the scalar k offset; a chunk at or past K is redirected out of bounds so it
  // reads as zero instead of running into the next row.  Past the end of K every chunk is out of bounds:
  // the loads write zeros into a stage nobody reads again, which keeps the number of loads in
  // flight, and so the vmcnt to wait for, constant.
  int k_issue = 0, st_issue = 0;
  auto dma = [&](int d) {
    if (d < A_IT) {
      const unsigned dst = wave_slot + st_issue * STAGE + d * NT * 16;
      dma16_to_lds(rA, (k_issue < la.klim[d]) ? la.voff[d] : OOB, k_issue, dst);
    } else {
      const int e = d - A_IT;
      const unsigned dst = wave_slot + st_issue * STAGE + A_BYTES + e * NT * 16;
      dma16_to_lds(rB, (k_issue < lb.klim[e]) ? lb.voff[e] : OOB, k_issue, dst);
    }
  };
  auto dma_advance = [&]() {
    k_issue += BK;
    st_issue = (st_issue + 1 == NSTAGE) ? 0 : st_issue + 1;
  };

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  // per-lane fragment addressing: row = (lane & 31) within a 32-row MFMA operand block,
  // logical chunk = 2*ks + (lane >> 5)
  const int frow = lane & 31;
  const int fsw = (frow >> SWZ) & (CH - 1);
  const int fhalf = lane >> 5;
  const int a_lane = (wm * WTM + frow) * BK;
  const int b_lane = A_BYTES + (wn * WTN + frow) * BK;

  v4i fa[2][TM], fb[2][TN];
  // fragment number r (A blocks first, then B blocks) of k-step ks of the stage -> register set buf
  auto load_frag = [&](const char* stage, int ks, int buf, int r) {
    const int coff = ((ks * 2 + fhalf) ^ fsw) * 16;
    if (r < TM) fa[buf][r] = *(const v4i*)(stage + a_lane + r * 32 * BK + coff);
    else fb[buf][r - TM] = *(const v4i*)(stage + b_lane + (r - TM) * 32 * BK + coff);
  };
  auto mfma = [&](int buf, int u) {
    const int i = u / TN, j = u % TN;
    if constexpr (OUTCLS == OUT8)  // rows of the MFMA result = n (4 consecutive n per lane)
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
    else  // rows of the MFMA result = m, lanes run along n
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[buf][i], fb[buf][j], acc[i][j], 0, 0, 0);
  };
  constexpr int NM = TM * TN, NR = TM + TN;
  // One k-step, pinned instruction order: MFMA u, then fragment read u for the next k-step, and
  // ND global->LDS loads spread evenly between the MFMAs.  A wave can only push one such load
  // into the memory pipeline every ~64 cycles, so loads issued back to back stall the wave's
  // instruction stream (and with it the matrix pipe); two or three MFMAs between loads hide it.
  auto kstep = [&](int buf, const char* rd_stage, int rd_ks, bool do_read, int d0, int nd) {
    int d = 0;
#pragma unroll
    for (int u = 0; u < NM; ++u) {
      mfma(buf, u);
      if (do_read) {
#pragma unroll
        for (int r = 0; r < NR; ++r)
          if (r * NM / NR == u || (NM > NR && r == u)) {
            if (NM > NR ? r == u : r * NM / NR == u) load_frag(rd_stage, rd_ks, buf ^ 1, r);
          }
      }
      if (d < nd && (u + 1) * nd >= (d + 1) * NM) {
        dma(d0 + d);
        ++d;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // loads of one k-tile are split over the k-steps: the last k-step (after the barrier) gets
  // LOADS_B of them, the others LOADS_A in total
  constexpr int PER_KS = (LOADS + KS - 1) / KS;
  constexpr int LOADS_B = (LOADS - PER_KS * (KS - 1) > 0) ? LOADS - PER_KS * (KS - 1) : 0;
  constexpr int LOADS_A = LOADS - LOADS_B;

  if (KT > 0) {
#pragma unroll
    for (int t = 0; t < DEPTH; ++t) {
#pragma unroll
      for (int d = 0; d < LOADS; ++d) dma(d);
      dma_advance();
    }
    wait_loads_and_barrier<LOADS*(DEPTH - 1)>();
#pragma unroll
    for (int r = 0; r < NR; ++r) load_frag(lds, 0, 0, r);
  }

  int st = 0;
  for (int kt = 0; kt < KT; ++kt) {
    const char* cur = lds + st * STAGE;
    st = (st + 1 == NSTAGE) ? 0 : st + 1;
    // k-steps 0 .. KS-2: read the fragments of the following k-step, fetch part A of k-tile kt+DEPTH
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
      const int d0 = ks * PER_KS;
      const int nd = (d0 + PER_KS <= LOADS_A) ? PER_KS : (LOADS_A - d0 > 0 ? LOADS_A - d0 : 0);
      kstep(ks & 1, cur, ks + 1, true, d0, nd);
    }
    // every LDS read of this k-tile is issued.  Wait for them and for k-tile kt+1 to have landed
    // (younger loads may stay in flight), then let the workgroup agree: after the barrier the
    // stage of k-tile kt+1 is readable and this k-tile's stage may be overwritten.
    wait_loads_and_barrier<LOADS*(DEPTH - 2) + LOADS_A>();
    // last k-step: first fragments of the next k-tile, part B of the fetch
    kstep((KS - 1) & 1, lds + st * STAGE, 0, kt + 1 < KT, LOADS_A, LOADS_B);
    dma_advance();
  }
  // the trailing (out-of-bounds) loads still write zeros into LDS: drain before re-using it
  wait_loads_and_barrier<0>();

  // ---- epilogue ----
  // The per-element code below is fully unrolled over the accumulator registers, so everything
  // that depends on the epilogue kind is decided once, outside the unrolled part: one uniform
  // branch selects a specialised body, and the remaining run-time options (rounding mode, ReLU,
  // bias present) are folded into branch-free selects.
  const EpiCtx e = make_epi(p, bz);
  char* Cb = (char*)p.C;
  const int lrow = lane & 31, lhi = lane >> 5;
  const bool has_bias = e.bias_kind != TI_BIAS_NONE;

  if constexpr (OUTCLS == OUT8) {
    // acc[i][j][r]: m = m0 + wm*WTM + i*32 + lrow;  n = n0 + wn*WTN + j*32 + 8*(r/4) + 4*lhi + r%4.
    // Quantise and pack 4 consecutive n into a dword X[g] (g = r/4).  Lanes l and l+32 hold the two
    // halves of every 8-byte group of a row, so two half-wave swaps, (X0, X2) and (X1, X3), leave
    // lane l with bytes 0..15 and lane l+32 with bytes 16..31 of the row's 32-byte segment: one
    // 16-byte store per 32x32 block and lane, no trip through LDS.
    // Per element: cvt, mul, (add), clamp in fp32 (v_med3_f32), then one add of 1.5*2^23: that
    // add rounds to the nearest integer, ties to even, and leaves the two's-complement int8 in the
    // low byte of the float's bit pattern.  Clamping first keeps the sum in the exact range; since
    // the bounds are integers, clamp-then-round equals round-then-clamp.  ReLU is a lower bound of 0.
    // (Truncation, the test-time rounding switch, is served by the gather kernel instead.)
    const float q_floor = e.epilogue == TI_EPI_SCALE_RELU_I8 ? 0.0f : -128.0f;
    int8_t* Cz = (int8_t*)Cb + (int64_t)bz * p.sCb;
    const bool vec_ok = ((p.sCm & 15) == 0) && ((((uintptr_t)Cz) & 15) == 0);
    auto body = [&](auto gelu_tag, auto bias_tag) {
      constexpr bool GELU = decltype(gelu_tag)::value;
      constexpr bool BIAS = decltype(bias_tag)::value;
      auto one = [&](int a, float col) -> float {
        float v = (float)a * e.alpha;
        if constexpr (BIAS) v = col + v;
        if constexpr (GELU) v = gelu_tanh_scaled(v, e.beta);
        return __builtin_amdgcn_fmed3f(v, q_floor, 127.0f);
      };
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int nj = n0 + wn * WTN + j * 32;
        float col[4][4];
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            if constexpr (BIAS)
              col[g][t] = column_term_t<GELU ? TI_BIAS_F32 : TI_BIAS_I8>(e, min(nj + 8 * g + 4 * lhi + t, p.N - 1), GELU);
            else
              col[g][t] = 0.0f;
          }
        const int n = nj + 16 * lhi;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          unsigned X[4];
          float f[4][4];
#pragma unroll
          for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int t = 0; t < 4; ++t) f[g][t] = one(acc[i][j][4 * g + t], col[g][t]);
          pack16_q8(f, X);
          const auto s02 = __builtin_amdgcn_permlane32_swap(X[0], X[2], false, false);
          const auto s13 = __builtin_amdgcn_permlane32_swap(X[1], X[3], false, false);
          v4u v;
          v[0] = s02[0]; v[1] = s02[1]; v[2] = s13[0]; v[3] = s13[1];
          const int m = m0 + wm * WTM + i * 32 + lrow;
          if (m >= p.M || n >= p.N) continue;
          int8_t* dst = Cz + (int64_t)m * p.sCm + n;
          if (vec_ok && n + 16 <= p.N) {
            *(v4u*)dst = v;
          } else {
            const int cnt = min(16, p.N - n);
            for (int t = 0; t < cnt; ++t) dst[t] = (int8_t)(v[t >> 2] >> ((t & 3) * 8));
          }
        }
      }
    };
    const bool gelu = e.epilogue == TI_EPI_GELU_I8;
    if (gelu && has_bias) body(std::true_type{}, std::true_type{});
    else if (gelu) body(std::true_type{}, std::false_type{});
    else if (has_bias) body(std::false_type{}, std::true_type{});
    else body(std::false_type{}, std::false_type{});
  } else {
    // acc[i][j][r]: m = m0 + wm*WTM + i*32 + 8*(r/4) + 4*lhi + r%4;  n = n0 + wn*WTN + j*32 + lrow.
    constexpr int ESZ = OUTCLS == OUT32 ? 4 : 2;
    char* Cz = Cb + (int64_t)bz * p.sCb * ESZ;
    // KIND: 0 raw int32 (+ int32 bias), 1 scaled -> int32, 2 scaled -> fp32, 3 -> fp16, 4 -> bf16
    auto body = [&](auto kind_tag) {
      constexpr int KIND = decltype(kind_tag)::value;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn * WTN + j * 32 + lrow;
        const int nc = min(n, p.N - 1);
        const float col = KIND == 0 ? 0.0f : column_term_t<KIND == 1 ? TI_BIAS_I32 : TI_BIAS_F32>(e, nc, false);
        const int bias_i32 = (KIND == 0 && e.bias_kind == TI_BIAS_I32) ? ((const int*)e.bias)[nc] : 0;
        const bool n_ok = n < p.N;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * lhi + (r & 3);
            if (!(n_ok && m < p.M)) continue;
            const int64_t off = (int64_t)m * p.sCm + (int64_t)n * p.sCn;
            const int a = acc[i][j][r];
            if constexpr (KIND == 0) {
              ((int*)Cz)[off] = (int)((unsigned)a + (unsigned)bias_i32);
            } else {
              float v = (float)a * e.alpha;
              const float vb = col + v;
              v = has_bias ? vb : v;
              if constexpr (KIND == 1) ((int*)Cz)[off] = q32(v, e.round_mode);
              else if constexpr (KIND == 2) ((float*)Cz)[off] = v;
              else if constexpr (KIND == 3) ((uint16_t*)Cz)[off] = f32_to_f16_bits(v);
              else ((uint16_t*)Cz)[off] = f32_to_bf16_bits(v);
            }
          }
        }
      }
    };
    if constexpr (OUTCLS == OUT32) {
      if (e.epilogue == TI_EPI_I32) body(std::integral_constant<int, 0>{});
      else if (e.epilogue == TI_EPI_SCALE_I32) body(std::integral_constant<int, 1>{});
      else body(std::integral_constant<int, 2>{});
    } else {
      if (p.out_dtype == TI_F16) body(std::integral_constant<int, 3>{});
      else body(std::integral_constant<int, 4>{});
    }
  }
}

// ---- epilogue of the persistent kernels ----------------------------------------------------------
// Stores one wave's (TM*32) x (TN*32) block of accumulators, whose first row / column in the
// output are mw / nw, through an unconditional, range-checked buffer store per element group
// (elements outside M x N are redirected out of the buffer's range and dropped), so that the
// number of store instructions per tile does not depend on the tile (2-byte outputs: one of two
// constants, by out16_pairs()).  `strip` is the wave's private
// LDS area (int8 outputs only): 32*WTN bytes for the row strip plus WTN floats of column terms.
#ifndef TI_STREAM_STORE_AUX
#define TI_STREAM_STORE_AUX 2  // nt: the outputs are streamed, keep the operand panels in L2
#endif
// bytes of the per-wave LDS strip of the int8 epilogue: 32 rows of the wave's WTN output bytes when
// WTN / 16 is a power of two (the swizzle below needs that), none otherwise (direct stores)
constexpr int epi_strip_bytes(int wtn) { return ((wtn / 16) & (wtn / 16 - 1)) == 0 ? 32 * wtn : 0; }

// 4-byte outputs: every store instruction writes two whole 128-byte lines, which go out non-temporal
// (measured on the P.V shape with fp32 output: 192 -> 162 us)
#ifndef TI_STREAM_STORE32_AUX
#define TI_STREAM_STORE32_AUX 2
#endif
// 2-byte outputs: pairs of neighbouring elements of a row can go out as one aligned dword
__device__ __forceinline__ bool out16_pairs(const GemmParams& p) {
  return !(p.N & 1) && !(p.sCm & 1) && !(p.sCb & 1) && !((uintptr_t)p.C & 3);
}
// LDS_COLS false: `strip` has no room for the column terms; int8 launches with a bias or GELU are not
// compiled in (the host refuses them for such a kernel).
template <int TM, int TN, int OUTCLS, bool LDS_COLS = true>
__device__ __forceinline__ void stream_epilogue(const GemmParams& p, const EpiCtx& e, v16i (&acc)[TM][TN], int bz,
                                                int mw, int nw, char* strip, int lane) {
  constexpr int WTN = TN * 32;
  constexpr int ESZ = OUTCLS == OUT8 ? 1 : (OUTCLS == OUT32 ? 4 : 2);
  const int OOB = (int)0x80000000;
  const int lrow = lane & 31, lhi = lane >> 5;
  const bool has_bias = e.bias_kind != TI_BIAS_NONE;
  const int c_extent = ((p.M - 1) * (int)p.sCm + p.N) * ESZ;
  const __amdgpu_buffer_rsrc_t rC =
      __builtin_amdgcn_make_buffer_rsrc((char*)p.C + (int64_t)bz * p.sCb * ESZ, 0, c_extent, 0x00020000);
  const int ldc = (int)p.sCm;
  if constexpr (OUTCLS == OUT8) {
    // acc[i][j][r]: m = mw + i*32 + lrow;  n = nw + j*32 + 8*(r/4) + 4*lhi + r%4.
    // Quantise (clamp in fp32, then add 1.5*2^23: round to nearest even, int8 in the low byte),
    // pack 4 consecutive n into a dword X[g], g = r/4.  Lanes l and l+32 hold the two halves of
    // every 8-byte group of a row; swapping wave halves of (X0, X2) and of (X1, X3) leaves lane l
    // with bytes 0..15 and lane l+32 with bytes 16..31 of the row's 32-byte segment.  A store
    // of those would touch 32 rows with 32 bytes each; instead the wave writes its 32 x WTN strip
    // to its own LDS area and reads it back with consecutive lanes along a row, so that a store
    // instruction covers 1024/WTN rows with WTN consecutive bytes each.  16-byte segment s of
    // strip row r lives at slot s ^ ((r / WRAP) % SEG), WRAP = rows per 256 bytes: conflict-free
    // for the column-wise writes and the row-wise reads.  The area is private to the wave: no
    // barrier, LDS operations of one wave execute in order.
    constexpr bool VIA_STRIP = epi_strip_bytes(WTN) != 0;
    constexpr int SEG = WTN / 16, RP = VIA_STRIP ? 64 / SEG : 1, WRAP = VIA_STRIP ? 256 / WTN : 1;
    static_assert(!VIA_STRIP || (32 % RP == 0 && 32 / RP == TN), "one read pass per 32-column block");
    float* cols = (float*)(strip + epi_strip_bytes(WTN));
    const float q_floor = e.epilogue == TI_EPI_SCALE_RELU_I8 ? 0.0f : -128.0f;
    const int w_swz = (lrow / WRAP) & (SEG - 1);
    const int r_row = lane / SEG, r_seg = lane % SEG;
    // Store addresses: the lane's own part (its column and its first row, or the out-of-range offset:
    // 2^31, which stays out of range with a row's offset added) is computed once, the part that changes
    // from store to store is a scalar added to it.  Not in the instruction's scalar-offset field as for
    // the 4-byte stores below: the compiler puts no wait state between a 16-byte buffer store with a
    // register in that field and a following VALU write of the store's data registers, and this GPU
    // needs one (the first data dword of some lanes came out overwritten).
    // N % 16 == 0: a 16-byte segment is wholly inside or outside.
    const int s_rows_left = p.M - mw - r_row;                                           // via the strip
    const int s_base = nw + r_seg * 16 < p.N ? (mw + r_row) * ldc + nw + r_seg * 16 : OOB;
    const int d_rows_left = p.M - mw - lrow, d_cols_left = p.N - nw - lhi * 16;         // direct
    const int d_base = (mw + lrow) * ldc + nw + lhi * 16;
    auto body = [&](auto gelu_tag, auto bias_tag) {
      constexpr bool GELU = decltype(gelu_tag)::value;
      constexpr bool BIAS = decltype(bias_tag)::value;
      if constexpr (BIAS) {
        // the wave's WTN per-column terms, once per tile (the loads come before this tile's
        // stores, so waiting for them does not wait for a store)
#pragma unroll
        for (int c = lane; c < WTN; c += 64)
          cols[c] = column_term_t<GELU ? TI_BIAS_F32 : TI_BIAS_I8>(e, min(nw + c, p.N - 1), GELU);
      }
      auto one = [&](int a, float col) -> float {
        float v = (float)a * e.alpha;
        if constexpr (BIAS) v = col + v;
        if constexpr (GELU) v = gelu_tanh_scaled(v, e.beta);
        return __builtin_amdgcn_fmed3f(v, q_floor, 127.0f);
      };
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          unsigned X[4];
          float f[4][4];
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            v4f col = {0.f, 0.f, 0.f, 0.f};
            if constexpr (BIAS) col = *(const v4f*)(cols + j * 32 + 8 * g + 4 * lhi);
#pragma unroll
            for (int t = 0; t < 4; ++t) f[g][t] = one(acc[i][j][4 * g + t], col[t]);
          }
          pack16_q8(f, X);
          const auto s02 = __builtin_amdgcn_permlane32_swap(X[0], X[2], false, false);
          const auto s13 = __builtin_amdgcn_permlane32_swap(X[1], X[3], false, false);
          v4u v;
          v[0] = s02[0]; v[1] = s02[1]; v[2] = s13[0]; v[3] = s13[1];
          if constexpr (VIA_STRIP) {
            *(v4u*)(strip + lrow * WTN + (((2 * j + lhi) ^ w_swz) * 16)) = v;
          } else {
            // no strip for this tile width: the lane stores its 16 bytes of row lrow itself (an
            // instruction touches 32 rows with 32 bytes each; left to L2 to merge into lines)
            const bool in = i * 32 < d_rows_left && j * 32 < d_cols_left;
            __builtin_amdgcn_raw_buffer_store_b128(v, rC, (in ? d_base : OOB) + (i * 32 * ldc + j * 32), 0, 0);
          }
        }
        if constexpr (VIA_STRIP) {
#pragma unroll
          for (int q = 0; q < TN; ++q) {
            const int row = q * RP + r_row;
            const v4u v = *(const v4u*)(strip + row * WTN + ((r_seg ^ ((row / WRAP) & (SEG - 1))) * 16));
            const int R = i * 32 + q * RP;  // row mw + R + r_row
            __builtin_amdgcn_raw_buffer_store_b128(v, rC, (R < s_rows_left ? s_base : OOB) + R * ldc, 0, TI_STREAM_STORE_AUX);
          }
        }
      }
    };
    const bool gelu = e.epilogue == TI_EPI_GELU_I8;
    if constexpr (!LDS_COLS) {
      body(std::false_type{}, std::false_type{});
    } else {
      if (gelu && has_bias) body(std::true_type{}, std::true_type{});
      else if (gelu) body(std::true_type{}, std::false_type{});
      else if (has_bias) body(std::false_type{}, std::true_type{});
      else body(std::false_type{}, std::false_type{});
    }
  } else {
    // acc[i][j][r]: m = mw + i*32 + 8*(r/4) + 4*lhi + r%4;  n = nw + j*32 + lrow.
    // KIND: 0 raw int32 (+ int32 bias), 1 scaled -> int32, 2 scaled -> fp32, 3 -> fp16, 4 -> bf16
    // A store's address is split: the lane's part (its column and its first row, or the out-of-range
    // offset) is one VGPR per column block, the row's part R * pitch rides in the instruction's scalar
    // offset, which the range check ignores; a row beyond M swaps the lane part for the out-of-range
    // offset.  Per store that is a compare and a select, no multiply and no branch.
    const int pitch = ldc * ESZ;
    const int rows_left = p.M - mw - 4 * lhi;
    auto body = [&](auto kind_tag) {
      constexpr int KIND = decltype(kind_tag)::value;
      if constexpr (KIND == 3 || KIND == 4) {
        // 2-byte outputs whose rows keep pairs of elements dword-aligned: straight from the MFMA layout a
        // store instruction would write 64 separate 2-byte pieces.  Instead (a) the upper half-wave of
        // column block j is exchanged with the lower half-wave of block j+1 (v_permlane32_swap), which
        // leaves a register with one row's 64 consecutive elements, and (b) even and odd lanes trade
        // elements of two such rows (one DPP move), so that even lanes hold dwords of row m and odd lanes
        // dwords of row m+1: half the store instructions, each writing two whole 128-byte lines.
        if (out16_pairs(p)) {
          const int odd = lane & 1;
          const int rows_left_pair = p.M - mw - odd;
          // per pair of column blocks: the two column terms and the lane part of the address; the loops
          // run rows outside, column blocks inside, so that a row's range test serves all its stores
          constexpr int NP = TN / 2;
          float col2[NP > 0 ? NP : 1][2];
          int base2[NP > 0 ? NP : 1];
#pragma unroll
          for (int jp = 0; jp < NP; ++jp) {
#pragma unroll
            for (int h = 0; h < 2; ++h) col2[jp][h] = column_term_t<TI_BIAS_F32>(e, min(nw + (2 * jp + h) * 32 + lrow, p.N - 1), false);
            const int n = nw + (2 * jp + lhi) * 32 + (lrow & ~1);  // first element of the lane's dword; N is even
            base2[jp] = n < p.N ? ((mw + odd) * ldc + n) * ESZ : OOB;
          }
#pragma unroll
          for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
              bool in[2];
#pragma unroll
              for (int h = 0; h < 2; ++h) in[h] = i * 32 + 8 * (r >> 2) + 4 * h + (r & 3) < rows_left_pair;
#pragma unroll
              for (int jp = 0; jp < NP; ++jp) {
                unsigned row[2][2];  // [r, r+1][lower, upper half-wave's row]
#pragma unroll
                for (int rr = 0; rr < 2; ++rr) {
                  unsigned bits[2];
#pragma unroll
                  for (int h = 0; h < 2; ++h) {
                    float v = (float)acc[i][2 * jp + h][r + rr] * e.alpha;
                    const float vb = col2[jp][h] + v;
                    v = has_bias ? vb : v;
                    bits[h] = KIND == 3 ? (unsigned)f32_to_f16_bits(v) : (unsigned)f32_to_bf16_bits(v);
                  }
                  const auto sw = __builtin_amdgcn_permlane32_swap(bits[0], bits[1], false, false);
                  row[rr][0] = sw[0];
                  row[rr][1] = sw[1];
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                  const unsigned lo_row = row[0][h], hi_row = row[1][h];  // rows m and m + 1, element n of each
                  const unsigned give = odd ? lo_row : hi_row;
                  const unsigned got = (unsigned)__builtin_amdgcn_mov_dpp((int)give, 0xB1, 0xf, 0xf, true);  // lane ^ 1
                  const unsigned dword = odd ? (got | (hi_row << 16)) : (lo_row | (got << 16));
                  const int R = i * 32 + 8 * (r >> 2) + 4 * h + (r & 3);  // row mw + R + odd
                  __builtin_amdgcn_raw_buffer_store_b32(dword, rC, in[h] ? base2[jp] : OOB, R * pitch, TI_STREAM_STORE32_AUX);
                }
              }
            }
          }
          if constexpr (TN % 2 == 1) {
            // the last column block has no partner: step (b) alone, 64-byte pieces of rows m and m + 1
            constexpr int j = TN - 1;
            const float col = column_term_t<TI_BIAS_F32>(e, min(nw + j * 32 + lrow, p.N - 1), false);
            const int n = nw + j * 32 + (lrow & ~1);
            const int base = n < p.N ? ((mw + 4 * lhi + odd) * ldc + n) * ESZ : OOB;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
              for (int r = 0; r < 16; r += 2) {
                unsigned row[2];
#pragma unroll
                for (int rr = 0; rr < 2; ++rr) {
                  float v = (float)acc[i][j][r + rr] * e.alpha;
                  const float vb = col + v;
                  v = has_bias ? vb : v;
                  row[rr] = KIND == 3 ? (unsigned)f32_to_f16_bits(v) : (unsigned)f32_to_bf16_bits(v);
                }
                const unsigned give = odd ? row[0] : row[1];
                const unsigned got = (unsigned)__builtin_amdgcn_mov_dpp((int)give, 0xB1, 0xf, 0xf, true);
                const unsigned dword = odd ? (got | (row[1] << 16)) : (row[0] | (got << 16));
                const int R = i * 32 + 8 * (r >> 2) + (r & 3);  // row mw + R + 4 * lhi + odd
                __builtin_amdgcn_raw_buffer_store_b32(dword, rC, R < rows_left - odd ? base : OOB, R * pitch, TI_STREAM_STORE32_AUX);
              }
            }
          }
          return;
        }
      }
      if constexpr (KIND == 2) {
        if (p.resid) {
          // fp32 output plus a residual of the same shape (C = epilogue value + resid[m][n], the sum rounded
          // once more, as the separate addition would): the residual's elements are fetched through a
          // descriptor of their own with the store's addressing, four rows of the tile at a time and one
          // group ahead, so that the wait for a group counts only the stores issued since and never waits
          // for them.
          const __amdgpu_buffer_rsrc_t rR =
              __builtin_amdgcn_make_buffer_rsrc((void*)p.resid, 0, ((p.M - 1) * (int)p.resid_rs + p.N) * 4, 0x00020000);
          const int rpitch = (int)p.resid_rs * 4;
          float colr[TN];
          int base_c[TN], base_r[TN];
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const int n = nw + j * 32 + lrow;
            colr[j] = column_term_t<TI_BIAS_F32>(e, min(n, p.N - 1), false);
            base_c[j] = n < p.N ? ((mw + 4 * lhi) * ldc + n) * ESZ : OOB;
            base_r[j] = n < p.N ? ((mw + 4 * lhi) * (int)p.resid_rs + n) * 4 : OOB;
          }
          constexpr int NG = TM * 4;  // groups of 4 rows: block i, quarter q = r / 4
          float res[2][4][TN];
          auto load_group = [&](int g, float (&dst)[4][TN]) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int R = (g >> 2) * 32 + 8 * (g & 3) + t;  // row mw + R + 4 * lhi
              const bool in = R < rows_left;
#pragma unroll
              for (int j = 0; j < TN; ++j)
                dst[t][j] = __uint_as_float((unsigned)__builtin_amdgcn_raw_buffer_load_b32(rR, in ? base_r[j] : OOB, R * rpitch, 0));
            }
          };
          load_group(0, res[0]);
#pragma unroll
          for (int g = 0; g < NG; ++g) {
            if (g + 1 < NG) load_group(g + 1, res[(g + 1) & 1]);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int R = (g >> 2) * 32 + 8 * (g & 3) + t;
              const bool in = R < rows_left;
#pragma unroll
              for (int j = 0; j < TN; ++j) {
                float v = (float)acc[g >> 2][j][4 * (g & 3) + t] * e.alpha;
                const float vb = colr[j] + v;
                v = has_bias ? vb : v;
                v = v + res[g & 1][t][j];
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rC, in ? base_c[j] : OOB, R * pitch, TI_STREAM_STORE32_AUX);
              }
            }
          }
          return;
        }
      }
      // rows outside, column blocks inside: a row's range test serves all its stores
      float col[TN];
      int bias_i32[TN], base[TN];
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = nw + j * 32 + lrow;
        const int nc = min(n, p.N - 1);
        col[j] = KIND == 0 ? 0.0f : column_term_t<KIND == 1 ? TI_BIAS_I32 : TI_BIAS_F32>(e, nc, false);
        bias_i32[j] = (KIND == 0 && e.bias_kind == TI_BIAS_I32) ? ((const int*)e.bias)[nc] : 0;
        base[j] = n < p.N ? ((mw + 4 * lhi) * ldc + n) * ESZ : OOB;
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int R = i * 32 + 8 * (r >> 2) + (r & 3);  // row mw + R + 4 * lhi
          const bool in = R < rows_left;
          const int soff = R * pitch;
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const int off = in ? base[j] : OOB;
            const int a = acc[i][j][r];
            if constexpr (KIND == 0) {
              __builtin_amdgcn_raw_buffer_store_b32((unsigned)a + (unsigned)bias_i32[j], rC, off, soff, TI_STREAM_STORE32_AUX);
            } else {
              float v = (float)a * e.alpha;
              const float vb = col[j] + v;
              v = has_bias ? vb : v;
              if constexpr (KIND == 1) __builtin_amdgcn_raw_buffer_store_b32((unsigned)q32(v, e.round_mode), rC, off, soff, TI_STREAM_STORE32_AUX);
              else if constexpr (KIND == 2) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), rC, off, soff, TI_STREAM_STORE32_AUX);
              else if constexpr (KIND == 3) __builtin_amdgcn_raw_buffer_store_b16(f32_to_f16_bits(v), rC, off, soff, 0);
              else __builtin_amdgcn_raw_buffer_store_b16(f32_to_bf16_bits(v), rC, off, soff, 0);
            }
          }
        }
      }
    };
    if constexpr (OUTCLS == OUT32) {
      if (e.epilogue == TI_EPI_I32) body(std::integral_constant<int, 0>{});
      else if (e.epilogue == TI_EPI_SCALE_I32) body(std::integral_constant<int, 1>{});
      else body(std::integral_constant<int, 2>{});
    } else {
      if (p.out_dtype == TI_F16) body(std::integral_constant<int, 3>{});
      else body(std::integral_constant<int, 4>{});
    }
  }
}

// ---- persistent ("stream") variant of the fast family --------------------------------------------
//
// One workgroup per CU slot walks a list of output tiles, and the global -> LDS pipeline does not
// stop at a tile boundary: the k-tiles of all its tiles form one stream, the loads run NSTAGE-1
// k-tiles ahead of the MFMAs, so the first operands of the next tile arrive while the epilogue of
// the current one runs, and the epilogue's stores drain while the next tile computes.  What a
// one-tile-per-workgroup launch pays per tile (first-load latency, the drain of its stores before
// the workgroup can retire, the launch of its successor) is paid once per workgroup instead.
//
// Work list: the tiles*batch items are folded into 8 contiguous ranges, one per XCD (workgroup
// b runs on XCD b % 8 when the grid is a multiple of 8), and the workgroups of an XCD interleave
// over its range, so that tiles running at the same time share operand panels in that XCD's L2.
//
// Load counting.  vmcnt retires loads and stores in order.  The waits inside a k-loop name how
// many younger operations may still be in flight; the epilogue's stores are younger than the
// loads that were issued before it, so for the first NSTAGE-2 k-tiles after an epilogue the
// count is raised by the number of store instructions STORES, which is exact because every store
// is an unconditional buffer store (elements outside M x N are redirected out of the buffer's
// range and dropped by the range check).  A count too small would only wait longer; 63 is the
// counter's maximum.
//
// 4-byte outputs are stored straight from the MFMA layout (32 consecutive n per row and
// instruction), 2-byte outputs as dword pairs after a lane exchange where the output's alignment
// allows, int8 outputs exchange dwords between the two wave halves so that every lane owns 16
// consecutive bytes of a row and go through a wave-private LDS strip.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int SWZ, int NSTAGE, int OUTCLS, int OCC = 1>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64, (WAVES_M * WAVES_N * OCC + 3) / 4) void gemm_mfma_stream_kernel(GemmParams p) {
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int CH = BK / 16;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int KS = BK / 32;
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  constexpr int STAGE = A_BYTES + B_BYTES;
  // int8 outputs: per wave a 32-row strip of its WTN output bytes (to turn the MFMA layout into
  // long row segments) and WTN per-column fp32 terms
  constexpr int STRIP = epi_strip_bytes(WTN), COLS = 4 * WTN;
  constexpr int EPI_LDS = OUTCLS == OUT8 ? WAVES_M * WAVES_N * (STRIP + COLS) : 0;
  constexpr int LDS_BYTES = NSTAGE * STAGE + EPI_LDS;
  constexpr int DEPTH = NSTAGE - 1;
  constexpr int STORES = OUTCLS == OUT8 ? TM * TN : TM * TN * 16;  // store instructions per tile
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 64 == 0, "tile shape");
  static_assert(NSTAGE >= 3 && LDS_BYTES <= 160 * 1024, "LDS budget");

  __shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // ---- this workgroup's items: ranks first, first + step, ... (count of them)
  const int T = p.tiles_m * p.tiles_n;
  const int W = T * p.batch;
  int first, step, count;
  {
    const int G = (int)gridDim.x, b = (int)blockIdx.x;
    if (G & 7) {
      first = b;
      step = G;
      count = b < W ? (W - b + G - 1) / G : 0;
    } else {
      const int xcd = b & 7, l = b >> 3, nb = G >> 3;
      const int per = W >> 3, rem = W & 7;
      const int cnt = per + (xcd < rem ? 1 : 0);
      first = xcd * per + min(xcd, rem) + l;
      step = nb;
      count = l < cnt ? (cnt - l + nb - 1) / nb : 0;
    }
    first = __builtin_amdgcn_readfirstlane(first);
    step = __builtin_amdgcn_readfirstlane(step);
    count = __builtin_amdgcn_readfirstlane(count);
  }
  if (count == 0) return;
  auto locate = [&](int i, int& bz, int& m0, int& n0) {
    const int g = first + i * step;
    const int b_ = g / T;
    int tm, tn;
    tile_from_rank(p, g - b_ * T, tm, tn);
    bz = __builtin_amdgcn_readfirstlane(b_);
    m0 = __builtin_amdgcn_readfirstlane(tm * BM);
    n0 = __builtin_amdgcn_readfirstlane(tn * BN);
  };

  const int lda = (int)p.sAm, ldb = (int)p.sBn;
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const unsigned wave_slot = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);

  // thread-constant offsets relative to the tile origin; the origin lives in the descriptors
  TileLoader<BM, BK, NT, SWZ> la;
  TileLoader<BN, BK, NT, SWZ> lb;
  la.init(tid, 0, lda, p.K);
  lb.init(tid, 0, ldb, p.K);
  constexpr int A_IT = decltype(la)::IT, B_IT = decltype(lb)::IT;
  constexpr int LOADS = A_IT + B_IT;
  const int KT = (p.K + BK - 1) / BK;
  const int KEND = KT * BK;
  const int OOB = (int)0x80000000;

  // ---- issue side of the stream: item i_issue, k offset k_issue, LDS stage st_issue
  v4i rA, rB;
  int i_issue = 0, k_issue = 0, st_issue = 0;
  auto aim = [&](int i) {
    if (i < count) {
      int bz, m0, n0;
      locate(i, bz, m0, n0);
      // rows at or past M (N) and bytes past K of the last row read as zero
      rA = make_rsrc(p.A + (int64_t)bz * p.sAb + (int64_t)m0 * lda, (p.M - 1 - m0) * lda + p.K);
      rB = make_rsrc(p.B + (int64_t)bz * p.sBb + (int64_t)n0 * ldb, (p.N - 1 - n0) * ldb + p.K);
    } else {
      // past the last item: empty buffers, the loads write zeros into stages nobody reads, which
      // keeps the number of loads in flight (and so the counts to wait for) constant
      rA = make_rsrc(p.A, 0);
      rB = make_rsrc(p.B, 0);
    }
  };
  auto dma = [&](int d) {
    if (d < A_IT) {
      const unsigned dst = wave_slot + st_issue * STAGE + d * NT * 16;
      dma16_to_lds(rA, (k_issue < la.klim[d]) ? la.voff[d] : OOB, k_issue, dst);
    } else {
      const int e = d - A_IT;
      const unsigned dst = wave_slot + st_issue * STAGE + A_BYTES + e * NT * 16;
      dma16_to_lds(rB, (k_issue < lb.klim[e]) ? lb.voff[e] : OOB, k_issue, dst);
    }
  };
  auto dma_advance = [&]() {
    k_issue += BK;
    st_issue = (st_issue + 1 == NSTAGE) ? 0 : st_issue + 1;
    if (k_issue >= KEND) {
      k_issue = 0;
      ++i_issue;
      aim(i_issue);
    }
  };

  v16i acc[TM][TN];
  const int frow = lane & 31;
  const int fsw = (frow >> SWZ) & (CH - 1);
  const int fhalf = lane >> 5;
  const int a_lane = (wm * WTM + frow) * BK;
  const int b_lane = A_BYTES + (wn * WTN + frow) * BK;

  v4i fa[2][TM], fb[2][TN];
  auto load_frag = [&](const char* stage, int ks, int buf, int r) {
    const int coff = ((ks * 2 + fhalf) ^ fsw) * 16;
    if (r < TM) fa[buf][r] = *(const v4i*)(stage + a_lane + r * 32 * BK + coff);
    else fb[buf][r - TM] = *(const v4i*)(stage + b_lane + (r - TM) * 32 * BK + coff);
  };
  // first: the tile's first k-step starts from a zero C operand (an inline constant of the
  // instruction) instead of accumulators cleared with one move each
  auto mfma = [&](int buf, int u, auto first_tag) {
    const int i = u / TN, j = u % TN;
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const v16i c = decltype(first_tag)::value ? zero : acc[i][j];
    if constexpr (OUTCLS == OUT8)  // rows of the MFMA result = n (4 consecutive n per lane)
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[buf][j], fa[buf][i], c, 0, 0, 0);
    else  // rows of the MFMA result = m, lanes run along n
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[buf][i], fb[buf][j], c, 0, 0, 0);
  };
  constexpr int NM = TM * TN, NR = TM + TN;
  auto kstep = [&](int buf, const char* rd_stage, int rd_ks, bool do_read, int d0, int nd, auto first_tag) {
    int d = 0;
#pragma unroll
    for (int u = 0; u < NM; ++u) {
      mfma(buf, u, first_tag);
      if (do_read) {
#pragma unroll
        for (int r = 0; r < NR; ++r)
          if (r * NM / NR == u || (NM > NR && r == u)) {
            if (NM > NR ? r == u : r * NM / NR == u) load_frag(rd_stage, rd_ks, buf ^ 1, r);
          }
      }
      if (d < nd && (u + 1) * nd >= (d + 1) * NM) {
        dma(d0 + d);
        ++d;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  constexpr int PER_KS = (LOADS + KS - 1) / KS;
  constexpr int LOADS_B = (LOADS - PER_KS * (KS - 1) > 0) ? LOADS - PER_KS * (KS - 1) : 0;
  constexpr int LOADS_A = LOADS - LOADS_B;
  constexpr int N_STEADY = LOADS * (DEPTH - 2) + LOADS_A;
  constexpr int N_AFTER_STORES = (N_STEADY + STORES > 63) ? 63 : N_STEADY + STORES;
  // 2-byte outputs stored as dword pairs take half the store instructions
  constexpr bool CAN_PAIR = OUTCLS == OUT16;
  constexpr int N_AFTER_PAIRED = (N_STEADY + STORES / 2 > 63) ? 63 : N_STEADY + STORES / 2;
  const bool paired = CAN_PAIR && out16_pairs(p);

  // ---- fill the pipeline
  aim(0);
#pragma unroll
  for (int t = 0; t < DEPTH; ++t) {
#pragma unroll
    for (int d = 0; d < LOADS; ++d) dma(d);
    dma_advance();
  }
  wait_loads_and_barrier<LOADS*(DEPTH - 1)>();

  int st = 0;
  for (int it = 0; it < count; ++it) {
    int bz, m0, n0;
    locate(it, bz, m0, n0);
    const EpiCtx e = make_epi(p, bz);  // scalar loads, long done when the epilogue needs them
    if (KT == 0) {  // K == 0: no MFMA defines the sums
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    }
    // k-tile 0 of this item has landed: the barrier of the previous k-tile (or the one above) saw to it
#pragma unroll
    for (int r = 0; r < NR; ++r) load_frag(lds + st * STAGE, 0, 0, r);

    for (int kt = 0; kt < KT; ++kt) {
      const char* cur = lds + st * STAGE;
      st = (st + 1 == NSTAGE) ? 0 : st + 1;
#pragma unroll
      for (int ks = 0; ks < KS - 1; ++ks) {
        const int d0 = ks * PER_KS;
        const int nd = (d0 + PER_KS <= LOADS_A) ? PER_KS : (LOADS_A - d0 > 0 ? LOADS_A - d0 : 0);
        if (ks == 0 && kt == 0) kstep(0, cur, 1, true, d0, nd, std::true_type{});  // starts the tile's sums
        else kstep(ks & 1, cur, ks + 1, true, d0, nd, std::false_type{});
      }
      // all LDS reads of this k-tile are issued; the next k-tile must have landed before the
      // barrier.  The stores of the previous item's epilogue are younger than that k-tile while
      // it is one of those that were fetched before the epilogue.
      if (it > 0 && kt < DEPTH - 1) {
        if (paired) wait_loads_and_barrier<N_AFTER_PAIRED>();
        else wait_loads_and_barrier<N_AFTER_STORES>();
      }
      else wait_loads_and_barrier<N_STEADY>();
      kstep((KS - 1) & 1, lds + st * STAGE, 0, kt + 1 < KT, LOADS_A, LOADS_B, std::false_type{});
      dma_advance();
    }

    // ---- epilogue
    stream_epilogue<TM, TN, OUTCLS>(p, e, acc, bz, m0 + wm * WTM, n0 + wn * WTN,
                                    lds + NSTAGE * STAGE + wave * (STRIP + COLS), lane);
  }
  // the trailing (empty-buffer) loads still write zeros into LDS: they must land before the
  // workgroup's LDS is handed to another one
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---- short-K persistent kernel -------------------------------------------------------------------
//
// K <= 128 (the attention Q.K^T: K is the head dimension): a 256 x 256 tile is 32 MFMAs per wave
// against 128 outputs per lane to scale, clamp, round, pack and store; the k-loop machinery of
// gemm_mfma_stream_kernel (a barrier and a wait per k-tile, loads dealt over the k-steps) buys nothing
// here.  The whole K of a tile sits in LDS (two tile buffers: one being read, one being loaded) and
// there is one barrier per tile: every wave issues its share of tile t+1's loads right after
// barrier t (into the buffer of tile t-1: all of its readers passed that barrier), runs tile t's
// MFMAs and epilogue, and waits for those loads before barrier t+1; the only younger operations are
// the epilogue's unconditional stores, so the count to wait for is exact.
// 4 x 2 waves of 64 x 128 outputs: an int8 row piece of a wave is a whole 128-byte line (with 2 x 4
// waves it is 64 bytes, and a write-only probe of this output pattern runs at 3.5 TB/s with 64-byte
// pieces against 5.3-5.6 TB/s with 128 bytes and more).  The 32 x 128-byte strips of the 8 waves
// and the two tile buffers fill the 160 KB of LDS exactly: there is no room to stage per-column
// terms, so int8 launches with a bias or the GELU epilogue go to the other kernels (the BMMs have
// neither).
// Tried and removed: a ping-pong order (the two waves of a SIMD in opposite order between barriers,
// one wave's MFMAs under the other's epilogue), 9-16 % slower than this order for every pairing of
// waves (160 x 2048 x 2048 x 128: 193 us against 209-224 us).
template <int OUTCLS>
__global__ __launch_bounds__(512) void gemm_mfma_shortk_kernel(GemmParams p) {
  constexpr int BM = 256, BN = 256, BK = 64, WAVES_N = 2, SWZ = 2, KTMAX = 2;
  constexpr int NT = 512, CH = BK / 16;
  constexpr int WTM = 64, WTN = 128, TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK, STAGE = A_BYTES + B_BYTES, TILE = KTMAX * STAGE;
  constexpr int STRIP = epi_strip_bytes(WTN);
  constexpr int EPI_LDS = OUTCLS == OUT8 ? 8 * STRIP : 0;
  constexpr int LDS_BYTES = 2 * TILE + EPI_LDS;
  constexpr int STORES_ALL = OUTCLS == OUT8 ? TM * TN : TM * TN * 16;  // store instructions per tile and wave
  constexpr int STORES = STORES_ALL > 63 ? 63 : STORES_ALL;            // 63: the counter's maximum (waits longer)
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");

  __shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // ---- this workgroup's items (as in gemm_mfma_stream_kernel)
  const int T = p.tiles_m * p.tiles_n;
  const int W = T * p.batch;
  int first, step, count;
  {
    const int G = (int)gridDim.x, b = (int)blockIdx.x;
    if (G & 7) {
      first = b;
      step = G;
      count = b < W ? (W - b + G - 1) / G : 0;
    } else {
      const int xcd = b & 7, l = b >> 3, nb = G >> 3;
      const int per = W >> 3, rem = W & 7;
      const int cnt = per + (xcd < rem ? 1 : 0);
      first = xcd * per + min(xcd, rem) + l;
      step = nb;
      count = l < cnt ? (cnt - l + nb - 1) / nb : 0;
    }
    first = __builtin_amdgcn_readfirstlane(first);
    step = __builtin_amdgcn_readfirstlane(step);
    count = __builtin_amdgcn_readfirstlane(count);
  }
  if (count == 0) return;
  auto locate = [&](int i, int& bz, int& m0, int& n0) {
    const int g = first + i * step;
    const int b_ = g / T;
    int tm, tn;
    tile_from_rank(p, g - b_ * T, tm, tn);
    bz = __builtin_amdgcn_readfirstlane(b_);
    m0 = __builtin_amdgcn_readfirstlane(tm * BM);
    n0 = __builtin_amdgcn_readfirstlane(tn * BN);
  };

  const int lda = (int)p.sAm, ldb = (int)p.sBn;
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const unsigned wave_slot = __builtin_amdgcn_readfirstlane(lds_base + wave * 1024);
  TileLoader<BM, BK, NT, SWZ> la;
  TileLoader<BN, BK, NT, SWZ> lb;
  la.init(tid, 0, lda, p.K);
  lb.init(tid, 0, ldb, p.K);
  constexpr int A_IT = decltype(la)::IT, B_IT = decltype(lb)::IT;
  const int KT = (p.K + BK - 1) / BK;  // 1 or 2 (host)
  const int OOB = (int)0x80000000;

  // all of item i's K into tile buffer buf; rows at or past M (N) and bytes past K read as zero
  auto load_tile = [&](int i, int buf) {
    int bz, m0, n0;
    locate(i, bz, m0, n0);
    const v4i rA = make_rsrc(p.A + (int64_t)bz * p.sAb + (int64_t)m0 * lda, (p.M - 1 - m0) * lda + p.K);
    const v4i rB = make_rsrc(p.B + (int64_t)bz * p.sBb + (int64_t)n0 * ldb, (p.N - 1 - n0) * ldb + p.K);
#pragma unroll
    for (int kt = 0; kt < KTMAX; ++kt) {
      if (kt < KT) {
        const int k0 = kt * BK;
        const unsigned dst = wave_slot + buf * TILE + kt * STAGE;
#pragma unroll
        for (int d = 0; d < A_IT; ++d) dma16_to_lds(rA, (k0 < la.klim[d]) ? la.voff[d] : OOB, k0, dst + d * NT * 16);
#pragma unroll
        for (int d = 0; d < B_IT; ++d) dma16_to_lds(rB, (k0 < lb.klim[d]) ? lb.voff[d] : OOB, k0, dst + A_BYTES + d * NT * 16);
      }
    }
  };

  v16i acc[TM][TN];
  const int frow = lane & 31;
  const int fsw = (frow >> SWZ) & (CH - 1);
  const int fhalf = lane >> 5;
  const int a_lane = (wm * WTM + frow) * BK;
  const int b_lane = A_BYTES + (wn * WTN + frow) * BK;
  v4i fa[2][TM], fb[2][TN];
  constexpr int NM = TM * TN, NR = TM + TN;
  auto load_frag = [&](const char* stage, int ks, int buf, int r) {
    const int coff = ((ks * 2 + fhalf) ^ fsw) * 16;
    if (r < TM) fa[buf][r] = *(const v4i*)(stage + a_lane + r * 32 * BK + coff);
    else fb[buf][r - TM] = *(const v4i*)(stage + b_lane + (r - TM) * 32 * BK + coff);
  };
  // one k-step: the MFMAs on fragment set buf, the reads of the next k-step's fragments (set buf ^ 1)
  // spread between them; first: the sums start from a zero C operand
  auto kstep = [&](int buf, const char* rd_stage, int rd_ks, bool do_read, auto first_tag) {
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < NM; ++u) {
      const int i = u / TN, j = u % TN;
      const v16i c = decltype(first_tag)::value ? zero : acc[i][j];
      if constexpr (OUTCLS == OUT8) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[buf][j], fa[buf][i], c, 0, 0, 0);
      else acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[buf][i], fb[buf][j], c, 0, 0, 0);
      if (do_read && u < NR) load_frag(rd_stage, rd_ks, buf ^ 1, u);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  load_tile(0, 0);
  for (int t = 0; t < count; ++t) {
    // this wave's loads of tile t have landed and its LDS reads are done; then meet the others.  The
    // operations younger than those loads are the stores of tile t-1's epilogue.
    if (t >= 1) wait_loads_and_barrier<STORES>();
    else wait_loads_and_barrier<0>();
    if (t + 1 < count) load_tile(t + 1, (t + 1) & 1);
    const char* s0 = lds + (t & 1) * TILE;
#pragma unroll
    for (int r = 0; r < NR; ++r) load_frag(s0, 0, 0, r);
    kstep(0, s0, 1, true, std::true_type{});
    if (KT == 2) {
      kstep(1, s0 + STAGE, 0, true, std::false_type{});
      kstep(0, s0 + STAGE, 1, true, std::false_type{});
    }
    kstep(1, s0, 0, false, std::false_type{});
    int bz, m0, n0;
    locate(t, bz, m0, n0);
    const EpiCtx e = make_epi(p, bz);
    stream_epilogue<TM, TN, OUTCLS, false>(p, e, acc, bz, m0 + wm * WTM, n0 + wn * WTN, lds + 2 * TILE + wave * STRIP, lane);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---- wave-specialised persistent kernel -------------------------------------------------------
//
// A wave that issues a 16-byte-per-lane load is held for about 64 cycles by the address path, and
// while it is held it issues no MFMA: with the loads spread over the MFMA waves the matrix pipe
// idles about a quarter of the k-loop.  Here the two jobs belong to different waves of the
// workgroup.  PW producer waves do nothing but the global -> LDS loads of the k-tile stream
// (tile list, descriptors, NSTAGE-1 k-tiles ahead, as in gemm_mfma_stream_kernel); the
// WAVES_M x WAVES_N consumer waves only read fragments from LDS and issue MFMAs, then run the
// epilogue.  With one consumer and one producer wave per SIMD the producer's address phases
// overlap the consumer's MFMAs.
//
// Hand-over, one s_barrier per k-tile joined by all waves.  Iteration g (stream k-tile g):
//   producer: issue the loads of k-tile g+NSTAGE-1 into the stage of k-tile g-1 (its readers
//             finished before barrier g-1); wait until k-tile g+1 has landed; barrier g.
//   consumer: k-steps 0..KS-2 of k-tile g (all LDS reads of its stage issued and complete);
//             barrier g; last k-step, reading the first fragments of k-tile g+1 meanwhile.
// The consumers issue no loads, so their stores (and bias loads) interfere with no counter; the
// producers run ahead during an epilogue until the next barrier holds them.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int SWZ, int NSTAGE, int OUTCLS, int PW>
__global__ __launch_bounds__((WAVES_M * WAVES_N + PW) * 64) void gemm_mfma_ws_kernel(GemmParams p) {
  constexpr int NWC = WAVES_M * WAVES_N;  // consumer waves
  constexpr int NTP = PW * 64;            // producer threads
  constexpr int CH = BK / 16;
  constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int KS = BK / 32;
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  constexpr int STAGE = A_BYTES + B_BYTES;
  constexpr int STRIP = epi_strip_bytes(WTN), COLS = 4 * WTN;
  constexpr int EPI_LDS = OUTCLS == OUT8 ? NWC * (STRIP + COLS) : 0;
  constexpr int LDS_BYTES = NSTAGE * STAGE + EPI_LDS;
  constexpr int DEPTH = NSTAGE - 1;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 64 == 0, "tile shape");
  static_assert(NSTAGE >= 3 && LDS_BYTES <= 160 * 1024, "LDS budget");

  __shared__ __attribute__((aligned(16))) char lds[LDS_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- this workgroup's items: ranks first, first + step, ... (count of them).  An item is a tile
  // of a batch entry, or, with split K (batch == 1), one of the `splits` runs of k-tiles of a tile;
  // the runs of a tile are neighbours in the list, so they are worked on at the same time.
  const int T = p.tiles_m * p.tiles_n;
  const int SPL = p.splits;
  const int W = T * p.batch * SPL;
  int first, step, count;
  {
    const int G = (int)gridDim.x, b = (int)blockIdx.x;
    if (G & 7) {
      first = b;
      step = G;
      count = b < W ? (W - b + G - 1) / G : 0;
    } else {
      const int xcd = b & 7, l = b >> 3, nb = G >> 3;
      const int per = W >> 3, rem = W & 7;
      const int cnt = per + (xcd < rem ? 1 : 0);
      first = xcd * per + min(xcd, rem) + l;
      step = nb;
      count = l < cnt ? (cnt - l + nb - 1) / nb : 0;
    }
    first = __builtin_amdgcn_readfirstlane(first);
    step = __builtin_amdgcn_readfirstlane(step);
    count = __builtin_amdgcn_readfirstlane(count);
  }
  if (count == 0) return;
  const int KT = (p.K + BK - 1) / BK;
  // item i: batch entry bz, tile origin (m0, n0), tile rank, split s with k-tiles [kt0, kt0 + kts)
  auto locate = [&](int i, int& bz, int& m0, int& n0, int& rank, int& s, int& kt0, int& kts) {
    int g = first + i * step;
    int s_ = 0;
    if (SPL > 1) {
      s_ = g % SPL;
      g /= SPL;
    }
    const int b_ = g / T;
    int tm, tn;
    tile_from_rank(p, g - b_ * T, tm, tn);
    bz = __builtin_amdgcn_readfirstlane(b_);
    m0 = __builtin_amdgcn_readfirstlane(tm * BM);
    n0 = __builtin_amdgcn_readfirstlane(tn * BN);
    rank = __builtin_amdgcn_readfirstlane(g - b_ * T);
    s = __builtin_amdgcn_readfirstlane(s_);
    kt0 = SPL > 1 ? s * p.kt_split : 0;
    kts = SPL > 1 ? min(p.kt_split, KT - kt0) : KT;
  };
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;

  if (wave >= NWC) {
    // ================================ producer ================================
    const int ptid = tid - NWC * 64;
    const int lda = (int)p.sAm, ldb = (int)p.sBn;
    const unsigned wave_slot = __builtin_amdgcn_readfirstlane(lds_base + (wave - NWC) * 1024);
    TileLoader<BM, BK, NTP, SWZ> la;
    TileLoader<BN, BK, NTP, SWZ> lb;
    la.init(ptid, 0, lda, p.K);
    lb.init(ptid, 0, ldb, p.K);
    constexpr int A_IT = decltype(la)::IT, B_IT = decltype(lb)::IT;
    constexpr int LOADS = A_IT + B_IT;
    static_assert(LOADS * DEPTH <= 63, "loads in flight must fit the counter");
    const int OOB = (int)0x80000000;
    v4i rA, rB;
    int i_issue = 0, k_issue = 0, st_issue = 0, kt_left = 0;
    // one column of tiles: every byte of A is read exactly once, so it need not stay in the caches
    const bool a_once = p.tiles_n == 1;
    auto aim = [&](int i) {
      kt_left = KT;
      k_issue = 0;
      if (i < count) {
        int bz, m0, n0, rank, sp, kt0, kts;
        locate(i, bz, m0, n0, rank, sp, kt0, kts);
        kt_left = kts;
        k_issue = kt0 * BK;
        // rows at or past M (N) and bytes past K of the last row read as zero
        rA = make_rsrc(p.A + (int64_t)bz * p.sAb + (int64_t)m0 * lda, (p.M - 1 - m0) * lda + p.K);
        rB = make_rsrc(p.B + (int64_t)bz * p.sBb + (int64_t)n0 * ldb, (p.N - 1 - n0) * ldb + p.K);
      } else {
        // past the last item: empty buffers, zeros into stages nobody reads; the number of loads
        // in flight, and so the count to wait for, stays constant
        rA = make_rsrc(p.A, 0);
        rB = make_rsrc(p.B, 0);
      }
    };
    auto issue_ktile = [&]() {
      if (a_once) {
#pragma unroll
        for (int d = 0; d < A_IT; ++d)
          dma16_to_lds_stream(rA, (k_issue < la.klim[d]) ? la.voff[d] : OOB, k_issue, wave_slot + st_issue * STAGE + d * NTP * 16);
      } else {
#pragma unroll
        for (int d = 0; d < A_IT; ++d)
          dma16_to_lds(rA, (k_issue < la.klim[d]) ? la.voff[d] : OOB, k_issue, wave_slot + st_issue * STAGE + d * NTP * 16);
      }
#pragma unroll
      for (int d = 0; d < B_IT; ++d)
        dma16_to_lds(rB, (k_issue < lb.klim[d]) ? lb.voff[d] : OOB, k_issue,
                     wave_slot + st_issue * STAGE + A_BYTES + d * NTP * 16);
      k_issue += BK;
      st_issue = (st_issue + 1 == NSTAGE) ? 0 : st_issue + 1;
      if (--kt_left == 0) {
        ++i_issue;
        aim(i_issue);
      }
    };
    if (wave == NWC) TI_TL(0);
    aim(0);
#pragma unroll
    for (int t = 0; t < DEPTH; ++t) issue_ktile();
    wait_loads_and_barrier<LOADS*(DEPTH - 1)>();  // k-tile 0 landed
    if (wave == NWC) TI_TL(1);
    int total = count * KT;  // k-tiles of all items = barriers to join
    if (SPL > 1) {
      total = 0;
      for (int i = 0; i < count; ++i) {
        int bz, m0, n0, rank, sp, kt0, kts;
        locate(i, bz, m0, n0, rank, sp, kt0, kts);
        total += kts;
      }
    }
    for (int g = 0; g < total; ++g) {
      issue_ktile();                                // k-tile g + DEPTH
      wait_loads_and_barrier<LOADS*(DEPTH - 1)>();  // k-tile g + 1 landed; barrier g
    }
    // the trailing (empty-buffer) loads still write zeros into LDS: they must land before the
    // workgroup's LDS is handed to another one
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }

  // ================================ consumer ================================
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  v16i acc[TM][TN];
  const int frow = lane & 31;
  const int fsw = (frow >> SWZ) & (CH - 1);
  const int fhalf = lane >> 5;
  const int a_lane = (wm * WTM + frow) * BK;
  const int b_lane = A_BYTES + (wn * WTN + frow) * BK;
  v4i fa[2][TM], fb[2][TN];
  auto load_frag = [&](const char* stage, int ks, int buf, int r) {
    const int coff = ((ks * 2 + fhalf) ^ fsw) * 16;
    if (r < TM) fa[buf][r] = *(const v4i*)(stage + a_lane + r * 32 * BK + coff);
    else fb[buf][r - TM] = *(const v4i*)(stage + b_lane + (r - TM) * 32 * BK + coff);
  };
  // first: the tile's first k-step starts from a zero C operand (an inline constant of the
  // instruction) instead of accumulators cleared with one move each: 16 * TM * TN vector
  // instructions per tile less, which is a seventh of the vector work of a K = 128 tile
  auto mfma = [&](int buf, int u, auto first_tag) {
    const int i = u / TN, j = u % TN;
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const v16i c = decltype(first_tag)::value ? zero : acc[i][j];
    if constexpr (OUTCLS == OUT8)  // rows of the MFMA result = n (4 consecutive n per lane)
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[buf][j], fa[buf][i], c, 0, 0, 0);
    else  // rows of the MFMA result = m, lanes run along n
      acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[buf][i], fb[buf][j], c, 0, 0, 0);
  };
  constexpr int NM = TM * TN, NR = TM + TN;
  // One k-step, pinned order: MFMA u, then RPM fragment reads of the following k-step.  The reads go
  // out in the order in which the next k-step's MFMAs (i major, j minor) first touch a fragment:
  // A0, B0 .. B(TN-1), A1 .. A(TM-1), so that every fragment has most of a k-step of MFMAs between
  // its read and its first use (an LDS read takes longer than three MFMAs to come back).
  auto kstep = [&](int buf, const char* rd_stage, int rd_ks, auto rpm_tag, auto first_tag) {
    constexpr int RPM_ = decltype(rpm_tag)::value;
    constexpr int RPM = RPM_ * NM >= NR ? RPM_ : (NR + NM - 1) / NM;
#pragma unroll
    for (int u = 0; u < NM; ++u) {
      mfma(buf, u, first_tag);
#pragma unroll
      for (int s = u * RPM; s < (u + 1) * RPM; ++s)
        if (s < NR) {
          const int r = s == 0 ? 0 : (s <= TN ? TM + s - 1 : s - TN);
          load_frag(rd_stage, rd_ks, buf ^ 1, r);
        }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using Rpm1 = std::integral_constant<int, 1>;
  using RpmLast = std::integral_constant<int, 2>;
  asm volatile("s_barrier" ::: "memory");  // k-tile 0 is in LDS
  int st = 0;
  for (int it = 0; it < count; ++it) {
    int bz, m0, n0, rank, sp, kt0, kts;
    locate(it, bz, m0, n0, rank, sp, kt0, kts);
    const EpiCtx e = make_epi(p, bz);  // scalar loads, long done when the epilogue needs them
    if (kts == 0) {  // K == 0: no MFMA defines the sums
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) load_frag(lds + st * STAGE, 0, 0, r);
    for (int kt = 0; kt < kts; ++kt) {
      const char* cur = lds + st * STAGE;
      st = (st + 1 == NSTAGE) ? 0 : st + 1;
      // k-step 0 of the tile's first k-tile starts the sums; it is the k-step before the barrier when a
      // k-tile has only two
      if (KS > 2) {
        if (kt == 0) kstep(0, cur, 1, Rpm1{}, std::true_type{});
        else kstep(0, cur, 1, Rpm1{}, std::false_type{});
      }
#pragma unroll
      for (int ks = 1; ks < KS - 2; ++ks) kstep(ks & 1, cur, ks + 1, Rpm1{}, std::false_type{});
      // the k-step before the barrier issues its reads early (two per MFMA), so that they have come
      // back when the barrier is reached
      if (KS == 2 && kt == 0) kstep(0, cur, 1, RpmLast{}, std::true_type{});
      else kstep((KS - 2) & 1, cur, KS - 1, RpmLast{}, std::false_type{});
      // every LDS read of this k-tile is issued: wait for them, then hand the stage back
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      // last k-step; the fragments it fetches are the first of the next k-tile (of the next item
      // after the last k-tile: landed as well, and simply fetched again at the item's start)
      kstep((KS - 1) & 1, lds + st * STAGE, 0, Rpm1{}, std::false_type{});
    }
    if (SPL > 1) {
      // Split K.  Each consumer wave settles its own quarter of the tile with the same wave of the
      // tile's other items, no workgroup barrier involved: it stores its sums (every instruction
      // 64 lanes x 16 consecutive bytes), waits until they are written and takes a ticket from the
      // quarter's counter.  The wave that draws the last ticket knows that all the others' sums are
      // in memory: it adds them to its own (integer sums: any order gives the same bits), puts the
      // counter back to zero for the next launch and stores the tile.  Nobody waits for anybody.
      // The sums travel with device-scope cache policy (sc1: written through to, and read from,
      // the memory side that all XCDs share), so no cache-wide write-back or invalidation is needed.
      constexpr int WAVE_BYTES = TM * TN * 16 * 64 * 4;
      constexpr int SC1 = 16;
      const __amdgpu_buffer_rsrc_t rP = __builtin_amdgcn_make_buffer_rsrc(p.sk_partial, 0, 0x7ffffff0, 0x00020000);
      const int mine = ((rank * SPL + sp) * NWC + wave) * WAVE_BYTES + lane * 16;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            __builtin_amdgcn_raw_buffer_store_b128(
                (v4u){(unsigned)acc[i][j][4 * q], (unsigned)acc[i][j][4 * q + 1], (unsigned)acc[i][j][4 * q + 2], (unsigned)acc[i][j][4 * q + 3]},
                rP, mine + ((i * TN + j) * 4 + q) * 1024, 0, SC1);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      int ticket = 0;
      if (lane == 0) ticket = atomicAdd(p.sk_counter + rank * NWC + wave, 1);
      ticket = __builtin_amdgcn_readfirstlane(ticket);
      if (ticket != SPL - 1) continue;
      for (int o = 0; o < SPL; ++o) {
        if (o == sp) continue;
        const int theirs = ((rank * SPL + o) * NWC + wave) * WAVE_BYTES + lane * 16;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rP, theirs + ((i * TN + j) * 4 + q) * 1024, 0, SC1);
              acc[i][j][4 * q] += (int)v[0]; acc[i][j][4 * q + 1] += (int)v[1];
              acc[i][j][4 * q + 2] += (int)v[2]; acc[i][j][4 * q + 3] += (int)v[3];
            }
      }
      if (lane == 0) atomicExch(p.sk_counter + rank * NWC + wave, 0);
    }
    if (wave == 0 && it == 0) TI_TL(2);
    stream_epilogue<TM, TN, OUTCLS>(p, e, acc, bz, m0 + wm * WTM, n0 + wn * WTN,
                                    lds + NSTAGE * STAGE + wave * (STRIP + COLS), lane);
    if (wave == 0 && it == 0) TI_TL(3);
  }
  if (wave == 0) TI_TL(4);
}

// ---- gather family -----------------------------------------------------------------------------
// 64x64 tile, BK = 32, 4 waves each owning one 32x32 MFMA block.  Every byte is fetched on its
// own with 64-bit addressing, so any stride pattern, alignment and K works.
template <int OUTCLS>
__global__ __launch_bounds__(256) void gemm_gather_kernel(GemmParams p) {
  constexpr int BM = 64, BN = 64, BK = 32, PITCH = BK + 16;  // 48-byte rows: 16-byte aligned, de-phased banks
  __shared__ __attribute__((aligned(16))) char sA[BM * PITCH];
  __shared__ __attribute__((aligned(16))) char sB[BN * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int tile_m, tile_n;
  tile_coords(p, blockIdx.x, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN, bz = blockIdx.y;
  const int8_t* Ab = p.A + (int64_t)bz * p.sAb;
  const int8_t* Bb = p.B + (int64_t)bz * p.sBb;
  // walk the tile so that consecutive threads touch consecutive memory when a unit stride exists
  const bool a_kfast = p.sAk == 1 || p.sAm != 1;
  const bool b_kfast = p.sBk == 1 || p.sBn != 1;

  v16i acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0;

  const int KT = (p.K + BK - 1) / BK;
  for (int kt = 0; kt < KT; ++kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int it = 0; it < BM * BK / 256; ++it) {
      const int e = it * 256 + tid;
      const int r = a_kfast ? e / BK : e % BM;
      const int k = a_kfast ? e % BK : e / BM;
      int8_t v = 0;
      if (m0 + r < p.M && k0 + k < p.K) v = Ab[(int64_t)(m0 + r) * p.sAm + (int64_t)(k0 + k) * p.sAk];
      sA[r * PITCH + k] = v;
    }
#pragma unroll
    for (int it = 0; it < BN * BK / 256; ++it) {
      const int e = it * 256 + tid;
      const int r = b_kfast ? e / BK : e % BN;
      const int k = b_kfast ? e % BK : e / BN;
      int8_t v = 0;
      if (n0 + r < p.N && k0 + k < p.K) v = Bb[(int64_t)(n0 + r) * p.sBn + (int64_t)(k0 + k) * p.sBk];
      sB[r * PITCH + k] = v;
    }
    __syncthreads();
    const v4i fa = *(const v4i*)(sA + (wm * 32 + (lane & 31)) * PITCH + (lane >> 5) * 16);
    const v4i fb = *(const v4i*)(sB + (wn * 32 + (lane & 31)) * PITCH + (lane >> 5) * 16);
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, acc, 0, 0, 0);
    __syncthreads();
  }

  const EpiCtx e = make_epi(p, bz);
  constexpr int ESZ = OUTCLS == OUT8 ? 1 : (OUTCLS == OUT32 ? 4 : 2);
  char* Cz = (char*)p.C + (int64_t)bz * p.sCb * ESZ;
  const int n = n0 + wn * 32 + (lane & 31);
  const int nc = min(n, p.N - 1);
  const float col = column_term(e, nc);
  const int bias_i32 = (e.epilogue == TI_EPI_I32 && e.bias_kind == TI_BIAS_I32) ? ((const int*)e.bias)[nc] : 0;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = m0 + wm * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
    if (m < p.M && n < p.N)
      store_one<OUTCLS>(e, Cz, (int64_t)m * p.sCm + (int64_t)n * p.sCn, acc[r], col, bias_i32, p.out_dtype);
  }
}

// ---- skinny family: M <= 64 (decode-shaped) ------------------------------------------------------
// With a handful of activation rows the GEMM is a stream over the weight matrix: every byte of B
// is read once and the matrix pipes idle.  Each wave owns a 16-row slab of B and, per 64-byte
// k-step, feeds it as the row operand of v_mfma_i32_16x16x64_i8 against up to four 16-row blocks
// of A (the 16 x 16 result block has rows = n, columns = m).  Operands go from global memory
// straight into registers in MFMA layout (lane = row + 16 * chunk); A is tiny and stays in L2.
// The 8 waves of a workgroup either take 8 different slabs (short K) or split K between them
// (each a contiguous run of k-steps, so a wave reads whole cache lines) and add their
// int32 partial sums through LDS — integer addition, so the result does not depend on the split.
template <int OUTCLS, int MBMAX, int G = 1, int UU = 0>
__global__ __launch_bounds__(512, UU ? 2 : 4) void gemm_skinny_kernel(GemmParams p) {
  constexpr int NW = 8;
  constexpr int U = UU ? UU : (MBMAX * G == 1 ? 6 : 8 / (MBMAX * G));  // k-steps per batch of loads; two batches are in flight
  __shared__ int red[NW][G * MBMAX][256];
  const int tid = threadIdx.x, lane = tid & 63;
  // The wave index must be known to be wave-uniform: the trip counts below depend on it, and a
  // branch the compiler believes divergent would wrap MFMAs in EXEC masking, which MFMAs ignore.
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ksplit = p.ksplit;
  // a wave owns a group of G consecutive 16-row slabs of B (they share the A fragments it loads)
  // and one of the ksplit contiguous runs of K
  const int group = blockIdx.x * (NW / ksplit) + wave / ksplit;
  const int kpart = wave % ksplit;
  const int bz = blockIdx.y;
  const int MB = (p.M + 15) >> 4;
  const int r16 = lane & 15, c4 = lane >> 4;
  const int8_t* Ab = p.A + (int64_t)bz * p.sAb;
  const int8_t* Bb = p.B + (int64_t)bz * p.sBb;
  const int8_t* wrow[G];
#pragma unroll
  for (int g = 0; g < G; ++g) wrow[g] = Bb + (int64_t)min((group * G + g) * 16 + r16, p.N - 1) * p.sBn + c4 * 16;
  const int8_t* xrow[MBMAX];
#pragma unroll
  for (int mb = 0; mb < MBMAX; ++mb) xrow[mb] = Ab + (int64_t)min(mb * 16 + r16, p.M - 1) * p.sAm + c4 * 16;

  v4i acc[G][MBMAX];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int mb = 0; mb < MBMAX; ++mb) acc[g][mb] = (v4i){0, 0, 0, 0};

  // The epilogue's scalars and per-column terms are fetched now, ahead of the weight stream: at the
  // end of the kernel each of them would cost a full memory round trip with nothing to overlap.
  const EpiCtx e = make_epi(p, bz);
  float col[G][4];
  int bias_i32[G][4];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = min((group * G + g) * 16 + 4 * c4 + i, p.N - 1);
      col[g][i] = column_term(e, n);
      bias_i32[g][i] = (e.epilogue == TI_EPI_I32 && e.bias_kind == TI_BIAS_I32) ? ((const int*)e.bias)[n] : 0;
    }

  // Whole 64-byte k-steps of this wave's run go in batches of U with two register sets: the loads
  // of batch b+1 are issued before the MFMAs of batch b, so a wave keeps up to 2*U*G weight loads
  // (1 KB each) in flight, and nothing in the batch loop looks at a loaded value before the MFMAs
  // do.  Left-over k-steps and a K tail (K % 64 != 0, the only place that needs zero fill) are
  // handled one at a time afterwards.  A is re-read by every group and is served by L2.
  const int KSF = p.K >> 6;  // whole k-steps
  const int per = (KSF + ksplit - 1) / ksplit;  // each wave takes a contiguous run of k-steps
  const int j0 = kpart * per;
  const int nj = min(max(KSF - j0, 0), per);
  const int nb = nj / U;
  constexpr int kstride = 64;
  v4i wf[2][U][G], xf[2][U][MBMAX];
  auto load_batch = [&](int buf, int b) {
    const int k0 = (j0 + b * U) * 64;
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int g = 0; g < G; ++g) wf[buf][u][g] = *(const v4i*)(wrow[g] + k0 + u * kstride);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mb = 0; mb < MBMAX; ++mb) xf[buf][u][mb] = *(const v4i*)(xrow[mb] + k0 + u * kstride);
  };
  auto compute = [&](int buf) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int mb = 0; mb < MBMAX; ++mb)
          acc[g][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[buf][u][g], xf[buf][u][mb], acc[g][mb], 0, 0, 0);
  };
  if (nb > 0) load_batch(0, 0);
  for (int b = 0; b < nb; b += 2) {
    if (b + 1 < nb) load_batch(1, b + 1);
    compute(0);
    if (b + 1 >= nb) break;
    if (b + 2 < nb) load_batch(0, b + 2);
    compute(1);
  }
  // left-over whole k-steps (fewer than U), then the K tail: one k-step at a time
  for (int j = nb * U; j < nj; ++j) {
    const int k0 = (j0 + j) * 64;
    v4i w1[G], x1[MBMAX];
#pragma unroll
    for (int g = 0; g < G; ++g) w1[g] = *(const v4i*)(wrow[g] + k0);
#pragma unroll
    for (int mb = 0; mb < MBMAX; ++mb) x1[mb] = *(const v4i*)(xrow[mb] + k0);
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int mb = 0; mb < MBMAX; ++mb)
        acc[g][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1[g], x1[mb], acc[g][mb], 0, 0, 0);
  }
  if ((p.K & 63) && kpart == 0) {
    const int k0 = KSF * 64;
    const bool ok = k0 + c4 * 16 < p.K;  // K is a multiple of 16: a chunk is all in or all out
    // a lane whose chunk lies past K reads the first 16 bytes of its row instead (the row pointers
    // already include the lane's chunk offset c4 * 16: without taking it back, a K below 64 would
    // put that read up to 48 bytes past the end of the row, and for the last row of the last batch
    // entry past the end of the operand)
    const int tail_off = ok ? k0 : -c4 * 16;
    v4i x1[MBMAX];
#pragma unroll
    for (int mb = 0; mb < MBMAX; ++mb) x1[mb] = *(const v4i*)(xrow[mb] + tail_off);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      v4i w1 = *(const v4i*)(wrow[g] + tail_off);
      if (!ok) w1 = (v4i){0, 0, 0, 0};
#pragma unroll
      for (int mb = 0; mb < MBMAX; ++mb)
        acc[g][mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(w1, x1[mb], acc[g][mb], 0, 0, 0);
    }
  }

  if (ksplit > 1) {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int mb = 0; mb < MBMAX; ++mb)
        if (mb < MB) *(v4i*)&red[wave][g * MBMAX + mb][lane * 4] = acc[g][mb];
    __syncthreads();
    if (kpart != 0) return;
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int mb = 0; mb < MBMAX; ++mb)
        if (mb < MB)
          for (int kp = 1; kp < ksplit; ++kp) acc[g][mb] += *(const v4i*)&red[wave + kp][g * MBMAX + mb][lane * 4];
  }

  // acc[g][mb][i]: n = (group*G + g)*16 + 4*c4 + i, m = mb*16 + r16
  constexpr int ESZ = OUTCLS == OUT8 ? 1 : (OUTCLS == OUT32 ? 4 : 2);
  char* Cz = (char*)p.C + (int64_t)bz * p.sCb * ESZ;
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = (group * G + g) * 16 + 4 * c4 + i;
      if (n >= p.N) continue;
#pragma unroll
      for (int mb = 0; mb < MBMAX; ++mb) {
        const int m = mb * 16 + r16;
        if (mb < MB && m < p.M)
          store_one<OUTCLS>(e, Cz, (int64_t)m * p.sCm + (int64_t)n * p.sCn, acc[g][mb][i], col[g][i], bias_i32[g][i],
                            p.out_dtype);
      }
    }
  }
}

// ---- decode kernel: M <= 16, weights streamed as whole 1 KB row pieces ----------------------------
//
// With 16 or fewer activation rows the GEMM is a read of the weight matrix, and what decides its
// speed is how the reads reach HBM.  Loading MFMA operands directly (16 rows x 64 bytes per
// instruction, gemm_skinny_kernel) scatters every wave's requests over 16 rows one row pitch
// apart.  Here a wave owns groups of 4 consecutive weight rows and copies them global -> LDS in
// 1 KB row pieces (one instruction = 64 lanes x 16 consecutive bytes), 3 stages of 4 x 1 KB in
// flight per wave, and the waves of the chip together sweep the matrix almost linearly.  The
// activations (16 x K bytes) are staged in LDS once per workgroup by a ninth wave, 1 KB of K at
// a time, three chunks deep, and shared by the 8 consumer waves; a barrier per chunk hands them
// over.  Operand fragments then come from LDS: rows 4..15 of the 16-row MFMA operand repeat rows
// 0..3 (their results are dropped), so no K split and no reduction between waves is needed.
// LDS row pitches: activation rows are read 16 rows x 4 chunks at a time (pitch = 4 banks mod 64: the
// 16 rows of a quarter wave hit 64 different banks); a weight job's 4 rows are read 4 rows x 4 chunks
// with every address shared by 4 lanes (pitch = 16 banks mod 64: 16 different bank groups).
// A workgroup with fewer units than waves lets only NWA of its 8 consumer waves stream, each with a
// deeper ring (NWA x NST = 24 stages of 4 x 1 KB either way): what a wave can pull is bounded by the
// bytes it keeps in flight, so 5 units on 5 waves x 3 stages leave a third of the CU's share unused.
constexpr int R4_NW = 8, R4_RG = 4, R4_KC = 1024, R4_PITCH = R4_KC + 16, R4_WPITCH = R4_KC + 64, R4_NST = 3, R4_XB = 3,
              R4_UMAX = 4;

// The store phase of gemm_rows4_kernel's epilogue: thread t of the 512 consumer threads takes row t / 32
// and the 4 outputs of unit unit0 + t % 32 from the LDS tile (row r at tile0 + (r/2) * ring + (r%2) * 2048),
// converts them and stores them as one piece, so a row's outputs leave as one contiguous run.  A
// function of its own: inlined, its operands cost the main loop registers.
template <int OUTCLS>
__device__ __attribute__((noinline)) void rows4_store_tile(const EpiCtx e, char* Cz, int64_t sCm, int64_t sCn, int M, int N,
                                                          int out_dtype, unsigned tile0, int tid, int unit0, int u_end,
                                                          int max_units, const float* resid, int64_t resid_rs, int bz,
                                                          const GemmParams* kp) {
  constexpr int ESZ = OUTCLS == OUT8 ? 1 : (OUTCLS == OUT32 ? 4 : 2);
  constexpr int RING = R4_NST * R4_RG * R4_WPITCH;  // the tile's geometry, whatever the kernel's ring depth
  const int row = tid >> 5, grp = tid & 31;
  const int unit = unit0 + grp;
  if (!(row < M && unit < u_end && grp < max_units)) return;
  const unsigned addr = tile0 + (row >> 1) * RING + (row & 1) * 2048 + grp * 16;
  const v4i a = *(const __attribute__((address_space(3))) v4i*)(uintptr_t)addr;
  const int n0 = unit * R4_RG;
  unsigned b[R4_RG];
#pragma unroll
  for (int i = 0; i < R4_RG; ++i) {
    const int n = min(n0 + i, N - 1);
    const int bias_i32 = (e.epilogue == TI_EPI_I32 && e.bias_kind == TI_BIAS_I32) ? ((const int*)e.bias)[n] : 0;
    b[i] = convert_one<OUTCLS>(e, a[i], column_term(e, n), bias_i32, out_dtype);
    if constexpr (OUTCLS == OUT32) {
      if (resid) b[i] = __float_as_uint(__uint_as_float(b[i]) + resid[(int64_t)row * resid_rs + n]);  // fp32 epilogues only (host)
    }
  }
  char* dst = Cz + ((int64_t)row * sCm + (int64_t)n0 * sCn) * ESZ;
  if constexpr (OUTCLS == OUT8) {
    if (bz > 0 && n0 + R4_RG <= N) {
      // KV-cache append of a decode step's k / v projections; the fields are read through kp, the
      // kernel's own argument block (the builtin that returns it yields null outside a kernel, so
      // the kernel passes it along)
      if (kp->kv_k) {
        const int D = kp->kv_D, head = n0 / D, d = n0 - head * D;
        if (bz == 1) {
          *(unsigned*)(kp->kv_k + (int64_t)head * kp->kv_k_hs + (int64_t)row * D + d) = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
        } else if (bz == 2) {
#pragma unroll
          for (int i = 0; i < R4_RG; ++i) kp->kv_vt[(int64_t)(n0 + i) * kp->kv_vt_rs + row] = (int8_t)b[i];
        }
      }
    }
  }
  if (sCn == 1 && n0 + R4_RG <= N && (((uintptr_t)dst) & (R4_RG * ESZ - 1)) == 0) {
    if constexpr (OUTCLS == OUT8) *(unsigned*)dst = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
    else if constexpr (OUTCLS == OUT32) *(v4u*)dst = (v4u){b[0], b[1], b[2], b[3]};
    else *(uint2*)dst = make_uint2(b[0] | (b[1] << 16), b[2] | (b[3] << 16));
  } else {
#pragma unroll
    for (int i = 0; i < R4_RG; ++i) {
      if (n0 + i < N) {
        char* d = dst + (int64_t)i * sCn * ESZ;
        if constexpr (OUTCLS == OUT8) *(int8_t*)d = (int8_t)b[i];
        else if constexpr (OUTCLS == OUT32) *(unsigned*)d = b[i];
        else *(uint16_t*)d = (uint16_t)b[i];
      }
    }
  }
}

template <int OUTCLS, int NWA, int NST>
__global__ __launch_bounds__((R4_NW + 1) * 64) void gemm_rows4_kernel(GemmParams p) {
  static_assert(NWA * NST == R4_NW * R4_NST && NWA <= R4_NW, "the rings share one LDS area");
  constexpr int STAGE = R4_RG * R4_WPITCH;  // one job: 4 rows x 1 KB (+ padding against bank conflicts)
  constexpr int XBUF = 16 * R4_PITCH;
  __shared__ __attribute__((aligned(16))) char lds[R4_XB * XBUF + R4_NW * R4_NST * STAGE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int bz = blockIdx.y;
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const int OOB = (int)0x80000000;
  const int lda = (int)p.sAm, ldb = (int)p.sBn;
  const int NCH = (p.K + R4_KC - 1) / R4_KC;  // chunks of K
  // KS = 2, 4 or 8 (only when the host asks for it): KS waves share a unit and take the chunks
  // kpart, kpart + KS, ... of K; their partial sums meet in LDS at the end.  Only with a single
  // pass.  The waves of a unit then take turns at the chunk barriers, which is why the host prefers
  // fewer streaming waves with deeper rings (NWA < 8) when a workgroup has few units.
  const int KS = NWA == R4_NW ? p.ksplit : 1;
  const int NSLOT = NWA / KS;  // units a workgroup works on at a time
  // units (groups of 4 weight rows) of this workgroup: [ub0, ub1), dealt to the slots round-robin,
  // at most NSLOT * R4_UMAX of them per pass over K
  const int NU = (p.N + R4_RG - 1) / R4_RG;
  const int per = (NU + (int)gridDim.x - 1) / (int)gridDim.x;
  const int ub0 = min(NU, (int)blockIdx.x * per), ub1 = min(NU, ub0 + per);
  const int npass = max(1, (ub1 - ub0 + NSLOT * R4_UMAX - 1) / (NSLOT * R4_UMAX));
  const int kl = lane * 16;  // this lane's byte inside a 1 KB piece

  if (wave == R4_NW) {
    // ---- activation producer: chunk g (counted over all passes) goes to buffer g % 3
    const v4i rX = make_rsrc(p.A + (int64_t)bz * p.sAb, (p.M - 1) * lda + p.K);
    const int total = npass * NCH;
    auto issue_x = [&](int g) {
      const int k0 = (g % NCH) * R4_KC;
      const bool in = g < total && k0 + kl < p.K;
      const unsigned dst = lds_base + (g % R4_XB) * XBUF;
#pragma unroll
      for (int m = 0; m < 16; ++m)
        dma16_to_lds(rX, in ? min(m, p.M - 1) * lda + kl : OOB, k0, dst + m * R4_PITCH);
    };
    issue_x(0);
    issue_x(1);
    int left = NCH;  // chunks until the end of the pass
    for (int g = 0; g < total; ++g) {
      wait_loads_and_barrier<16>();  // chunk g has landed (chunk g+1 may be in flight); hand it over
      issue_x(g + 2);                // into the buffer of chunk g-1, whose readers passed the barrier
      if (--left == 0) {
        // end of a pass: the consumers' reduction barrier (K split) and the two of their epilogue
        left = NCH;
        if (KS > 1) asm volatile("s_barrier" ::: "memory");
        asm volatile("s_barrier\n\ts_barrier" ::: "memory");
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }

  // ---- consumers
  // waves NWA..7 (kpart >= KS): no units, barriers only
  const int slot = NWA == R4_NW ? wave % NSLOT : wave, kpart = NWA == R4_NW ? wave / NSLOT : (wave >= NWA ? 1 : 0);
  const v4i rW = make_rsrc(p.B + (int64_t)bz * p.sBb, (p.N - 1) * ldb + p.K);
  const int ring_i = wave < NWA ? wave : 0;
  const unsigned ring = lds_base + R4_XB * XBUF + ring_i * (NST * STAGE);
  char* ring_p = lds + R4_XB * XBUF + ring_i * (NST * STAGE);
  const int r16 = lane & 15, c4 = lane >> 4;
  const int w_lane = (r16 & (R4_RG - 1)) * R4_WPITCH + c4 * 16;  // rows 4..15 of the operand repeat rows 0..3
  const int x_lane = r16 * R4_PITCH + c4 * 16;
  const EpiCtx e = make_epi(p, bz);
  constexpr int ESZ = OUTCLS == OUT8 ? 1 : (OUTCLS == OUT32 ? 4 : 2);
  char* Cz = (char*)p.C + (int64_t)bz * p.sCb * ESZ;
  const int nch_mine = (NCH - kpart + KS - 1) / KS;  // chunks kpart, kpart + KS, ...

  int g = 0;  // chunk counter over all passes (selects the activation buffer)
  for (int pass = 0; pass < npass; ++pass) {
    const int u_first = ub0 + pass * (NSLOT * R4_UMAX) + slot;  // this wave's units: u_first + NSLOT*i, i < nu
    const int u_end = min(ub1, ub0 + (pass + 1) * (NSLOT * R4_UMAX));
    const int nu = (u_first < u_end && wave < NWA) ? (u_end - u_first + NSLOT - 1) / NSLOT : 0;
    const int njobs = nu * nch_mine;
    // job j = (this wave's chunk number j / nu, unit j % nu): 4 loads of 1 KB, into ring slot j % NST;
    // beyond the last job the loads are redirected out of range (zeros into a slot nobody reads)
    // so that the number in flight stays constant
    auto issue_job = [&](int j) {
      const bool real = j < njobs;
      const int cm = real ? j / nu : 0, ui = real ? j - cm * nu : 0;
      // uniform; says so to the compiler (the load helper keeps the wait states a VMEM read of this
      // VALU-written register needs)
      const int k0 = __builtin_amdgcn_readfirstlane((kpart + cm * KS) * R4_KC);
      const int row0 = (u_first + ui * NSLOT) * R4_RG;
      const bool in = real && k0 + kl < p.K;
      const unsigned dst = ring + (j % NST) * STAGE;
#pragma unroll
      for (int r = 0; r < R4_RG; ++r)
        dma16_to_lds_stream(rW, in ? min(row0 + r, p.N - 1) * ldb + kl : OOB, k0, dst + r * R4_WPITCH);
    };
    v4i acc[R4_UMAX];
#pragma unroll
    for (int i = 0; i < R4_UMAX; ++i) acc[i] = (v4i){0, 0, 0, 0};
    if (nu > 0) {
#pragma unroll
      for (int i = 0; i < NST - 1; ++i) issue_job(i);
    }
    int j = 0;
    for (int c = 0; c < NCH; ++c, ++g) {
      asm volatile("s_barrier" ::: "memory");  // activation chunk g is in LDS
      if (nu == 0 || c % KS != kpart) continue;
      // the chunk's 16 activation fragments are read once and serve all of the wave's units
      // (bytes past K were loaded as zeros, so all 16 k-steps can always be used)
      const char* xb = lds + (g % R4_XB) * XBUF + x_lane;
      v4i xf[16];
#pragma unroll
      for (int s = 0; s < 16; ++s) xf[s] = *(const v4i*)(xb + s * 64);
#pragma unroll
      for (int ui = 0; ui < R4_UMAX; ++ui) {
        if (ui < nu) {
          issue_job(j + NST - 1);
          asm volatile("s_waitcnt vmcnt(%0)" ::"n"(R4_RG * (NST - 1)) : "memory");  // job j has landed
          const char* wb = ring_p + (j % NST) * STAGE + w_lane;
#pragma unroll
          for (int s = 0; s < 16; ++s)
            acc[ui] = __builtin_amdgcn_mfma_i32_16x16x64_i8(*(const v4i*)(wb + s * 64), xf[s], acc[ui], 0, 0, 0);
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // slot j % NST is free for job j + NST
          ++j;
        }
      }
    }
    if (nu > 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // trailing redirected loads
    if (KS > 1) {
      // the waves of the later chunks park their sums in their own (now idle) rings; the wave of the
      // first chunks adds them
      if (kpart > 0) {
#pragma unroll
        for (int ui = 0; ui < R4_UMAX; ++ui)
          if (ui < nu) *(v4i*)(ring_p + ui * 1024 + lane * 16) = acc[ui];
      }
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if (kpart == 0) {
        for (int kp = 1; kp < KS; ++kp) {
          const char* other = ring_p + kp * NSLOT * (NST * STAGE);
#pragma unroll
          for (int ui = 0; ui < R4_UMAX; ++ui)
            if (ui < nu) acc[ui] += *(const v4i*)(other + ui * 1024 + lane * 16);
        }
      }
    }
    // ---- epilogue.  acc[ui][i], lanes 0..15: n = unit*4 + i, m = lane.  The workgroup's units of a pass
    // are consecutive, so its outputs are 16 rows x (4 x units) consecutive columns: the sums go to
    // an LDS tile (row r in the third ring slot of wave r/2, which no load touches before the next
    // pass's first chunk barrier) and leave as whole row pieces, 4 elements per thread, instead of
    // single elements scattered over 16 rows (20480 x 5120: 2.5 us of a 22.5 us launch).  Every load
    // of every wave has landed before the tile is written (first barrier); the second publishes it.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    auto tile_row = [&](int r) -> char* { return lds + R4_XB * XBUF + (r >> 1) * (R4_NST * STAGE) + 2 * STAGE + (r & 1) * 2048; };
    if (kpart == 0 && c4 == 0) {
#pragma unroll
      for (int ui = 0; ui < R4_UMAX; ++ui)
        if (ui < nu) *(v4i*)(tile_row(r16) + (slot + ui * NSLOT) * 16) = acc[ui];
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    rows4_store_tile<OUTCLS>(e, Cz, p.sCm, p.sCn, p.M, p.N, p.out_dtype, lds_base + R4_XB * XBUF + 2 * STAGE, tid,
                             ub0 + pass * (NSLOT * R4_UMAX), u_end, NSLOT * R4_UMAX, p.resid, p.resid_rs, bz,
                             (const GemmParams*)__builtin_amdgcn_kernarg_segment_ptr());
  }
}

// ---- host side ---------------------------------------------------------------------------------

typedef void (*KernelFn)(GemmParams);

struct Config {
  const char* name;
  KernelFn fn[3];  // by OutClass
  int bm, bn, bk, threads;
  bool fast;       // needs the aligned K-contiguous layout
  bool skinny = false;  // gemm_skinny_kernel: M <= 64, grid over 16-row slabs of B
  int stream_occ = 0;   // > 0: gemm_mfma_stream_kernel, this many workgroups per CU walk the tile list
  bool rows4 = false;   // gemm_rows4_kernel: M <= 16
  int ws_waves = 0;     // > 0: gemm_mfma_ws_kernel with this many consumer waves (it can split K)
  int max_k = 0;        // > 0: the kernel holds a tile's whole K in LDS and takes 16 <= K <= max_k only
};

#define TI_FAST(BM, BN, BK, WM, WN, SWZ, NS)                                              \
  {                                                                                       \
    "mfma_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_s" #SWZ "_p" #NS,                        \
        {gemm_mfma_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT8>,                               \
         gemm_mfma_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT32>,                              \
         gemm_mfma_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT16>},                             \
        BM, BN, BK, WM * WN * 64, true                                                    \
  }

#define TI_STREAM(BM, BN, BK, WM, WN, SWZ, NS, OCC)                                        \
  {                                                                                       \
    "stream_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_s" #SWZ "_p" #NS "_o" #OCC,            \
        {gemm_mfma_stream_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT8, OCC>,                   \
         gemm_mfma_stream_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT32, OCC>,                  \
         gemm_mfma_stream_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT16, OCC>},                 \
        BM, BN, BK, WM * WN * 64, true, false, OCC                                        \
  }

#define TI_WS(BM, BN, BK, WM, WN, SWZ, NS, PW)                                            \
  {                                                                                       \
    "ws_" #BM "x" #BN "x" #BK "_w" #WM "x" #WN "_s" #SWZ "_p" #NS "_l" #PW,                 \
        {gemm_mfma_ws_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT8, PW>,                        \
         gemm_mfma_ws_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT32, PW>,                       \
         gemm_mfma_ws_kernel<BM, BN, BK, WM, WN, SWZ, NS, OUT16, PW>},                      \
        BM, BN, BK, (WM * WN + PW) * 64, true, false, 1, false, WM * WN                   \
  }

enum ConfigId {
  CFG_GATHER = 0,
  CFG_TILE_256x128,   // one tile per workgroup: any output layout the fast loads allow
  CFG_TILE_256x256,
  CFG_TILE_128x128,
  CFG_TILE_64x64,
  CFG_SKINNY_16,
  CFG_SKINNY_32,
  CFG_SKINNY_64,
  CFG_STREAM_256x256,       // persistent: row-major, 16-byte aligned outputs
  CFG_WS_256x128,           // persistent, loads issued by dedicated producer waves
  CFG_STREAM_128x128,
  CFG_SKINNY_16_G2,  // M <= 16, a wave owns 2 slabs that share its A fragments
  CFG_ROWS4_16,      // M <= 16, K >= 1024: weights streamed as 1 KB row pieces
  CFG_WS_256x160,    // 2048 x 5120 outputs are exactly 256 of these tiles: one full round of the chip
  CFG_WS_128x128,    // few activation rows and a long K: split K over enough of these to fill the chip
  CFG_SHORTK_256x256,  // K <= 128 (attention Q.K^T): a tile's whole K in LDS, one barrier per tile, 128-byte int8 row pieces
  CFG_WS_64x128,       // 32 < M <= 128 against a long K: six stages of a 64-row tile keep more weight bytes in flight per CU
  CFG_WS_32x128,       // 16 < M <= 32: seven stages
};

static const Config g_configs[] = {
    {"gather_64x64x32", {gemm_gather_kernel<OUT8>, gemm_gather_kernel<OUT32>, gemm_gather_kernel<OUT16>}, 64, 64, 32, 256, false},
    TI_FAST(256, 128, 128, 2, 2, 1, 3),
    TI_FAST(256, 256, 64, 2, 4, 2, 4),
    TI_FAST(128, 128, 64, 2, 2, 2, 4),
    TI_FAST(64, 64, 128, 2, 2, 1, 3),
    {"skinny_m16_slab16", {gemm_skinny_kernel<OUT8, 1>, gemm_skinny_kernel<OUT32, 1>, gemm_skinny_kernel<OUT16, 1>}, 16, 16, 64, 512, true, true},
    {"skinny_m32_slab16", {gemm_skinny_kernel<OUT8, 2>, gemm_skinny_kernel<OUT32, 2>, gemm_skinny_kernel<OUT16, 2>}, 32, 16, 64, 512, true, true},
    {"skinny_m64_slab16", {gemm_skinny_kernel<OUT8, 4>, gemm_skinny_kernel<OUT32, 4>, gemm_skinny_kernel<OUT16, 4>}, 64, 16, 64, 512, true, true},
    TI_STREAM(256, 256, 64, 2, 4, 2, 4, 1),
    TI_WS(256, 128, 128, 2, 2, 1, 3, 4),
    TI_STREAM(128, 128, 64, 2, 2, 2, 3, 2),
    {"skinny_m16_slab32", {gemm_skinny_kernel<OUT8, 1, 2>, gemm_skinny_kernel<OUT32, 1, 2>, gemm_skinny_kernel<OUT16, 1, 2>}, 16, 32, 64, 512, true, true},
    {"rows4_m16", {gemm_rows4_kernel<OUT8, 8, 3>, gemm_rows4_kernel<OUT32, 8, 3>, gemm_rows4_kernel<OUT16, 8, 3>}, 16, 4, 1024, (R4_NW + 1) * 64, true, false, 0, true},
    TI_WS(256, 160, 128, 4, 1, 1, 3, 4),
    TI_WS(128, 128, 128, 2, 2, 1, 4, 4),
    {"shortk_256x256x64_w4x2_k128", {gemm_mfma_shortk_kernel<OUT8>, gemm_mfma_shortk_kernel<OUT32>, gemm_mfma_shortk_kernel<OUT16>}, 256, 256, 64, 512,
     true, false, 1, false, 0, 128},
    TI_WS(64, 128, 128, 2, 2, 1, 6, 4),
    TI_WS(32, 128, 128, 1, 4, 1, 7, 4),
};
static const int g_num_configs = (int)(sizeof(g_configs) / sizeof(g_configs[0]));

static int out_class(int out_dtype) {
  switch (out_dtype) {
    case TI_I8: return OUT8;
    case TI_I32:
    case TI_F32: return OUT32;
    default: return OUT16;
  }
}

static bool fast_eligible(const GemmParams& p) {
  if (p.sAk != 1 || p.sBk != 1) return false;
  if (p.K <= 0 || (p.K & 15)) return false;
  if ((p.sAm & 15) || (p.sBn & 15) || (p.sAb & 15) || (p.sBb & 15)) return false;
  if (((uintptr_t)p.A & 15) || ((uintptr_t)p.B & 15)) return false;
  if (p.sAm < p.K || p.sBn < p.K) return false;
  if (out_class(p.out_dtype) == OUT8 && p.sCn != 1) return false;
  // 32-bit byte offsets inside one batch slice, including the rows a ragged last tile touches
  const int64_t lim = (int64_t)1 << 31;
  if (((int64_t)p.M + 512) * p.sAm + p.K >= lim) return false;
  if (((int64_t)p.N + 512) * p.sBn + p.K >= lim) return false;
  return true;
}

// The stream kernels store through range-checked buffer descriptors with 32-bit offsets and, for
// int8, whole 16-byte segments only.
static bool stream_eligible(const GemmParams& p) {
  if (!fast_eligible(p)) return false;
  if (p.sCn != 1 || p.sCm < p.N || p.sCb < 0) return false;
  const int oc = out_class(p.out_dtype);
  const int esz = oc == OUT8 ? 1 : (oc == OUT32 ? 4 : 2);
  // 32-bit store offsets, including those of the rows a ragged last tile computes past M before the
  // range check drops them: (first row of the tile + row inside it) * pitch must not wrap back into range
  if (((int64_t)(p.M + 512) * p.sCm + p.N) * esz >= ((int64_t)1 << 31)) return false;
  if ((uintptr_t)p.C % esz) return false;
  if (oc == OUT8 && ((p.N & 15) || (p.sCm & 15) || (p.sCb & 15) || ((uintptr_t)p.C & 15))) return false;
  return true;
}

// k-tiles per split and the number of non-empty splits for `want` splits of a K of `kt` k-tiles
static void sk_shape(int kt, int want, int& splits, int& kt_split) {
  want = want < 1 ? 1 : (want > kt ? (kt > 0 ? kt : 1) : want);
  kt_split = (kt + want - 1) / want;
  splits = kt_split > 0 ? (kt + kt_split - 1) / kt_split : 1;
}

// Estimated run time (arbitrary unit) of the GEMM on configuration k with `want` K splits:
//   rounds of work items over the chip's workgroup slots
//   x the K bytes an item walks, plus a fixed part per item (pipeline fill, epilogue and store: about
//     four k-tiles' worth) and, when K is split, the exchange of partial sums (the store of an
//     item's sums plus, for the last item of a tile, one read per other split: measured about
//     1 + 2.6 us per split for a 256 x 128 tile, i.e. four plus six k-tiles' worth per split)
//   x the tile's outputs / the measured relative efficiency of the tile class (per slot)
// with a small bonus for few rounds (a chip that is partly idle in its only round runs that round
// faster than a full chip runs the first of two).  Padded parts of edge tiles cost like real ones.
static double config_cost(const GemmParams& p, const Config& k, double eff, int want, int& splits) {
  const int occ = k.stream_occ > 1 ? k.stream_occ : 1;
  const int slots = 256 * occ;
  const int64_t tm = (p.M + k.bm - 1) / k.bm, tn = (p.N + k.bn - 1) / k.bn;
  const int kt = (p.K + k.bk - 1) / k.bk;
  int kt_split = kt;
  splits = 1;
  if (want > 1 && k.ws_waves && p.batch == 1) sk_shape(kt, want, splits, kt_split);
  const int64_t items = tm * tn * p.batch * splits;
  const int64_t rounds = (items + slots - 1) / slots;
  // a last round that fills only part of the chip runs faster than a full one (the busy CUs share the
  // power and the memory system of the idle ones): 2.5 rounds of 256 x 128 tiles measure like 2.7-2.8
  const double idle = 1.0 - (double)(items - (rounds - 1) * slots) / (double)slots;
  const double rounds_eff = (double)rounds - (rounds > 1 ? 0.4 : 0.2) * idle;
  const double k_len = (double)kt_split * k.bk + 512.0 + (splits > 1 ? 512.0 + 768.0 * splits : 0.0);
  return rounds_eff * k_len * (double)(k.bm * k.bn) * occ / eff / (1.0 + 0.1 / (double)rounds);
}

// Number of K splits for a wave-specialised configuration: as many as fill the chip's 256 workgroup
// slots once, but no split shorter than 2560 bytes of K (K = 4096 is faster whole, K = 5120 in two
// parts) and no more than 8 (the last item of a tile reads the other splits' sums one after the other).
static int pick_splits(const GemmParams& p, const Config& k, double eff, double* cost_out) {
  int want = 1;
  if (k.ws_waves && p.batch == 1) {
    const int64_t tiles = (int64_t)((p.M + k.bm - 1) / k.bm) * ((p.N + k.bn - 1) / k.bn);
    const int64_t fill = tiles > 0 ? 256 / tiles : 1;
    const int by_k = p.K / 2560;
    want = (int)(fill < by_k ? fill : by_k);
    want = want < 1 ? 1 : (want > 8 ? 8 : want);
  }
  int used = 1;
  double cost = config_cost(p, k, eff, want, used);
  if (used > 1) {  // whole K may still be the cheaper of the two
    int one = 1;
    const double whole = config_cost(p, k, eff, 1, one);
    if (whole <= cost) cost = whole, used = 1;
  }
  if (cost_out) *cost_out = cost;
  return used;
}

// Tile choice: the configuration (and K split) with the lowest estimated run time.  The class
// efficiencies were measured with weights streamed from HBM.  Outputs the persistent kernels can
// store (row-major, aligned) go to them; the rest to the one-tile kernels.
static int pick_config(const GemmParams& p, int* splits_out) {
  *splits_out = 1;
  if (!fast_eligible(p)) return CFG_GATHER;
  if (p.M <= 16) {
    // one GEMM over a long K: stream the weights as whole row pieces; short K or batched (the
    // decode attention BMMs): MFMA-layout loads, two slabs per wave while enough waves remain
    if (p.batch <= 4 && p.K >= 1024) return CFG_ROWS4_16;
    return (p.N + 31) / 32 >= 160 ? CFG_SKINNY_16_G2 : CFG_SKINNY_16;
  }
  const bool stream = stream_eligible(p);
  if (p.M <= 128 && stream && p.batch == 1 && p.K >= 1024) {
    // a few rows against a long K: the GEMM is a read of the weight matrix, and what decides its speed is how
    // many weight bytes a CU keeps in flight.  K is split over enough workgroups to have every CU pulling its
    // own slab, and the tile has no more activation rows than needed, so that the LDS holds more stages of
    // weights: 32 x 128 tiles with 7 stages up to 32 rows, 64 x 128 with 6 stages beyond (a 128 x 128 tile has
    // room for 4).  Measured in steady state, weights rotated through 350 MB, N = 6848, K = 10240, against
    // the 128 x 128 tile: M = 17 .. 32 34 -> 22-23 us, M = 64 35 -> 28.5 us, M = 128 38 -> 33 us; N = K = 5120:
    // 18.5-19 -> 15-16 us, M = 128 20.4 -> 16.6 us.
    const int cfg = p.M <= 32 ? CFG_WS_32x128 : CFG_WS_64x128;
    *splits_out = pick_splits(p, g_configs[cfg], 1.0, nullptr);
    return cfg;
  }
  if (p.M <= 64) return CFG_SKINNY_16 + (p.M > 16) + (p.M > 32);
  // K <= 128, int8 out, at least two 256 x 256 tiles per workgroup: the epilogue is most of the work
  // (and tiles that are mostly output, not padding)
  if (stream && p.K >= 16 && p.K <= g_configs[CFG_SHORTK_256x256].max_k && out_class(p.out_dtype) == OUT8 &&
      (!p.bias || p.bias_kind == TI_BIAS_NONE) && p.epilogue != TI_EPI_GELU_I8) {
    const int64_t tm = (p.M + 255) / 256, tn = (p.N + 255) / 256;
    if (tm * tn * p.batch >= 512 && (double)p.M * p.N >= 0.6 * (double)(tm * 256) * (double)(tn * 256)) return CFG_SHORTK_256x256;
  }
  // short K: the epilogue dominates and the larger tile halves the operand traffic per output
  const double big = p.K <= 512 ? 1.20 : 0.92;
  // 256 x 160 tiles: as good as 256 x 128 per unit of work with 2- and 4-byte outputs; with int8 outputs
  // the tile has no LDS room left for the epilogue's row strip and stores 32-byte pieces (measured per
  // output column, 2048 x 5120 x 5120: 0.32 us against 0.27 us).  Still the choice where it saves a
  // round: 2048 x 5120 outputs are one round of 256 such tiles (56 us against 74 us), 2048 x 20480 take
  // four rounds of them or five of the narrower tile (199 us against 182 us)
  const double wide160 = out_class(p.out_dtype) == OUT8 ? 0.80 : 1.00;
  struct Cand { int cfg; double eff; };
  const Cand cands[] = {
      {stream ? CFG_STREAM_256x256 : CFG_TILE_256x256, stream ? big : 1.00},
      {stream ? CFG_WS_256x128 : CFG_TILE_256x128, stream ? 1.00 : 0.90},
      {stream ? CFG_STREAM_128x128 : CFG_TILE_128x128, stream ? 0.70 : 0.78},
      {CFG_TILE_64x64, 0.25},
      {stream ? CFG_WS_256x160 : -1, wide160},
      {stream ? CFG_WS_128x128 : -1, 0.80},
  };
  int best = CFG_TILE_64x64;
  double best_cost = -1.0;
  for (const Cand& c : cands) {
    if (c.cfg < 0) continue;
    double cost;
    const int splits = pick_splits(p, g_configs[c.cfg], c.eff, &cost);
    if (best_cost < 0 || cost < best_cost) best_cost = cost, best = c.cfg, *splits_out = splits;
  }
  return best;
}

// gemm_rows4_kernel with nwa of its 8 consumer waves streaming (24 / nwa ring stages each)
static KernelFn rows4_kernel(int oc, int nwa) {
  static const KernelFn fns[3][3] = {
      {gemm_rows4_kernel<OUT8, 8, 3>, gemm_rows4_kernel<OUT32, 8, 3>, gemm_rows4_kernel<OUT16, 8, 3>},
      {gemm_rows4_kernel<OUT8, 6, 4>, gemm_rows4_kernel<OUT32, 6, 4>, gemm_rows4_kernel<OUT16, 6, 4>},
      {gemm_rows4_kernel<OUT8, 4, 6>, gemm_rows4_kernel<OUT32, 4, 6>, gemm_rows4_kernel<OUT16, 4, 6>},
  };
  return fns[nwa == 6 ? 1 : (nwa == 4 ? 2 : 0)][oc];
}

static int pick_group_m(const GemmParams& p, const Config& k) {
  // Each XCD is dealt tiles/8 consecutive tiles and has 32 CUs: the tiles it runs at the same
  // time share its L2, so that set should touch as few operand rows as possible (roughly square).
  const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
  const int at_once = 32 * (k.stream_occ > 1 ? k.stream_occ : 1);
  const int per_xcd = (int)((tiles + 7) / 8) < at_once ? (int)((tiles + 7) / 8) : at_once;
  int best = 1;
  int64_t best_cost = -1;
  // powers of two, and all of a short column of row tiles (3 or 6 row tiles in groups of 2 or 4
  // would send the odd ones through the weight panels a second time)
  for (int g = 1; g <= p.tiles_m && g <= 64; g = (g * 2 > p.tiles_m && g < p.tiles_m && p.tiles_m <= 64) ? p.tiles_m : g * 2) {
    const int cols = (per_xcd + g - 1) / g;
    const int passes = (p.tiles_m + g - 1) / g;  // a short last group still walks all weight panels
    const int64_t cost = ((int64_t)g * k.bm + (int64_t)cols * k.bn) * passes * g / p.tiles_m;
    if (best_cost < 0 || cost < best_cost) best_cost = cost, best = g;
  }
  return best;
}

static int validate(const GemmParams& p) {
  if (p.batch < 0 || p.M < 0 || p.N < 0 || p.K < 0) return fail(TI_E_SHAPE, "negative size");
  if (p.batch == 0 || p.M == 0 || p.N == 0) return TI_OK;
  if (!p.A && p.K > 0) return fail(TI_E_NULL, "A is NULL");
  if (!p.B && p.K > 0) return fail(TI_E_NULL, "B is NULL");
  if (!p.C) return fail(TI_E_NULL, "C is NULL");
  if (p.batch > 65535) return fail(TI_E_SHAPE, "batch %d > 65535", p.batch);
  const int bk = p.bias ? p.bias_kind : TI_BIAS_NONE;
  bool ok = false;
  switch (p.epilogue) {
    case TI_EPI_I32: ok = p.out_dtype == TI_I32 && (bk == TI_BIAS_NONE || bk == TI_BIAS_I32); break;
    case TI_EPI_SCALE_I32: ok = p.out_dtype == TI_I32 && (bk == TI_BIAS_NONE || bk == TI_BIAS_I32); break;
    case TI_EPI_SCALE_I8:
    case TI_EPI_SCALE_RELU_I8: ok = p.out_dtype == TI_I8 && (bk == TI_BIAS_NONE || bk == TI_BIAS_I8); break;
    case TI_EPI_SCALE_F:
      ok = (p.out_dtype == TI_F32 || p.out_dtype == TI_F16 || p.out_dtype == TI_BF16) &&
           (bk == TI_BIAS_NONE || bk == TI_BIAS_F32 || bk == TI_BIAS_F16 || bk == TI_BIAS_BF16);
      break;
    case TI_EPI_GELU_I8: ok = p.out_dtype == TI_I8 && (bk == TI_BIAS_NONE || bk == TI_BIAS_F32); break;
    default: break;
  }
  if (!ok) return fail(TI_E_COMBO, "epilogue %d / out dtype %d / bias kind %d is not a defined combination", p.epilogue, p.out_dtype, bk);
  if (p.epilogue != TI_EPI_I32 && !p.alpha) return fail(TI_E_NULL, "alpha is NULL");
  if (bk != TI_BIAS_NONE && p.epilogue != TI_EPI_I32 && !p.beta) return fail(TI_E_NULL, "beta is NULL");
  if (p.epilogue == TI_EPI_GELU_I8 && !p.beta) return fail(TI_E_NULL, "beta (output scale) is NULL");
  if (p.round_mode != TI_ROUND_RNE_CLAMP && p.round_mode != TI_ROUND_TRUNC) return fail(TI_E_COMBO, "round mode %d", p.round_mode);
  if (p.sCm == 0 && p.M > 1) return fail(TI_E_STRIDE, "output row stride is 0");
  if (p.sCn == 0 && p.N > 1) return fail(TI_E_STRIDE, "output column stride is 0");
  return TI_OK;
}

static thread_local int g_last_config = -1;
static thread_local int g_last_splits = 1;

// ---- split-K workspace -----------------------------------------------------------------------------
// One allocation per (device, stream): ticket counters (zeroed once; every launch leaves them at
// zero) followed by the items' int32 partial sums.  Launches on one stream run one after the other,
// so they can share it; launches on different streams may overlap and get their own.  It grows on
// demand.
constexpr size_t SK_COUNTER_INTS = 1 << 16;             // tiles x consumer waves of one launch
constexpr size_t SK_MAX_PARTIAL_BYTES = (size_t)96 << 20;  // < 2 GiB: the kernel addresses it with 32-bit offsets
struct SkWorkspace { int dev; hipStream_t stream; char* base; size_t partial_bytes; std::vector<char*> outgrown; };
static std::mutex g_sk_mutex;
static std::vector<SkWorkspace> g_sk_ws;

__global__ __launch_bounds__(256) void sk_clear_counters_kernel(int* counters, int n) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) counters[i] = 0;
}

// 0 and the pointers, or a status.  With allocate == false (the stream is being captured into a
// graph: no allocation possible) an existing workspace that is large enough is used, else TI_E_COMBO.
static int sk_workspace(hipStream_t stream, size_t partial_bytes, bool allocate, int** partial, int** counter) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail((int)err, "hipGetDevice: %s", hipGetErrorString(err));
  std::lock_guard<std::mutex> lock(g_sk_mutex);
  SkWorkspace* w = nullptr;
  for (auto& e : g_sk_ws)
    if (e.dev == dev && e.stream == stream) w = &e;
  if (!w || w->partial_bytes < partial_bytes) {
    if (!allocate) return TI_E_COMBO;
    if (w && partial_bytes < 2 * w->partial_bytes) partial_bytes = 2 * w->partial_bytes;
    if (partial_bytes > SK_MAX_PARTIAL_BYTES) partial_bytes = SK_MAX_PARTIAL_BYTES;
    char* base = nullptr;
    const size_t bytes = SK_COUNTER_INTS * sizeof(int) + partial_bytes;
    err = hipMalloc((void**)&base, bytes);
    if (err != hipSuccess) return fail((int)err, "split-K workspace of %zu bytes: %s", bytes, hipGetErrorString(err));
    // cleared on the launch stream, so that the clear is ordered before the launch on any kind of stream
    // (a memset on the null stream is not ordered against a non-blocking stream)
    sk_clear_counters_kernel<<<dim3(64), dim3(256), 0, stream>>>((int*)base, (int)SK_COUNTER_INTS);
    const int rc = launch_status("sk_clear_counters_kernel");
    if (rc != TI_OK) {
      (void)hipFree(base);
      return rc;
    }
    if (!w) {
      g_sk_ws.push_back({dev, stream, nullptr, 0, {}});
      w = &g_sk_ws.back();
    }
    // The outgrown block is kept until the workspace is released: earlier launches on the stream, or a
    // captured graph, may still use it.  Growing at least doubles the size, so the blocks kept sum to
    // less than the current one.
    if (w->base) w->outgrown.push_back(w->base);
    w->base = base;
    w->partial_bytes = partial_bytes;
  }
  *counter = (int*)w->base;
  *partial = (int*)(w->base + SK_COUNTER_INTS * sizeof(int));
  return TI_OK;
}

// Frees the current device's workspace of `stream` (all streams' when all != 0), outgrown blocks
// included, after the stream's queued work has finished.  For callers that create streams per request:
// without it every stream that ever ran a split-K launch keeps its blocks for the life of the process.
// The caller must not replay a graph that captured a split-K launch on that stream afterwards.
static int sk_release(hipStream_t stream, bool all, int64_t* freed_bytes) {
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail((int)err, "hipGetDevice: %s", hipGetErrorString(err));
  std::vector<SkWorkspace> mine;
  {
    std::lock_guard<std::mutex> lock(g_sk_mutex);
    for (size_t i = 0; i < g_sk_ws.size();) {
      if (g_sk_ws[i].dev == dev && (all || g_sk_ws[i].stream == stream)) {
        mine.push_back(g_sk_ws[i]);
        g_sk_ws[i] = g_sk_ws.back();
        g_sk_ws.pop_back();
      } else {
        ++i;
      }
    }
  }
  int64_t freed = 0;
  int rc = TI_OK;
  for (auto& w : mine) {
    err = hipStreamSynchronize(w.stream);  // the launches that use the blocks
    if (err != hipSuccess && rc == TI_OK) rc = fail((int)err, "hipStreamSynchronize: %s", hipGetErrorString(err));
    if (w.base) {
      (void)hipFree(w.base);
      freed += (int64_t)(SK_COUNTER_INTS * sizeof(int) + w.partial_bytes);
    }
    for (char* b : w.outgrown) (void)hipFree(b);
  }
  if (freed_bytes) *freed_bytes = freed;
  return rc;
}

// ---- split-K scratch that needs no allocation ---------------------------------------------------------
// For callers that cannot allocate (a stream under graph capture, a serving loop that forbids it):
// the same layout as the allocated workspace, ticket counters followed by partial sums, in a
// file-scope device array of fixed size.  Every GPU the library runs on holds its own copy for the
// life of the process.  Host code never uses the array's name as an address: its device address
// is looked up once per device, with that device current, and that pointer is what kernels get.
constexpr size_t SK_STATIC_COUNTER_INTS = 1 << 14;            // tiles x consumer waves of one launch
constexpr size_t SK_STATIC_PARTIAL_BYTES = (size_t)32 << 20;  // 256 work items of a 256 x 128 tile
constexpr size_t SK_STATIC_INTS = SK_STATIC_COUNTER_INTS + SK_STATIC_PARTIAL_BYTES / sizeof(int);
static __device__ __align__(256) int scratch[SK_STATIC_INTS];
static int* g_scratch_ptr[64];

// Device address of the calling thread's current device's copy of `scratch`.  First call on a
// device: looks the address up.  The ticket counters need no clearing: a file-scope device array is
// zero-initialised when the code object is loaded, and every launch leaves them at zero; so the call
// enqueues nothing but the GEMM itself (a first call under graph capture records no extra node).
static int sk_static_scratch(hipStream_t stream, int** partial, int** counter) {
  (void)stream;
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail((int)err, "hipGetDevice: %s", hipGetErrorString(err));
  if (dev < 0 || dev >= 64) return fail(TI_E_DEVICE, "device index %d beyond the %d the static scratch table covers", dev, 64);
  std::lock_guard<std::mutex> lock(g_sk_mutex);
  if (!g_scratch_ptr[dev]) {
    int* ptr = nullptr;
    err = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr) return fail(err != hipSuccess ? (int)err : TI_E_NULL, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(err));
    g_scratch_ptr[dev] = ptr;
  }
  *counter = g_scratch_ptr[dev];
  *partial = g_scratch_ptr[dev] + SK_STATIC_COUNTER_INTS;
  return TI_OK;
}

// What run() launches for a problem: filled instead of launching when run() is given one (ti_gemm_plan).
struct LaunchPlan {
  int config = -1, splits = 1, kt_split = 0, tiles_m = 0, tiles_n = 0, group_m = 1;
  unsigned grid_x = 0, grid_y = 0;
  int threads = 0, ksplit = 1, nwa = 0;
  int64_t partial_bytes = 0;  // split-K partial sums the launch needs
};

// `config`: bits 0..7 the configuration (0xff or a negative value: choose), bits 8..15 the number of
// K splits to use with a wave-specialised configuration (0: choose).
// static_scratch: split-K launches use the fixed device array instead of the allocated workspace, and a
// launch whose partial sums do not fit it is refused (nothing is allocated or freed on this path).
// dry: every decision is taken as for a launch (same code), but no device is touched, nothing is
// allocated or launched, and *dry receives the launch's configuration and grid.
static int run(GemmParams p, int config, hipStream_t stream, bool static_scratch = false, LaunchPlan* dry = nullptr) {
  g_last_splits = 1;
  int want_splits = config < 0 ? 0 : (config >> 8) & 0xff;
  if (config >= 0) config = (config & 0xff) == 0xff ? -1 : (config & 0xff);
  int rc = validate(p);
  if (rc != TI_OK) return rc;
  if (p.batch == 0 || p.M == 0 || p.N == 0) return TI_OK;
  if (!dry) {
    rc = check_device();
    if (rc != TI_OK) return rc;
  }
  if (!p.bias) p.bias_kind = TI_BIAS_NONE;
  // the fast kernels quantise to int8 with round-half-even only; the truncating test switch runs
  // on the gather kernel
  const bool trunc8 = p.round_mode == TI_ROUND_TRUNC && out_class(p.out_dtype) == OUT8;
  int auto_splits = 1;
  if (config < 0) {
    // int8 truncation (a test-time switch) is implemented by the gather kernel and the M <= 64 kernels
    if (trunc8 && p.M > 16) config = (p.M <= 64 && fast_eligible(p)) ? CFG_SKINNY_16 + 1 + (p.M > 32) : CFG_GATHER;
    else config = pick_config(p, &auto_splits);
  }
  else if (config < g_num_configs && !want_splits && g_configs[config].ws_waves) auto_splits = pick_splits(p, g_configs[config], 1.0, nullptr);
  if (config >= g_num_configs) return fail(TI_E_COMBO, "config %d out of range", config);
  const Config& k = g_configs[config];
  if (!k.fn[out_class(p.out_dtype)]) return fail(TI_E_COMBO, "config %s has no kernel for output dtype %d", k.name, p.out_dtype);
  if (k.fast && !k.skinny && !k.rows4 && trunc8) return fail(TI_E_COMBO, "config %s does not implement TI_ROUND_TRUNC for int8 outputs", k.name);
  if (k.fast && !fast_eligible(p)) return fail(TI_E_COMBO, "config %s needs K-contiguous 16-byte aligned operands", k.name);
  if (k.stream_occ && !stream_eligible(p)) return fail(TI_E_COMBO, "config %s needs a row-major output with 16-byte aligned rows", k.name);
  if (k.max_k && (p.K < 16 || p.K > k.max_k)) return fail(TI_E_COMBO, "config %s needs 16 <= K <= %d", k.name, k.max_k);
  if (k.max_k && out_class(p.out_dtype) == OUT8 && (p.bias_kind != TI_BIAS_NONE || p.epilogue == TI_EPI_GELU_I8))
    return fail(TI_E_COMBO, "config %s has no int8 epilogue with a bias or GELU", k.name);
  if (k.rows4) {
    if (p.M > k.bm) return fail(TI_E_COMBO, "config %s needs M <= %d", k.name, k.bm);
    // K is not split over waves unless a test asks for it: the waves of a unit take turns at the
    // chunk barriers instead of streaming side by side (measured slower on every decode shape)
    const int units = (p.N + R4_RG - 1) / R4_RG;
    p.ksplit = 1;
    // forced by a test: low nibble the K split (1, 2, 4, 8), high nibble the streaming waves (4, 6, 8)
    int want_nwa = 0;
    if (want_splits) {
      const int ks = want_splits & 15;
      want_nwa = want_splits >> 4;
      if (ks != 0 && ks != 1 && ks != 2 && ks != 4 && ks != 8)
        return fail(TI_E_COMBO, "config %s splits K over 1, 2, 4 or 8 waves, not %d", k.name, ks);
      if (want_nwa != 0 && want_nwa != 4 && want_nwa != 6 && want_nwa != 8)
        return fail(TI_E_COMBO, "config %s streams on 4, 6 or 8 waves, not %d", k.name, want_nwa);
      if (ks) p.ksplit = ks;
      if (want_nwa && want_nwa != 8) p.ksplit = 1;
    }
    // One workgroup per CU (its LDS allows no second one), all batches together in one round of
    // the 256 CUs, every CU busy: what a CU can pull from memory is the limit (about 27 GB/s each),
    // so an idle CU costs more than waves of a workgroup that carry one unit less than others
    // (three grouped 5120 x 5120 projections: 25.6 -> 17.9 us).
    const int wgs = p.batch >= 256 ? 1 : 256 / p.batch;
    const int per = (units + wgs - 1) / wgs;
    const int blocks = (units + per - 1) / per;
    // the K split needs all of a workgroup's units in one pass
    if (p.ksplit > 1 && per > (R4_NW / p.ksplit) * R4_UMAX) {
      if (want_splits) return fail(TI_E_COMBO, "config %s: %d units per workgroup do not fit one pass with K split over %d waves", k.name, per, p.ksplit);
      p.ksplit = 1;
    }
    // 6 or fewer units per workgroup: 6 streaming waves with 4 ring stages each instead of 8 with 3
    // (weights rotated through > 600 MB: 5120 x 20480 28.6 -> 25.3 us, 4096 x 16384 24.0 -> 20.0 us,
    // 4096 x 4096 10.0 -> 8.7 us; 4 waves with 6 stages: equal or slower than 6 with 4)
    int nwa = want_nwa ? want_nwa : (p.ksplit == 1 && per <= 6 ? 6 : 8);
    if (nwa < 8 && per > nwa) return fail(TI_E_COMBO, "config %s: %d units per workgroup need more than %d waves", k.name, per, nwa);
    g_last_config = config;
    g_last_splits = p.ksplit;
    if (dry) {
      dry->config = config; dry->grid_x = (unsigned)blocks; dry->grid_y = (unsigned)p.batch; dry->threads = k.threads;
      dry->ksplit = p.ksplit; dry->nwa = nwa;
      return TI_OK;
    }
    rows4_kernel(out_class(p.out_dtype), nwa)<<<dim3((unsigned)blocks, (unsigned)p.batch), dim3(k.threads), 0, stream>>>(p);
    return launch_status(k.name);
  }
  if (k.skinny) {
    if (p.M > k.bm) return fail(TI_E_COMBO, "config %s needs M <= %d", k.name, k.bm);
    // a wave owns one group of k.bn rows of B; split K between the waves of a workgroup while
    // that makes more waves than the chip holds at once and leaves each at least 8 k-steps
    // (a wave streams slowly: short runs in many waves beat long runs in few)
    const int64_t groups = (int64_t)((p.N + k.bn - 1) / k.bn) * p.batch;
    const int ksteps = (p.K + 63) / 64;
    int ksplit = 1;
    while (ksplit < 8 && groups * ksplit < 4096 && ksteps / (ksplit * 2) >= 8) ksplit *= 2;
    p.ksplit = ksplit;
    const int per_block = 8 / ksplit;
    dim3 grid((unsigned)(((p.N + k.bn - 1) / k.bn + per_block - 1) / per_block), (unsigned)p.batch, 1);
    g_last_config = config;
    if (dry) {
      dry->config = config; dry->grid_x = grid.x; dry->grid_y = grid.y; dry->threads = k.threads; dry->ksplit = ksplit;
      return TI_OK;
    }
    k.fn[out_class(p.out_dtype)]<<<grid, dim3(k.threads), 0, stream>>>(p);
    return launch_status(k.name);
  }
  p.tiles_m = (p.M + k.bm - 1) / k.bm;
  p.tiles_n = (p.N + k.bn - 1) / k.bn;
  if ((int64_t)p.tiles_m * p.tiles_n > 0x7fffffff) return fail(TI_E_SHAPE, "too many tiles");
  p.group_m = pick_group_m(p, k);
  g_last_config = config;
  p.splits = 1;
  p.kt_split = 0;
  if (want_splits > 1 && !(k.ws_waves && p.batch == 1)) return fail(TI_E_COMBO, "config %s cannot split K (batch %d)", k.name, p.batch);
  if (k.ws_waves && p.batch == 1) {
    const int kt = (p.K + k.bk - 1) / k.bk;
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    int splits = want_splits ? want_splits : auto_splits;
    sk_shape(kt, splits, splits, p.kt_split);
    const size_t item_bytes = (size_t)k.bm * k.bn * sizeof(int);
    if (splits > 1 && static_scratch &&
        ((size_t)tiles * k.ws_waves > SK_STATIC_COUNTER_INTS || (size_t)tiles * splits * item_bytes > SK_STATIC_PARTIAL_BYTES)) {
      // a split the caller forced is refused; one the library chose itself gives way to the unsplit launch,
      // which needs no scratch at all (as the allocating path does when its workspace limit is exceeded)
      if (want_splits)
        return fail(TI_E_SHAPE, "%d K splits of %lld tiles need %zu bytes of partial sums: more than the %zu bytes of static scratch "
                    "(use ti_bmm_i8, which allocates its workspace)", splits, (long long)tiles, (size_t)tiles * splits * item_bytes,
                    SK_STATIC_PARTIAL_BYTES);
      sk_shape(kt, 1, splits, p.kt_split);
    }
    if (splits > 1 && static_scratch) {
      if (!dry) {
        rc = sk_static_scratch(stream, &p.sk_partial, &p.sk_counter);
        if (rc != TI_OK) return rc;
      }
    } else if (splits > 1 && ((size_t)tiles * k.ws_waves > SK_COUNTER_INTS || (size_t)tiles * splits * item_bytes > SK_MAX_PARTIAL_BYTES)) {
      if (want_splits) return fail(TI_E_SHAPE, "%d splits of %lld tiles exceed the split-K workspace", splits, (long long)tiles);
      splits = 1;
    }
    if (splits > 1 && !static_scratch && !dry) {
      hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
      (void)hipStreamIsCapturing(stream, &cap);
      rc = sk_workspace(stream, (size_t)tiles * splits * item_bytes, cap == hipStreamCaptureStatusNone, &p.sk_partial, &p.sk_counter);
      if (rc == TI_E_COMBO && !want_splits) splits = 1;  // capturing and nothing allocated yet: run unsplit
      else if (rc == TI_E_COMBO) return fail(TI_E_COMBO, "no split-K workspace on this stream and none can be allocated during graph capture");
      else if (rc != TI_OK) return rc;
    }
    p.splits = splits;
    if (dry && splits > 1) dry->partial_bytes = (int64_t)((size_t)tiles * splits * item_bytes);
  }
  g_last_splits = p.splits;
  if (dry) {
    dry->config = config; dry->splits = p.splits; dry->kt_split = p.kt_split; dry->tiles_m = p.tiles_m; dry->tiles_n = p.tiles_n;
    dry->group_m = p.group_m; dry->threads = k.threads;
  }
  if (k.stream_occ) {
    const int64_t items = (int64_t)p.tiles_m * p.tiles_n * p.batch * p.splits;
    if (items > 0x7fffffff) return fail(TI_E_SHAPE, "too many tiles");
    // a multiple of 8 keeps workgroup b on XCD b % 8; rounded up, so that no workgroup gets a second
    // item while CUs are idle (162 items on 160 workgroups took twice the time of 162 on 168; the
    // workgroups without an item return at once)
    int64_t g = items < 256 * k.stream_occ ? items : 256 * k.stream_occ;
    if (g >= 8) g = (g + 7) & ~(int64_t)7;
    if (dry) {
      dry->grid_x = (unsigned)g; dry->grid_y = 1;
      return TI_OK;
    }
    k.fn[out_class(p.out_dtype)]<<<dim3((unsigned)g), dim3(k.threads), 0, stream>>>(p);
    return launch_status(k.name);
  }
  dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)p.batch, 1);
  if (dry) {
    dry->grid_x = grid.x; dry->grid_y = grid.y;
    return TI_OK;
  }
  k.fn[out_class(p.out_dtype)]<<<grid, dim3(k.threads), 0, stream>>>(p);
  return launch_status(k.name);
}

}  // namespace ti

namespace ti {

// C[m][n] += R[m][n] for fp32 row-major matrices (unit column stride): the second launch of a linear
// with a residual when the GEMM kernel that ran does not add it itself.
__global__ __launch_bounds__(256) void add_rows_f32_kernel(float* C, int64_t ldc, const float* R, int64_t ldr, int M, int N, int vec) {
  const int64_t per_row = vec ? N / 4 : N;
  const int64_t total = (int64_t)M * per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / per_row, c = i - m * per_row;
    if (vec) {
      v4f* d = (v4f*)(C + m * ldc) + c;
      *d = *d + *((const v4f*)(R + m * ldr) + c);
    } else {
      C[m * ldc + c] += R[m * ldr + c];
    }
  }
}

static int run_with_residual(GemmParams p, const float* R, int64_t ldr, hipStream_t stream) {
  int rc = validate(p);
  if (rc != TI_OK) return rc;
  if (p.M == 0 || p.N == 0) return TI_OK;
  if (!R) return fail(TI_E_NULL, "residual is NULL");
  if ((const void*)R == (const void*)p.C) return fail(TI_E_STRIDE, "the output must not alias the residual");
  if (ldr < p.N || p.sCn != 1 || p.sCm < p.N) return fail(TI_E_STRIDE, "residual and output rows must be contiguous and cover a row");
  rc = check_device();
  if (rc != TI_OK) return rc;
  if (!p.bias) p.bias_kind = TI_BIAS_NONE;
  int splits = 1;
  const int cfg = pick_config(p, &splits);
  if (g_configs[cfg].rows4) {  // the decode kernel adds the residual in its store phase
    p.resid = R;
    p.resid_rs = ldr;
    return run(p, cfg, stream);
  }
  // the persistent kernels add it in their fp32 epilogue (unsplit K only: partial sums carry no residual);
  // 32-bit offsets into the residual, like the stores
  const bool persistent = g_configs[cfg].stream_occ > 0 || g_configs[cfg].ws_waves > 0 || g_configs[cfg].max_k > 0;
  if (persistent && splits == 1 && p.batch == 1 && p.out_dtype == TI_F32 && p.epilogue == TI_EPI_SCALE_F &&
      ((int64_t)(p.M + 512) * ldr + p.N) * 4 < ((int64_t)1 << 31)) {
    p.resid = R;
    p.resid_rs = ldr;
    return run(p, cfg | (1 << 8), stream);
  }
  rc = run(p, cfg | (splits << 8), stream);
  if (rc != TI_OK) return rc;
  const int vec = (p.N % 4 == 0) && (p.sCm % 4 == 0) && (ldr % 4 == 0) && (((uintptr_t)p.C | (uintptr_t)R) & 15) == 0;
  const int64_t items = (int64_t)p.M * (vec ? p.N / 4 : p.N);
  const unsigned blocks = (unsigned)(items / 256 + 1 < 256 * 16 ? items / 256 + 1 : 256 * 16);
  add_rows_f32_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((float*)p.C, p.sCm, R, ldr, p.M, p.N, vec);
  return launch_status("add_rows_f32_kernel");
}

}  // namespace ti

extern "C" {

int ti_bmm_i8_config(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk, const int8_t* B, int64_t sBb,
                     int64_t sBn, int64_t sBk, void* C, int64_t sCb, int64_t sCm, int64_t sCn, int batch, int M,
                     int N, int K, const void* bias, int bias_kind, const float* alpha, const float* beta,
                     int epilogue, int out_dtype, int round_mode, int config, void* stream) {
  ti::GemmParams p;
  p.A = A; p.B = B; p.C = C;
  p.sAb = sAb; p.sAm = sAm; p.sAk = sAk;
  p.sBb = sBb; p.sBn = sBn; p.sBk = sBk;
  p.sCb = sCb; p.sCm = sCm; p.sCn = sCn;
  p.batch = batch; p.M = M; p.N = N; p.K = K;
  p.bias = bias; p.bias_kind = bias_kind;
  p.alpha = alpha; p.beta = beta;
  p.epilogue = epilogue; p.out_dtype = out_dtype; p.round_mode = round_mode;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1; p.ksplit = 1;
  p.bias_bs = 0; p.scale_bs = 0;
  p.resid = nullptr; p.resid_rs = 0;
  p.kv_k = p.kv_vt = nullptr; p.kv_k_hs = p.kv_vt_rs = 0; p.kv_D = 1;
  p.splits = 1; p.kt_split = 0; p.sk_partial = p.sk_counter = nullptr;
  return ti::run(p, config, (hipStream_t)stream);
}

int ti_bmm_i8_grouped(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk, const int8_t* B, int64_t sBb,
                      int64_t sBn, int64_t sBk, void* C, int64_t sCb, int64_t sCm, int64_t sCn, int batch, int M,
                      int N, int K, const void* bias, int bias_kind, int64_t bias_batch_stride, const float* alpha,
                      const float* beta, int64_t scale_batch_stride, int epilogue, int out_dtype, int round_mode,
                      int config, void* stream) {
  if (bias_batch_stride < 0 || scale_batch_stride < 0) return ti::fail(TI_E_STRIDE, "negative batch stride of bias or scales");
  ti::GemmParams p;
  p.A = A; p.B = B; p.C = C;
  p.sAb = sAb; p.sAm = sAm; p.sAk = sAk;
  p.sBb = sBb; p.sBn = sBn; p.sBk = sBk;
  p.sCb = sCb; p.sCm = sCm; p.sCn = sCn;
  p.batch = batch; p.M = M; p.N = N; p.K = K;
  p.bias = bias; p.bias_kind = bias_kind;
  p.alpha = alpha; p.beta = beta;
  p.epilogue = epilogue; p.out_dtype = out_dtype; p.round_mode = round_mode;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1; p.ksplit = 1;
  p.bias_bs = bias_batch_stride; p.scale_bs = scale_batch_stride;
  p.resid = nullptr; p.resid_rs = 0;
  p.kv_k = p.kv_vt = nullptr; p.kv_k_hs = p.kv_vt_rs = 0; p.kv_D = 1;
  p.splits = 1; p.kt_split = 0; p.sk_partial = p.sk_counter = nullptr;
  return ti::run(p, config, (hipStream_t)stream);
}

int ti_qkv_decode_i8(const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw, const int8_t* bias,
                     const float* alpha3, const float* beta3, int8_t* C, int64_t ldc, int M, int N, int K,
                     int8_t* k_dst, int64_t k_head_stride, int8_t* vt_dst, int64_t vt_row_stride, int D,
                     void* stream) {
  using namespace ti;
  if (M > 16 || K < 1024 || D <= 0 || (D & 15) || N % D) return fail(TI_E_COMBO, "needs M <= 16, K >= 1024, D %% 16 == 0, N %% D == 0");
  if (!k_dst || !vt_dst) return fail(TI_E_NULL, "k_dst and vt_dst are required");
  if (((uintptr_t)k_dst & 3) || (k_head_stride & 3)) return fail(TI_E_STRIDE, "k_dst and its head stride must be multiples of 4 bytes");
  GemmParams p;
  p.A = A; p.B = W; p.C = C;
  p.sAb = 0; p.sAm = lda; p.sAk = 1;
  p.sBb = (int64_t)N * ldw; p.sBn = ldw; p.sBk = 1;
  p.sCb = N; p.sCm = ldc; p.sCn = 1;
  p.batch = 3; p.M = M; p.N = N; p.K = K;
  p.bias = bias; p.bias_kind = bias ? TI_BIAS_I8 : TI_BIAS_NONE;
  p.alpha = alpha3; p.beta = beta3;
  p.epilogue = TI_EPI_SCALE_I8; p.out_dtype = TI_I8; p.round_mode = TI_ROUND_RNE_CLAMP;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1; p.ksplit = 1;
  p.bias_bs = N; p.scale_bs = 1;
  p.resid = nullptr; p.resid_rs = 0;
  p.kv_k = k_dst; p.kv_vt = vt_dst; p.kv_k_hs = k_head_stride; p.kv_vt_rs = vt_row_stride; p.kv_D = D;
  p.splits = 1; p.kt_split = 0; p.sk_partial = p.sk_counter = nullptr;
  int rc = validate(p);
  if (rc != TI_OK) return rc;
  if (M == 0 || N == 0) return TI_OK;
  rc = check_device();
  if (rc != TI_OK) return rc;
  int splits = 1;
  const int cfg = pick_config(p, &splits);
  if (!g_configs[cfg].rows4) return fail(TI_E_COMBO, "operands not eligible for the decode kernel (16-byte aligned, K-contiguous)");
  return run(p, cfg, (hipStream_t)stream);
}

int ti_bmm_i8(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk, const int8_t* B, int64_t sBb, int64_t sBn,
              int64_t sBk, void* C, int64_t sCb, int64_t sCm, int64_t sCn, int batch, int M, int N, int K,
              const void* bias, int bias_kind, const float* alpha, const float* beta, int epilogue, int out_dtype,
              int round_mode, void* stream) {
  return ti_bmm_i8_config(A, sAb, sAm, sAk, B, sBb, sBn, sBk, C, sCb, sCm, sCn, batch, M, N, K, bias, bias_kind,
                          alpha, beta, epilogue, out_dtype, round_mode, -1, stream);
}

int ti_bmm_i8_static_scratch(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk, const int8_t* B, int64_t sBb, int64_t sBn,
                             int64_t sBk, void* C, int64_t sCb, int64_t sCm, int64_t sCn, int batch, int M, int N, int K,
                             const void* bias, int bias_kind, const float* alpha, const float* beta, int epilogue,
                             int out_dtype, int round_mode, int config, void* stream) {
  ti::GemmParams p;
  p.A = A; p.B = B; p.C = C;
  p.sAb = sAb; p.sAm = sAm; p.sAk = sAk;
  p.sBb = sBb; p.sBn = sBn; p.sBk = sBk;
  p.sCb = sCb; p.sCm = sCm; p.sCn = sCn;
  p.batch = batch; p.M = M; p.N = N; p.K = K;
  p.bias = bias; p.bias_kind = bias_kind;
  p.alpha = alpha; p.beta = beta;
  p.epilogue = epilogue; p.out_dtype = out_dtype; p.round_mode = round_mode;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1; p.ksplit = 1;
  p.bias_bs = 0; p.scale_bs = 0;
  p.resid = nullptr; p.resid_rs = 0;
  p.kv_k = p.kv_vt = nullptr; p.kv_k_hs = p.kv_vt_rs = 0; p.kv_D = 1;
  p.splits = 1; p.kt_split = 0; p.sk_partial = p.sk_counter = nullptr;
  return ti::run(p, config, (hipStream_t)stream, true);
}

int ti_linear_i8_residual_f32(const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw, const float* bias,
                              const float* alpha, const float* beta, const float* residual, int64_t ldr, float* C,
                              int64_t ldc, int M, int N, int K, void* stream) {
  ti::GemmParams p;
  p.A = A; p.B = W; p.C = C;
  p.sAb = 0; p.sAm = lda; p.sAk = 1;
  p.sBb = 0; p.sBn = ldw; p.sBk = 1;
  p.sCb = 0; p.sCm = ldc; p.sCn = 1;
  p.batch = 1; p.M = M; p.N = N; p.K = K;
  p.bias = bias; p.bias_kind = bias ? TI_BIAS_F32 : TI_BIAS_NONE;
  p.alpha = alpha; p.beta = beta;
  p.epilogue = TI_EPI_SCALE_F; p.out_dtype = TI_F32; p.round_mode = TI_ROUND_RNE_CLAMP;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1; p.ksplit = 1;
  p.bias_bs = 0; p.scale_bs = 0;
  p.resid = nullptr; p.resid_rs = 0;
  p.kv_k = p.kv_vt = nullptr; p.kv_k_hs = p.kv_vt_rs = 0; p.kv_D = 1;
  p.splits = 1; p.kt_split = 0; p.sk_partial = p.sk_counter = nullptr;
  return ti::run_with_residual(p, residual, ldr, (hipStream_t)stream);
}


int ti_gemm_plan(const int8_t* A, int64_t sAb, int64_t sAm, int64_t sAk, const int8_t* B, int64_t sBb, int64_t sBn,
                 int64_t sBk, void* C, int64_t sCb, int64_t sCm, int64_t sCn, int batch, int M, int N, int K,
                 const void* bias, int bias_kind, const float* alpha, const float* beta, int epilogue, int out_dtype,
                 int round_mode, int config, int static_scratch, int64_t* plan) {
  if (!plan) return ti::fail(TI_E_NULL, "plan is NULL");
  ti::GemmParams p;
  p.A = A; p.B = B; p.C = C;
  p.sAb = sAb; p.sAm = sAm; p.sAk = sAk;
  p.sBb = sBb; p.sBn = sBn; p.sBk = sBk;
  p.sCb = sCb; p.sCm = sCm; p.sCn = sCn;
  p.batch = batch; p.M = M; p.N = N; p.K = K;
  p.bias = bias; p.bias_kind = bias_kind;
  p.alpha = alpha; p.beta = beta;
  p.epilogue = epilogue; p.out_dtype = out_dtype; p.round_mode = round_mode;
  p.tiles_m = p.tiles_n = 0; p.group_m = 1; p.ksplit = 1;
  p.bias_bs = 0; p.scale_bs = 0;
  p.resid = nullptr; p.resid_rs = 0;
  p.kv_k = p.kv_vt = nullptr; p.kv_k_hs = p.kv_vt_rs = 0; p.kv_D = 1;
  p.splits = 1; p.kt_split = 0; p.sk_partial = p.sk_counter = nullptr;
  ti::LaunchPlan lp;
  const int rc = ti::run(p, config, nullptr, static_scratch != 0, &lp);
  const int64_t out[TI_PLAN_INTS] = {lp.config, lp.splits, lp.kt_split, lp.tiles_m, lp.tiles_n, lp.group_m, (int64_t)lp.grid_x,
                                     (int64_t)lp.grid_y, lp.threads, lp.ksplit, lp.nwa, lp.partial_bytes};
  for (int i = 0; i < TI_PLAN_INTS; ++i) plan[i] = out[i];
  return rc;
}

int ti_release_workspaces(void* stream, int all_streams, int64_t* freed_bytes) {
  return ti::sk_release((hipStream_t)stream, all_streams != 0, freed_bytes);
}

#ifdef TI_GEMM_TIMELINE
int ti_debug_timeline(unsigned long long* host, int n) {
  return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(ti::g_timeline), sizeof(unsigned long long) * n);
}
#endif

int ti_gemm_num_configs(void) { return ti::g_num_configs; }

int ti_gemm_last_config(void) { return ti::g_last_config; }

int ti_gemm_last_splits(void) { return ti::g_last_splits; }

const char* ti_gemm_config_name(int config) {
  return (config >= 0 && config < ti::g_num_configs) ? ti::g_configs[config].name : "";
}

}  // extern "C"
