// attention_i8.hip — int8 attention for one block of query rows without the score round trip.
//
// The reference's callers chain three launches per attention block (nn/bmm.py:10-29 for Q.K^T,
// a softmax in the caller, nn/bmm.py:10-29 / :54-74 for P.V):
//     scores = q8(qk_alpha * (q . k))                      int8 [BH, S, T]   (kernels/bmm.py:576-612)
//     probs  = rne(127 * softmax(scores * score_scale))    int8 [BH, S, T]   values 0..127
//     ctx    = q8(pv_alpha * (probs . v))                  int8 [BH, S, D]   (kernels/bmm.py:576-612)
// At 2048 x 2048 scores per head the two intermediates are 4 x 168 MB of HBM traffic for 40 heads.
// This kernel computes the same three steps per 32 x 32 block of scores in registers: the int8
// score quantisation, the probability quantisation and the context quantisation are the same
// fp32 operations as in the three kernels, and a row's exponentials are summed as integers (see
// the softmax-quantise arithmetic in ti_common.h), so the result is the three-kernel chain's bit
// for bit although the keys are visited in another order.
//
// Three passes over the keys of a query block.  Pass 0 finds each row's largest score (the
// exponent's reference point): the quantisation is monotone in the int32 accumulator, so it is a
// maximum over accumulators, one instruction per two scores.  Pass 1 recomputes the scores
// (K = 128 deep: cheap) and sums the exponentials.  Pass 2 recomputes them once more, forms the
// int8 probabilities in the MFMA operand layout straight from the accumulator registers (two
// half-wave swaps put a row's keys in order) and feeds them to the P.V MFMAs, so P never goes
// through memory.
//
// (Blocks of 16 or fewer query rows take attention_decode_i8_kernel further down instead.)
//
// Workgroup = 4 waves = 128 query rows of one head; a wave owns 32 rows.  K and V^T are staged
// through LDS in tiles of 64 keys, double-buffered, one barrier per tile.  Causal masking skips
// whole key tiles beyond a wave's last visible key and masks inside the tiles on the diagonal.
#include <type_traits>

#include "ti_common.h"

namespace ti {

constexpr int AT_D = 128;                // head dimension this kernel is written for
constexpr int AT_ROWS = 128;             // query rows per workgroup
constexpr int AT_KT = 64;                // keys per LDS tile
constexpr int AT_KP = AT_D + 16;         // K tile row pitch (bytes): 16-byte reads of 16 rows hit 64 different banks
constexpr int AT_VP = AT_KT + 16;        // V^T tile row pitch
constexpr int AT_KBYTES = AT_KT * AT_KP;
constexpr int AT_VBYTES = AT_D * AT_VP;

struct AttnParams {
  const int8_t* q; const int8_t* k; const int8_t* vt; int8_t* out;
  int64_t sQb, sQm, sKb, sKn, sVb, sVd, sOb, sOm;
  int S, T, causal_q_len, nblk, batch;
  float qk_alpha, s2, pv_alpha;  // s2 = score_scale * log2(e)
};

__device__ __forceinline__ int attn_limit(const AttnParams& p, int row) {
  return p.causal_q_len > 0 ? min(p.T, (row % p.causal_q_len) + (p.T - p.causal_q_len) + 1) : p.T;
}

__global__ __launch_bounds__(256, 2) void attention_i8_kernel(AttnParams p) {
  __shared__ __attribute__((aligned(16))) char lds[2 * (AT_KBYTES + AT_VBYTES)];
  __shared__ int wg_lim[4];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lrow = lane & 31, lhi = lane >> 5;
  // Work item = (head, block of 128 query rows).  Under a causal mask a later row block sees more
  // keys, and every workgroup of a launch of this size is resident at once, workgroup i on the same
  // CU as i + 256 and i + 512 (measured placement).  The items are therefore taken in order of
  // decreasing work and dealt to the workgroup indices in a snake: 0..255 forward, 256..511
  // backward, ..., which gives every CU about the same total.
  const int n_items = p.nblk * p.batch;
  const int pass = (int)blockIdx.x >> 8, c = (int)blockIdx.x & 255;
  const int cnt = min(256, n_items - pass * 256);
  const int pos = pass * 256 + ((pass & 1) ? cnt - 1 - c : c);
  const int bh = pos % p.batch;
  const int m0 = (p.nblk - 1 - pos / p.batch) * AT_ROWS + wave * 32;
  const int8_t* qb = p.q + (int64_t)bh * p.sQb;
  const int8_t* kb_ = p.k + (int64_t)bh * p.sKb;
  const int8_t* vb = p.vt + (int64_t)bh * p.sVb;

  // ---- per-lane row, visible-key limit; wave and workgroup bounds
  const int row = m0 + lrow;
  const int rowc = min(row, p.S - 1);                       // rows past S repeat the last row, never stored
  const int lim_lane = attn_limit(p, min(max(rowc, 0), p.S - 1));
  int lim_hi = lim_lane, lim_lo = lim_lane;
#pragma unroll
  for (int off = 16; off > 0; off >>= 1) {
    lim_hi = max(lim_hi, __shfl_xor(lim_hi, off, 64));
    lim_lo = min(lim_lo, __shfl_xor(lim_lo, off, 64));
  }
  lim_hi = __builtin_amdgcn_readfirstlane(lim_hi);
  lim_lo = __builtin_amdgcn_readfirstlane(lim_lo);
  const bool wave_live = m0 < p.S;                          // a wave wholly past S computes nothing
  if (lane == 0) wg_lim[wave] = wave_live ? lim_hi : 0;
  __syncthreads();
  const int wg_hi = max(max(wg_lim[0], wg_lim[1]), max(wg_lim[2], wg_lim[3]));
  const int ntiles = __builtin_amdgcn_readfirstlane((wg_hi + AT_KT - 1) / AT_KT);

  // ---- this wave's Q fragments (32 rows x 128 d): lane (row, half) holds 16 bytes per 32-deep step
  v4i qf[4];
#pragma unroll
  for (int ds = 0; ds < 4; ++ds)
    qf[ds] = *(const v4i*)(qb + (int64_t)rowc * p.sQm + ds * 32 + lhi * 16);

  // ---- tile staging: thread t copies two 16-byte chunks of the K tile and two of the V^T tile
  v4i kreg[2], vreg[2];
  auto fetch = [&](int t, bool with_v) {
    const int key0 = t * AT_KT;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int q_ = c * 256 + tid;          // chunk index: 64 keys x 8 chunks
      const int kr = q_ >> 3, kc = q_ & 7;
      const bool in = key0 + kr < p.T;
      kreg[c] = in ? *(const v4i*)(kb_ + (int64_t)(key0 + kr) * p.sKn + kc * 16) : (v4i){0, 0, 0, 0};
    }
    if (with_v) {
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int q_ = c * 256 + tid;        // chunk index: 128 d x 4 chunks of 16 keys
        const int vr = q_ >> 2, vc = q_ & 3;
        const bool in = key0 + vc * 16 < p.T;  // T % 16 == 0: a chunk is wholly inside or outside
        vreg[c] = in ? *(const v4i*)(vb + (int64_t)vr * p.sVd + key0 + vc * 16) : (v4i){0, 0, 0, 0};
      }
    }
  };
  auto stash = [&](int buf, bool with_v) {
    char* kt = lds + buf * (AT_KBYTES + AT_VBYTES);
    char* vt = kt + AT_KBYTES;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int q_ = c * 256 + tid;
      *(v4i*)(kt + (q_ >> 3) * AT_KP + (q_ & 7) * 16) = kreg[c];
    }
    if (with_v) {
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int q_ = c * 256 + tid;
        *(v4i*)(vt + (q_ >> 2) * AT_VP + (q_ & 3) * 16) = vreg[c];
      }
    }
  };

  const float MAGIC = 12582912.0f;  // 1.5 * 2^23: adding it rounds to the nearest even integer

  // ================= pass 0: each row's largest score =================
  // q8(alpha * f(acc)) does not decrease with acc when alpha >= 0 (and does not increase when
  // alpha < 0), so the largest score is the quantised largest (smallest) accumulator.
  const bool want_max = p.qk_alpha >= 0.0f;
  int ext = want_max ? (int)0x80000000 : 0x7fffffff;
  auto score_ext_t = [&](const char* kt, int key0, auto mask_tag, auto max_tag) {
    constexpr bool MASK = decltype(mask_tag)::value;
    constexpr bool MAX = decltype(max_tag)::value;
    v4i kf[2][4];
#pragma unroll
    for (int ds = 0; ds < 4; ++ds)
#pragma unroll
      for (int b = 0; b < 2; ++b) kf[b][ds] = *(const v4i*)(kt + (b * 32 + lrow) * AT_KP + ds * 32 + lhi * 16);
    v16i s[2];
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int ds = 0; ds < 4; ++ds)
#pragma unroll
      for (int b = 0; b < 2; ++b)
        s[b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[b][ds], qf[ds], ds == 0 ? zero : s[b], 0, 0, 0);
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        int v = s[b][r];
        if constexpr (MASK) {
          const int key = key0 + 32 * b + 8 * (r >> 2) + 4 * lhi + (r & 3);
          v = key < lim_lane ? v : (MAX ? (int)0x80000000 : 0x7fffffff);
        }
        ext = MAX ? max(ext, v) : min(ext, v);
      }
  };
  auto score_ext = [&](const char* kt, int key0) {
    const bool mask = key0 + AT_KT > lim_lo;
    if (want_max) {
      if (mask) score_ext_t(kt, key0, std::true_type{}, std::true_type{});
      else score_ext_t(kt, key0, std::false_type{}, std::true_type{});
    } else {
      if (mask) score_ext_t(kt, key0, std::true_type{}, std::false_type{});
      else score_ext_t(kt, key0, std::false_type{}, std::false_type{});
    }
  };
  fetch(0, false);
  stash(0, false);
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    if (t + 1 < ntiles) fetch(t + 1, false);
    const char* kt = lds + (t & 1) * (AT_KBYTES + AT_VBYTES);
    if (wave_live && t * AT_KT < lim_hi) score_ext(kt, t * AT_KT);
    if (t + 1 < ntiles) stash((t + 1) & 1, false);
    __syncthreads();
  }
  {
    const int other = __shfl_xor(ext, 32, 64);  // the two lane halves hold different keys of the same row
    ext = want_max ? max(ext, other) : min(ext, other);
  }
  float cref;  // -(largest score * s2): the exponent's reference point of this lane's row
  {
    float v = (float)ext * p.qk_alpha;
    v = __builtin_amdgcn_fmed3f(v, -128.0f, 127.0f);
    cref = -(__builtin_rintf(v) * p.s2);
  }
  // Scores of one 64-key tile -> exponentials.  The tile's two 32-key blocks are two independent
  // MFMA chains, interleaved, with all fragment reads issued first; e[b][r] belongs to key
  // key0 + 32*b + 8*(r/4) + 4*lhi + r%4.  A block that lies wholly beyond the wave's last visible
  // key is computed too and masked to zero (at most one per wave and pass).
  auto score_exp_t = [&](const char* kt, int key0, float (&e)[2][16], auto mask_tag) {
    constexpr bool MASK = decltype(mask_tag)::value;
    v4i kf[2][4];
#pragma unroll
    for (int ds = 0; ds < 4; ++ds)
#pragma unroll
      for (int b = 0; b < 2; ++b) kf[b][ds] = *(const v4i*)(kt + (b * 32 + lrow) * AT_KP + ds * 32 + lhi * 16);
    v16i s[2];
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int ds = 0; ds < 4; ++ds)
#pragma unroll
      for (int b = 0; b < 2; ++b)
        s[b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[b][ds], qf[ds], ds == 0 ? zero : s[b], 0, 0, 0);  // rows of the result = keys
#pragma unroll
    for (int b = 0; b < 2; ++b) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float v = (float)s[b][r] * p.qk_alpha;
        v = __builtin_amdgcn_fmed3f(v, -128.0f, 127.0f);
        const float x = __builtin_rintf(v);  // the int8 score, as a float (round half to even, like the BMM's)
        e[b][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(x, p.s2, cref));
      }
      if constexpr (MASK) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + 32 * b + 8 * (r >> 2) + 4 * lhi + (r & 3);
          e[b][r] = key < lim_lane ? e[b][r] : 0.0f;
        }
      }
    }
  };
  // Off the diagonal no row's limit falls inside or before the tile and the selects above must
  // cost nothing: two instantiations behind a wave-uniform branch (the MFMAs inside keep the
  // compiler from folding them back into one block of selects).
  auto score_exp = [&](const char* kt, int key0, float (&e)[2][16]) {
    if (key0 + AT_KT > lim_lo) score_exp_t(kt, key0, e, std::true_type{});
    else score_exp_t(kt, key0, e, std::false_type{});
  };

  // ================= pass 1: row sums (exact integers, see ti_common.h) =================
  unsigned long long sum = 0;
  fetch(0, false);
  stash(0, false);
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    if (t + 1 < ntiles) fetch(t + 1, false);
    const char* kt = lds + (t & 1) * (AT_KBYTES + AT_VBYTES);
    if (wave_live && t * AT_KT < lim_hi) {
      float e[2][16];
      score_exp(kt, t * AT_KT, e);
      unsigned s0 = 0, s1 = 0;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s0 += sm_unit_bits(e[0][r]);
        s1 += sm_unit_bits(e[1][r]);
      }
      sum += (unsigned)(s0 + s1 - 32u * SM_ONE_BITS);  // modulo 2^32: the tile's 32 units of this lane, below 2^29
    }
    if (t + 1 < ntiles) stash((t + 1) & 1, false);
    __syncthreads();
  }
  {
    // the two lane halves hold different keys of the same row
    const unsigned lo = (unsigned)__shfl_xor((int)(unsigned)sum, 32, 64);
    const unsigned hi = (unsigned)__shfl_xor((int)(unsigned)(sum >> 32), 32, 64);
    sum += ((unsigned long long)hi << 32) | lo;
  }
  const float rinv = sm_scale_from_sum(sum);

  // ================= pass 2: probabilities and P.V =================
  v16i o[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0;
  fetch(0, true);
  stash(0, true);
  __syncthreads();
  for (int t = 0; t < ntiles; ++t) {
    if (t + 1 < ntiles) fetch(t + 1, true);
    const char* kt = lds + (t & 1) * (AT_KBYTES + AT_VBYTES);
    const char* vt = kt + AT_KBYTES;
    if (wave_live && t * AT_KT < lim_hi) {
      float e[2][16];
      score_exp(kt, t * AT_KT, e);
      v4i vf[2][4];
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int b = 0; b < 2; ++b) vf[b][db] = *(const v4i*)(vt + (db * 32 + lrow) * AT_VP + b * 32 + lhi * 16);
      v4i pf[2];  // 16 int8 probabilities of this lane's row per block, keys in accumulator order
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const unsigned b0 = __float_as_uint(__builtin_fmaf(e[b][4 * g + 0], rinv, MAGIC));
          const unsigned b1 = __float_as_uint(__builtin_fmaf(e[b][4 * g + 1], rinv, MAGIC));
          const unsigned b2 = __float_as_uint(__builtin_fmaf(e[b][4 * g + 2], rinv, MAGIC));
          const unsigned b3 = __float_as_uint(__builtin_fmaf(e[b][4 * g + 3], rinv, MAGIC));
          pf[b][g] = (int)(__builtin_amdgcn_perm(b1, b0, 0x0c0c0400u) | __builtin_amdgcn_perm(b3, b2, 0x04000c0cu));
        }
      // The accumulators hold a row's 32 keys of a block as alternate 4-key groups in the two lane
      // halves; two half-wave swaps give lane half h the keys 16h .. 16h+15 in order, which is how
      // the MFMA wants its 32-deep operand and how V^T lies in LDS.
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const auto s02 = __builtin_amdgcn_permlane32_swap((unsigned)pf[b][0], (unsigned)pf[b][2], false, false);
        const auto s13 = __builtin_amdgcn_permlane32_swap((unsigned)pf[b][1], (unsigned)pf[b][3], false, false);
        pf[b][0] = (int)s02[0]; pf[b][1] = (int)s02[1]; pf[b][2] = (int)s13[0]; pf[b][3] = (int)s13[1];
      }
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int db = 0; db < 4; ++db)
          o[db] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf[b][db], pf[b], o[db], 0, 0, 0);  // rows of the result = d
    }
    if (t + 1 < ntiles) stash((t + 1) & 1, true);
    __syncthreads();
  }

  // ---- context: o[db][r] is row lrow, d = 32*db + 8*(r/4) + 4*lhi + r%4 -> int8, 16 bytes per lane
  if (!wave_live) return;
  int8_t* ob = p.out + (int64_t)bh * p.sOb;
#pragma unroll
  for (int db = 0; db < 4; ++db) {
    unsigned X[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      unsigned b[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        float v = (float)o[db][4 * g + t] * p.pv_alpha;
        v = __builtin_amdgcn_fmed3f(v, -128.0f, 127.0f);
        b[t] = __float_as_uint(v + MAGIC);
      }
      X[g] = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u) | __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
    }
    // lanes l and l+32 hold alternate 4-byte groups of the row's 32 bytes: after the two swaps
    // lane l has bytes 0..15 and lane l+32 bytes 16..31
    const auto s02 = __builtin_amdgcn_permlane32_swap(X[0], X[2], false, false);
    const auto s13 = __builtin_amdgcn_permlane32_swap(X[1], X[3], false, false);
    v4u v;
    v[0] = s02[0]; v[1] = s02[1]; v[2] = s13[0]; v[3] = s13[1];
    if (row < p.S) *(v4u*)(ob + (int64_t)row * p.sOm + db * 32 + lhi * 16) = v;
  }
}


// ---- few query rows (decode): one workgroup per head ------------------------------------------------
//
// With 16 or fewer query rows per head a head's whole attention fits one workgroup: 16 waves, one
// pass.  Wave w computes the scores of the 16-key chunks w, w + 16, ... with 16x16x64 MFMAs (K rows
// loaded from memory straight into the operand layout: 16 rows x 64 bytes per instruction) and keeps
// them in registers; row maximum and sum go through LDS; the int8 probabilities are written to LDS in
// key order ([16 queries][T]), from where every wave reads them back as MFMA operands for P.V: wave w
// owns 16 of the 128 output columns (V^T rows, also loaded straight into the operand layout) and
// one half of the 64-key groups; the two halves meet in LDS.  The arithmetic is that of the three
// kernels (score quantisation, exponent against the row maximum, 127 / sum, context quantisation);
// only the order of a row's sum differs.
constexpr int AD_WAVES = 16;
constexpr int AD_MAXT = 4096;

// CPW: 16-key chunks per wave (T <= 256 * CPW).  DBW: 16-column blocks of the output a workgroup
// produces (8: the whole head; fewer: the head is spread over 8 / DBW workgroups, each of which
// repeats the scores and the softmax and reads only its rows of V^T — a single CU fills its caches at
// about 30 GB/s, so a head's 512 KB of K and V^T through one CU alone would take 17 us).
template <int CPW, int DBW>
__global__ __launch_bounds__(AD_WAVES * 64) void attention_decode_i8_kernel(AttnParams p) {
  constexpr int TMAX = 256 * CPW;
  constexpr int PP = TMAX + 16;             // LDS pitch of a query's probabilities
  constexpr int KPARTS = AD_WAVES / DBW;    // waves that share an output block and split the keys
  constexpr int GPW = (TMAX / 64 + KPARTS - 1) / KPARTS;  // 64-key groups per wave in P.V
  constexpr int HOIST = CPW >= 16 ? (GPW < 4 ? GPW : 4) : GPW;  // V^T operands fetched before the softmax reductions
  __shared__ __attribute__((aligned(16))) char p_lds[16 * PP];
  __shared__ float red_max[AD_WAVES][16];
  __shared__ unsigned red_sum[AD_WAVES][16];
  __shared__ __attribute__((aligned(16))) v4i ctx_red[AD_WAVES][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, kq = lane >> 4;  // operand row / 16-byte quarter of a 64-deep k-step
  // the workgroups of a head are p.batch apart: with a batch that is a multiple of 8 they run on the
  // same XCD and share its L2 for K
  const int bh = blockIdx.x % p.batch;
  const int dbase = (blockIdx.x / p.batch) * DBW;
  const int OOB = 0x7ffffff0;
  const float MAGIC = 12582912.0f;
  const __amdgpu_buffer_rsrc_t rQ =
      __builtin_amdgcn_make_buffer_rsrc((void*)(p.q + (int64_t)bh * p.sQb), 0, (int)((p.S - 1) * p.sQm + AT_D), 0x00020000);
  const __amdgpu_buffer_rsrc_t rK =
      __builtin_amdgcn_make_buffer_rsrc((void*)(p.k + (int64_t)bh * p.sKb), 0, (int)((p.T - 1) * p.sKn + AT_D), 0x00020000);
  const __amdgpu_buffer_rsrc_t rV =
      __builtin_amdgcn_make_buffer_rsrc((void*)(p.vt + (int64_t)bh * p.sVb), 0, (int)((AT_D - 1) * p.sVd + p.T), 0x00020000);
  const int NCH = p.T >> 4;         // 16-key chunks
  const int NG = (p.T + 63) >> 6;   // 64-key groups
  const int db = dbase + wave % DBW, kh = wave / DBW;

  // ---- scores: f = the int8 score as a float, -inf where masked or beyond T
  v4i qf[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
    qf[ks] = __builtin_amdgcn_raw_buffer_load_b128(rQ, n < p.S ? n * (int)p.sQm + ks * 64 + kq * 16 : OOB, 0, 0);
  const int limit = p.causal_q_len > 0 ? min(p.T, (n % p.causal_q_len) + (p.T - p.causal_q_len) + 1) : p.T;
  const float NEG = -__builtin_inff();
  float f[CPW][4];
  constexpr int NB = CPW < 8 ? CPW : (CPW > 8 ? 4 : 8);  // chunks whose K operands are in flight together
#pragma unroll
  for (int b0 = 0; b0 < CPW; b0 += NB) {
    v4i kf[NB][2];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int c = wave + AD_WAVES * (b0 + i);
      const int off = (c * 16 + n) * (int)p.sKn + kq * 16;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) kf[i][ks] = __builtin_amdgcn_raw_buffer_load_b128(rK, c < NCH ? off + ks * 64 : OOB, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int c = wave + AD_WAVES * (b0 + i);
      v4i acc = {0, 0, 0, 0};
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf[i][0], qf[0], acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf[i][1], qf[1], acc, 0, 0, 0);
      // acc[r]: key c*16 + 4*kq + r, query n
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = (float)acc[r] * p.qk_alpha;
        v = __builtin_amdgcn_fmed3f(v, -128.0f, 127.0f);
        const int key = c * 16 + 4 * kq + r;
        f[b0 + i][r] = key < limit ? __builtin_rintf(v) : NEG;
      }
    }
  }
  // V^T operands of this wave's first groups: in flight during the reductions below
  v4i vf[HOIST];
#pragma unroll
  for (int i = 0; i < HOIST; ++i) {
    const int g = kh + KPARTS * i;
    const int col = 64 * g + 16 * kq;
    vf[i] = __builtin_amdgcn_raw_buffer_load_b128(rV, col < p.T ? (16 * db + n) * (int)p.sVd + col : OOB, 0, 0);
  }

  // ---- row maximum (exact: integers), exponentials, row sum
  float mx = NEG;
#pragma unroll
  for (int i = 0; i < CPW; ++i) mx = fmaxf(fmaxf(mx, fmaxf(f[i][0], f[i][1])), fmaxf(f[i][2], f[i][3]));
  mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
  mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
  if (kq == 0) red_max[wave][n] = mx;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < AD_WAVES; ++w) mx = fmaxf(mx, red_max[w][n]);
  const float c0 = -(mx * p.s2);
  // exact integer row sum (see ti_common.h): a lane holds at most 64 scores (below 2^29 units), the
  // four lanes of a query below 2^31, the 16 waves meet in 64 bits
  unsigned bits = 0;
#pragma unroll
  for (int i = 0; i < CPW; ++i)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      f[i][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(f[i][r], p.s2, c0));
      bits += sm_unit_bits(f[i][r]);
    }
  bits -= (unsigned)(CPW * 4) * SM_ONE_BITS;  // modulo 2^32
  bits += (unsigned)__shfl_xor((int)bits, 16, 64);
  bits += (unsigned)__shfl_xor((int)bits, 32, 64);
  if (kq == 0) red_sum[wave][n] = bits;
  __syncthreads();
  unsigned long long sum = 0;
#pragma unroll
  for (int w = 0; w < AD_WAVES; ++w) sum += red_sum[w][n];
  const float rcp = sm_scale_from_sum(sum);

  // ---- int8 probabilities into LDS, key order; keys in [T, 64 * NG) get zeros (their f is -inf)
#pragma unroll
  for (int i = 0; i < CPW; ++i) {
    const int c = wave + AD_WAVES * i;
    if (c < 4 * NG) {
      const unsigned b0 = __float_as_uint(__builtin_fmaf(f[i][0], rcp, MAGIC)), b1 = __float_as_uint(__builtin_fmaf(f[i][1], rcp, MAGIC));
      const unsigned b2 = __float_as_uint(__builtin_fmaf(f[i][2], rcp, MAGIC)), b3 = __float_as_uint(__builtin_fmaf(f[i][3], rcp, MAGIC));
      *(unsigned*)(p_lds + n * PP + 16 * c + 4 * kq) =
          __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u) | __builtin_amdgcn_perm(b3, b2, 0x04000c0cu);
    }
  }
  __syncthreads();

  // ---- P.V: D[d = 16*db + 4*kq + r][query n] over this wave's key groups
  v4i o = {0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < HOIST; ++i) {
    const int g = kh + KPARTS * i;
    if (g < NG) o = __builtin_amdgcn_mfma_i32_16x16x64_i8(vf[i], *(const v4i*)(p_lds + n * PP + 64 * g + 16 * kq), o, 0, 0, 0);
  }
#pragma unroll
  for (int i0 = HOIST; i0 < GPW; i0 += 4) {
    v4i vb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = 64 * (kh + KPARTS * (i0 + i)) + 16 * kq;
      vb[i] = __builtin_amdgcn_raw_buffer_load_b128(rV, col < p.T ? (16 * db + n) * (int)p.sVd + col : OOB, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int g = kh + KPARTS * (i0 + i);
      if (g < NG) o = __builtin_amdgcn_mfma_i32_16x16x64_i8(vb[i], *(const v4i*)(p_lds + n * PP + 64 * g + 16 * kq), o, 0, 0, 0);
    }
  }
  if (kh > 0) ctx_red[wave][lane] = o;
  __syncthreads();
  if (kh == 0 && n < p.S) {
#pragma unroll
    for (int k2 = 1; k2 < KPARTS; ++k2) o += ctx_red[wave + k2 * DBW][lane];
    unsigned b[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v = (float)o[r] * p.pv_alpha;
      v = __builtin_amdgcn_fmed3f(v, -128.0f, 127.0f);
      b[r] = __float_as_uint(v + MAGIC);
    }
    *(unsigned*)(p.out + (int64_t)bh * p.sOb + (int64_t)n * p.sOm + 16 * db + 4 * kq) =
        __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u) | __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
  }
}

}  // namespace ti

extern "C" int ti_attention_i8(const int8_t* q, int64_t q_batch_stride, int64_t q_row_stride, const int8_t* k,
                               int64_t k_batch_stride, int64_t k_row_stride, const int8_t* vt,
                               int64_t vt_batch_stride, int64_t vt_row_stride, int8_t* out, int64_t out_batch_stride,
                               int64_t out_row_stride, int batch, int S, int T, int D, float qk_alpha,
                               float score_scale, float pv_alpha, int causal_q_len, void* stream) {
  using namespace ti;
  if (batch < 0 || S < 0 || T < 0 || causal_q_len < 0) return fail(TI_E_SHAPE, "negative size");
  if (batch == 0 || S == 0) return TI_OK;
  if (!q || !k || !vt || !out) return fail(TI_E_NULL, "q, k, vt and out are required");
  if (D != AT_D) return fail(TI_E_SHAPE, "head dimension %d: this kernel is built for %d", D, AT_D);
  if (T <= 0 || (T & 15)) return fail(TI_E_SHAPE, "T = %d must be a positive multiple of 16", T);
  if (batch > 65535) return fail(TI_E_SHAPE, "batch %d > 65535", batch);
  if (causal_q_len > T) return fail(TI_E_SHAPE, "causal_q_len %d > T %d", causal_q_len, T);
  if (causal_q_len > 0 && S % causal_q_len) return fail(TI_E_SHAPE, "S %d not a multiple of causal_q_len %d", S, causal_q_len);
  if (q_row_stride < D || k_row_stride < D || out_row_stride < D || vt_row_stride < T)
    return fail(TI_E_STRIDE, "row strides must cover a row");
  const uintptr_t align = (uintptr_t)q | (uintptr_t)k | (uintptr_t)vt | (uintptr_t)out | (uintptr_t)q_batch_stride |
                          (uintptr_t)q_row_stride | (uintptr_t)k_batch_stride | (uintptr_t)k_row_stride |
                          (uintptr_t)vt_batch_stride | (uintptr_t)vt_row_stride | (uintptr_t)out_batch_stride |
                          (uintptr_t)out_row_stride;
  if (align & 15) return fail(TI_E_STRIDE, "pointers and strides must be multiples of 16 bytes");
  const float s2 = score_scale * 1.44269504088896340736f;
  if (!(score_scale > 0.0f) || !(score_scale <= SM_MAX_SCALE))
    return fail(TI_E_COMBO, "score_scale %g outside (0, %g]: the quantised softmax is exact in that range only", (double)score_scale, (double)SM_MAX_SCALE);
  const int64_t lim32 = (int64_t)1 << 31;
  const bool few_rows = S <= 16 && T <= AD_MAXT && (int64_t)T * k_row_stride < lim32 && (int64_t)AT_D * vt_row_stride < lim32 &&
                        (int64_t)S * q_row_stride < lim32;
  int rc = check_device();
  if (rc != TI_OK) return rc;
  AttnParams p;
  p.q = q; p.k = k; p.vt = vt; p.out = out;
  p.sQb = q_batch_stride; p.sQm = q_row_stride; p.sKb = k_batch_stride; p.sKn = k_row_stride;
  p.sVb = vt_batch_stride; p.sVd = vt_row_stride; p.sOb = out_batch_stride; p.sOm = out_row_stride;
  p.S = S; p.T = T; p.causal_q_len = causal_q_len;
  p.qk_alpha = qk_alpha; p.s2 = s2; p.pv_alpha = pv_alpha;
  p.nblk = (S + AT_ROWS - 1) / AT_ROWS;
  p.batch = batch;
  if (few_rows) {
    // spread a head over as many workgroups as keep the launch within one round of the 256 CUs
    // (measured, 40 heads x 16 rows x 2048 keys: 18.9 / 15.3 / 13.6 us for 1 / 2 / 4 workgroups per head,
    // 24 us for 8, which no longer fit one round)
    int dbw = 8;
    while (dbw > 1 && (int64_t)batch * (16 / dbw) <= 256) dbw /= 2;
    const dim3 grid((unsigned)(batch * (8 / dbw))), block(AD_WAVES * 64);
    const hipStream_t st = (hipStream_t)stream;
#define TI_AD_LAUNCH(C) \
    (dbw == 8 ? attention_decode_i8_kernel<C, 8><<<grid, block, 0, st>>>(p) : dbw == 4 ? attention_decode_i8_kernel<C, 4><<<grid, block, 0, st>>>(p) \
     : dbw == 2 ? attention_decode_i8_kernel<C, 2><<<grid, block, 0, st>>>(p) : attention_decode_i8_kernel<C, 1><<<grid, block, 0, st>>>(p))
    if (T <= 1024) TI_AD_LAUNCH(4);
    else if (T <= 2048) TI_AD_LAUNCH(8);
    else TI_AD_LAUNCH(16);
#undef TI_AD_LAUNCH
    return launch_status("attention_decode_i8_kernel");
  }
  attention_i8_kernel<<<dim3((unsigned)(p.nblk * batch)), dim3(256), 0, (hipStream_t)stream>>>(p);
  return launch_status("attention_i8_kernel");
}
