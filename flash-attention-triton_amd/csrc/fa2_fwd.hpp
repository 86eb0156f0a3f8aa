// Causal FlashAttention-2 forward for gfx950.
//
// Computes what the reference's _forward_kernel computes
// (src/flash_attention_triton/_triton_kernels_v2.py:11-189): O = softmax(scale*QK^T + mask) V and
// the row log-sum-exp, with the online-softmax recurrence of lines 122-171, but laid out for
// wave64 MFMA instead of Triton blocks:
//
//  * A workgroup of 4 waves owns 128 query rows; each wave owns 32 of them for the whole kernel.
//  * Scores are produced TRANSPOSED, S^T = K Q^T (key rows x query columns), so that one lane
//    owns one query column: the running max and sum live in that lane's registers and a row
//    reduction is an in-lane reduction plus one exchange with lane^32.
//  * The accumulator is O^T = V^T P^T.  P^T leaves the first MFMA in exactly the register layout
//    the second MFMA wants for its B operand, so probabilities never touch LDS.  V^T fragments are
//    read from the row-major V tile with the transposing LDS read.
//  * K and V tiles are staged in LDS (two stages each in the generic kernel, three K stages and
//    two V stages in the fast one); the next tiles' global loads are in flight while the current
//    tile is being multiplied.
//  * Unlike the reference (mask applied to every tile, lines 139-147) the mask is evaluated only
//    on tiles that touch the diagonal or the end of the key sequence, and sub-blocks entirely
//    above the diagonal are skipped.
//  * The maximum the probabilities are formed against is raised lazily (see kRescaleSlack); the
//    reference floors its maximum with the running lse (line 150).  Both only change rounding.
#pragma once

#include <type_traits>

#include "fa2_common.hpp"

namespace fa2 {

// The running max is only raised (and the accumulator rescaled) when some row's new maximum
// exceeds the one in use by more than this many powers of two; until then probabilities are
// formed against the stale maximum and may reach 2^kRescaleSlack, which fp32 sums and bf16/fp16
// operands hold without loss.  The final division by the row sum removes the common factor.
constexpr float kRescaleSlack = 8.0f;
// The fast forward kernel tests a lane's sum of sixteen new probabilities instead of their maximum.
constexpr float kSumTrigger = 1024.0f;

template <int DP, int BKV>
struct FwdLayout {
  static constexpr int KLD = DP + 8;    // K tile row pitch: conflict-free 16-byte row reads
  static constexpr int VLD = DP + 32;   // V tile row pitch: conflict-free transposing reads
  static constexpr int K_ELEMS = BKV * KLD;
  static constexpr int V_ELEMS = BKV * VLD;
  static constexpr int STAGE_ELEMS = K_ELEMS + V_ELEMS;
  static constexpr int PATCH_ELEMS = kFwdWaves * 32 * (DP + 8);
  static constexpr int TOTAL_ELEMS =
      (2 * STAGE_ELEMS > PATCH_ELEMS) ? 2 * STAGE_ELEMS : PATCH_ELEMS;
};

// One key/value tile for one wave: S^T = K Q^T, online softmax, O^T += V^T P^T.
// MASKED tiles apply the causal and key-length masks element by element.
template <typename T, int DP, int BKV, bool MASKED>
__device__ __forceinline__ void fwd_tile(const short *sk, const short *sv, const s16x8 (&qf)[DP / 16],
                                         f32x16 (&oacc)[DP / 32], float &m_ref, float &l_run,
                                         float scale_log2, int kvt, int qrow, int seqlen_k,
                                         int k_frag_off, int v_frag_off) {
  using L = FwdLayout<DP, BKV>;
  constexpr int KS = DP / 16, DB = DP / 32, MB = BKV / 32, KS2 = BKV / 16;
  const int h = (threadIdx.x >> 5) & 1;

  f32x16 s[MB];
#pragma unroll
  for (int mb = 0; mb < MB; mb++) {
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    s[mb] = zero;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      s16x8 a = *reinterpret_cast<const s16x8 *>(sk + k_frag_off + 32 * mb * L::KLD + 16 * ks);
      s[mb] = Elem<T>::mfma(a, qf[ks], s[mb]);
    }
  }
  if (MASKED) {
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int kv = kvt + 32 * mb + 8 * (i >> 2) + 4 * h + (i & 3);
        if (kv > qrow || kv >= seqlen_k) s[mb][i] = -INFINITY;
      }
  }

  float mloc = s[0][0];
#pragma unroll
  for (int mb = 0; mb < MB; mb++)
#pragma unroll
    for (int i = 0; i < 16; i++) mloc = fmaxf(mloc, s[mb][i]);
  mloc = max_over_halves(mloc);

  // Raise the reference maximum only when some row needs it (wave-uniform branch).
  const bool grow = (mloc - m_ref) * scale_log2 > kRescaleSlack;  // true on the first tile (m_ref = -inf)
  if (__builtin_amdgcn_ballot_w64(grow) != 0) {
    const float m_new = fmaxf(m_ref, mloc);
    // Every query column of a processed tile sees at least key kvt, so m_new is finite.
    const float alpha = fast_exp2((m_ref - m_new) * scale_log2);
    m_ref = m_new;
    l_run *= alpha;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
  }
  const float mc = m_ref * scale_log2;

  s16x8 pf[KS2];
#pragma unroll
  for (int mb = 0; mb < MB; mb++) {
    f32x16 e;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      e[i] = fast_exp2(s[mb][i] * scale_log2 - mc);
      l_run += e[i];
    }
    f32x8 lo = {e[0], e[1], e[2], e[3], e[4], e[5], e[6], e[7]};
    f32x8 hi = {e[8], e[9], e[10], e[11], e[12], e[13], e[14], e[15]};
    pf[2 * mb] = Elem<T>::pack8(lo);
    pf[2 * mb + 1] = Elem<T>::pack8(hi);
  }

#pragma unroll
  for (int ks2 = 0; ks2 < KS2; ks2++) {
#pragma unroll
    for (int db = 0; db < DB; db++) {
      s16x8 a = lds_read_tr_frag(sv + v_frag_off + 16 * ks2 * L::VLD + 32 * db, L::VLD);
      oacc[db] = Elem<T>::mfma(a, pf[ks2], oacc[db]);
    }
  }
}

template <typename T, int DP, int BKV, bool VEC>
__global__ __launch_bounds__(64 * kFwdWaves, (DP <= 128 ? 2 : 1)) void fwd_kernel(const FwdParams p) {
  using L = FwdLayout<DP, BKV>;
  constexpr int KS = DP / 16;    // k-steps of Q K^T
  constexpr int DB = DP / 32;    // 32-row blocks of O^T
  constexpr int CPR = DP / 8;    // 16-byte chunks per tile row
  constexpr int NTHREADS = 64 * kFwdWaves;
  constexpr int CPT = (BKV * CPR) / NTHREADS;  // chunks per thread per tile
  static_assert((BKV * CPR) % NTHREADS == 0, "tile must split evenly over the workgroup");

  __shared__ __attribute__((aligned(16))) short smem[L::TOTAL_ELEMS];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, g2 = (lane >> 4) & 1;

  // Workgroup -> (batch*head, query tile).  Consecutive workgroup ids go to different XCDs, so
  // taking the head from id % BH keeps every tile of one head on one XCD's L2 when BH % 8 == 0;
  // query tiles are issued heaviest (longest key range) first.
  const int BH = p.batch * p.nheads;
  int bh, rank;
  map_workgroup(blockIdx.x, BH, p.n_qtiles, p.head_group, bh, rank);
  const int qt = p.n_qtiles - 1 - rank;  // the last query tile sees the most keys
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const int q0 = qt * kFwdBlockQ;
  const int q0w = q0 + 32 * wave;

  const short *Q = (const short *)p.q.ptr + b * p.q.stride_batch + hd * p.q.stride_head;
  const short *K = (const short *)p.k.ptr + b * p.k.stride_batch + hd * p.k.stride_head;
  const short *V = (const short *)p.v.ptr + b * p.v.stride_batch + hd * p.v.stride_head;
  short *O = (short *)p.o.ptr + b * p.o.stride_batch + hd * p.o.stride_head;
  float *LSE = p.lse + (int64_t)bh * p.seqlen_q_rounded;

  // Q^T fragments (B operand of S^T = K Q^T): lane (c, h) holds Q[q0w + c][16 ks + 8 h + j].
  s16x8 qf[KS];
  {
    const int row = q0w + c;
    const bool ok = row < p.seqlen_q;
    const short *rp = Q + (int64_t)row * p.q.stride_seq;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = load_chunk(rp, 16 * ks + 8 * h, p.headdim, ok, VEC);
  }

  const int kv_end = min(q0 + kFwdBlockQ, p.seqlen_k);
  const int n_tiles = (kv_end + BKV - 1) / BKV;
  // Leading tiles that lie entirely at or below this wave's first query row and inside the key
  // range need no mask; tiles starting beyond the wave's last row are skipped.
  const int n_full = max(0, min(min(q0w + 1, p.seqlen_k) / BKV, n_tiles));

  s16x8 kreg[CPT], vreg[CPT];
  auto load_tile = [&](int kvt) {
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      const int id = tid + NTHREADS * i;
      const int r = id / CPR, cc = id % CPR;
      const int kv = kvt + r;
      const bool ok = kv < p.seqlen_k;
      kreg[i] = load_chunk(K + (int64_t)kv * p.k.stride_seq, cc * 8, p.headdim, ok, VEC);
      vreg[i] = load_chunk(V + (int64_t)kv * p.v.stride_seq, cc * 8, p.headdim, ok, VEC);
    }
  };
  auto store_tile = [&](int buf) {
    short *sk = smem + buf * L::STAGE_ELEMS;
    short *sv = sk + L::K_ELEMS;
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      const int id = tid + NTHREADS * i;
      const int r = id / CPR, cc = id % CPR;
      *reinterpret_cast<s16x8 *>(sk + r * L::KLD + cc * 8) = kreg[i];
      *reinterpret_cast<s16x8 *>(sv + r * L::VLD + cc * 8) = vreg[i];
    }
  };

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;
  float m_ref = -INFINITY;  // maximum (raw, unscaled scores) the probabilities are formed against
  float l_run = 0.f;        // this lane's share of the running sum (its half of the key rows)

  load_tile(0);
  store_tile(0);
  __syncthreads();

  // Per-lane LDS offsets that do not depend on the tile.
  const int k_frag_off = c * L::KLD + 8 * h;                                       // + 32mb*KLD + 16ks
  const int v_frag_off = (4 * h + (i16 >> 2)) * L::VLD + 16 * g2 + 4 * (i16 & 3);  // + 16ks2*VLD + 32db
  const int qrow = q0w + c;

  for (int t = 0; t < n_tiles; t++) {
    const int buf = t & 1;
    const int kvt = t * BKV;
    const bool more = (t + 1) < n_tiles;
    if (more) load_tile(kvt + BKV);

    const short *sk = smem + buf * L::STAGE_ELEMS;
    const short *sv = sk + L::K_ELEMS;
    if (t < n_full) {
      fwd_tile<T, DP, BKV, false>(sk, sv, qf, oacc, m_ref, l_run, p.scale_log2, kvt, qrow,
                                  p.seqlen_k, k_frag_off, v_frag_off);
    } else if (kvt <= q0w + 31) {
      fwd_tile<T, DP, BKV, true>(sk, sv, qf, oacc, m_ref, l_run, p.scale_log2, kvt, qrow,
                                 p.seqlen_k, k_frag_off, v_frag_off);
    }

    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  // Epilogue: normalise, write lse and O.
  const float l_tot = sum_over_halves(l_run);
  const float inv_l = 1.f / l_tot;
  if (h == 0 && q0w + c < p.seqlen_q) LSE[q0w + c] = m_ref * p.scale + __logf(l_tot);
  if (qt == p.n_qtiles - 1) {
    for (int r = p.seqlen_q + tid; r < p.seqlen_q_rounded; r += NTHREADS) LSE[r] = 0.f;
  }
  // All waves passed the loop's final barrier, so the K/V stages are free to reuse.
  short *patch = smem + wave * 32 * (DP + 8);
  store_transposed_acc<T, DP>(oacc, inv_l, patch, O + (int64_t)q0w * p.o.stride_seq,
                              p.o.stride_seq, p.seqlen_q - q0w, p.headdim, VEC);
}

// ------------------------------------------------------------------------------------------
// Fast path: 16-byte aligned rows and a head dimension that is a multiple of 8; instantiated for 32,
// 64, 96, 128, 192 and 256 columns (two workgroups or more per CU up to 128; at 192 and 256 the
// five tile stages fill the CU's 160 KiB of LDS and the output accumulator moves into accumulation
// registers: one workgroup per CU, one wave per SIMD).
//
//  * K and V tiles (64 rows) go straight from global memory into swizzled, unpadded LDS
//    (global_load_lds_dwordx4: no staging registers, no LDS stores); three K stages and two V
//    stages, one workgroup barrier per tile.
//  * The work is software-pipelined over 32-key blocks so that every MFMA has independent
//    vector work of the same wave next to it (about four VALU instructions issue for free under
//    a 32x32x16 MFMA, and short alternating phases are also what lets two waves of one SIMD
//    overlap).  For block j:
//        X(j): S_{j+1}^T = K_{j+1} Q^T   interleaved with   packing P_j for the MFMA
//        Y(j): O^T += V_j^T P_j^T         interleaved with   P_{j+1} = exp2(scale*S_{j+1} - m), row sums
//    One score buffer and one probability buffer are enough: each is consumed in the phase after
//    the one that fills it.
//  * MFMA operand fragments travel through a ring of DP/16 register sets that is refilled as it
//    is consumed (K fragments of block j+2 during Y(j), V fragments of block j during X(j)), so
//    LDS latency hides behind the MFMAs.
// ------------------------------------------------------------------------------------------
template <int DP, int BKV>
struct FwdDirectLayout {
  static constexpr int LP = lds_pitch(DP);  // LDS row pitch
  static constexpr int TILE_ELEMS = BKV * LP;
  static constexpr int K_STAGES = 3, V_STAGES = 2;
  static constexpr int K_BASE = 0;
  static constexpr int V_BASE = K_STAGES * TILE_ELEMS;
  static constexpr int STAGE_ELEMS = (K_STAGES + V_STAGES) * TILE_ELEMS;
  static constexpr int PATCH_ELEMS = kFwdWaves * 32 * (DP + 8);
  static constexpr int TOTAL_ELEMS = (STAGE_ELEMS > PATCH_ELEMS) ? STAGE_ELEMS : PATCH_ELEMS;
};



// Which half of a 64-row tile a step works on, and whether the step is known to lie well inside
// the wave's key range (no block-count tests needed).
template <int HALF, bool INNER>
struct HalfTag {
  static constexpr int value = HALF;
  static constexpr bool inner = INNER;
};

// PAD: the head dimension is a multiple of 8 below DP; the columns beyond it are zeros in LDS and in
// the register fragments, and are not stored.
// PRE: the Q fragments are multiplied by scale * log2(e) and rounded to half precision once, and
// every score chain starts from minus the maximum in use (the MFMA's C operand), so that the score
// MFMAs deliver the base-2 exponents themselves and no multiply-add is left in front of the
// exponentials.
template <typename T, int DP, int BKV, bool PAD, bool PRE>
__global__ __launch_bounds__(64 * kFwdWaves, (DP <= 128 ? 2 : 1)) void fwd_direct_kernel(const FwdParams p) {
  using L = FwdDirectLayout<DP, BKV>;
  constexpr int KS = DP / 16, DB = DP / 32, LP = L::LP;
  constexpr int NTHREADS = 64 * kFwdWaves;
  constexpr int BLK = 32;  // keys per pipeline block
  static_assert(BKV == 2 * BLK && KS == 2 * DB, "schedule is written for 64-row tiles of two blocks");
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

  __shared__ __attribute__((aligned(1024))) short smem[L::TOTAL_ELEMS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in an SGPR
  const int c = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, g2 = (lane >> 4) & 1;

  const int BH = p.batch * p.nheads;
  int bh, rank;
  map_workgroup(blockIdx.x, BH, p.n_qtiles, p.head_group, bh, rank);
  const int qt = p.n_qtiles - 1 - rank;  // the last query tile sees the most keys
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const int q0 = qt * kFwdBlockQ;
  const int q0w = q0 + 32 * wave;

  const short *Q = (const short *)p.q.ptr + b * p.q.stride_batch + hd * p.q.stride_head;
  const short *K = (const short *)p.k.ptr + b * p.k.stride_batch + hd * p.k.stride_head;
  const short *V = (const short *)p.v.ptr + b * p.v.stride_batch + hd * p.v.stride_head;
  short *O = (short *)p.o.ptr + b * p.o.stride_batch + hd * p.o.stride_head;
  float *LSE = p.lse + (int64_t)bh * p.seqlen_q_rounded;

  const int hdim = PAD ? p.headdim : DP;
  const TileLoader<DP, BKV, kFwdWaves, PAD> kload(K, p.k.stride_seq, hdim / 8), vload(V, p.v.stride_seq, hdim / 8);
  const int seqlen_k = p.seqlen_k;
  const float scale_log2 = p.scale_log2;

  const int kv_end = min(q0 + kFwdBlockQ, seqlen_k);
  const int n_tiles = (kv_end + BKV - 1) / BKV;
  // Blocks this wave multiplies: those that exist and start at or before its last query row.
  const int n_mine = min((kv_end + BLK - 1) / BLK, q0w / BLK + 1);
  // Leading blocks that need no mask (entirely at or below the wave's first row, inside the keys).
  const int n_full = min(q0w + 1, seqlen_k) / BLK;
  const int n_inside = seqlen_k / BKV;  // tiles whose every row exists

  const unsigned lds_base = lds_u32(smem);  // LDS byte address of smem
  if (PAD) {
    zero_lds<NTHREADS>(smem, L::STAGE_ELEMS);
    __syncthreads();
  }
  auto issue_k = [&](int t) {
    const unsigned dst = lds_base + 2u * (unsigned)(L::K_BASE + (t % L::K_STAGES) * L::TILE_ELEMS);
    if (t < n_inside) kload.issue(t * BKV, dst); else kload.issue_clamped(t * BKV, seqlen_k, dst);
  };
  auto issue_v = [&](int t) {
    const unsigned dst = lds_base + 2u * (unsigned)(L::V_BASE + (t % L::V_STAGES) * L::TILE_ELEMS);
    if (t < n_inside) vload.issue(t * BKV, dst); else vload.issue_clamped(t * BKV, seqlen_k, dst);
  };
  // K_0, the workgroup's Q rows, V_0 and K_1 are loaded here; after that tile t brings in K_{t+2}
  // and V_{t+1}.  The Q rows travel like a K tile: coalesced LDS-direct loads (a wave-load covers
  // whole rows) into the two stages nothing else uses yet, query rows 0..63 of the workgroup in
  // the third K stage and 64..127 in the second V stage, from where every wave reads its
  // fragments.  Loaded straight into registers, a wave's fragment loads touch 32 different rows
  // each, eight times over, and keep the CU's address path busy for a microsecond per workgroup.
  // Rows beyond the sequence are read from its last row: finite values whose results are never stored.
  constexpr unsigned Q_LO = 2u * (unsigned)(L::K_BASE + 2 * L::TILE_ELEMS);
  constexpr unsigned Q_HI = 2u * (unsigned)(L::V_BASE + 1 * L::TILE_ELEMS);
  const TileLoader<DP, BKV, kFwdWaves, PAD> qload(Q + (int64_t)q0 * p.q.stride_seq, p.q.stride_seq, hdim / 8);
  const int q_rows = p.seqlen_q - q0;  // rows of this query tile that exist (>= 1)
  issue_k(0);
  if (q_rows >= BKV) qload.issue(0, lds_base + Q_LO); else qload.issue_clamped(0, q_rows, lds_base + Q_LO);
  if (q_rows >= 2 * BKV) qload.issue(BKV, lds_base + Q_HI); else qload.issue_clamped(BKV, q_rows, lds_base + Q_HI);
  issue_v(0);
  if (n_tiles > 1) issue_k(1);

  // Fragment addresses (swizzled, 32-bit LDS pointers).  kcur points into the stage of the K tile
  // after the current one, vcur into the stage of the current V tile; both advance by a uniform
  // amount per tile, and half-tile offsets are immediates.
  lds_cptr kcur[KS], vlo[DB], vhi[DB];
  const lds_cptr lds0 = to_lds(smem);
#pragma unroll
  for (int ks = 0; ks < KS; ks++) kcur[ks] = lds0 + L::K_BASE + swz_off<LP>(c, 2 * ks + h);
  {
    const int rowlo = 4 * h + (i16 >> 2);
    const int sub = (i16 & 1) * 4;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      const int chunk = 4 * db + 2 * g2 + ((i16 & 3) >> 1);
      vlo[db] = lds0 + L::V_BASE + swz_off<LP>(rowlo, chunk) + sub;
      vhi[db] = lds0 + L::V_BASE + swz_off<LP>(rowlo + 8, chunk) + sub;
    }
  }
  // K fragment ks of the half-tile `half` of the tile kcur points at.
  auto k_frag = [&](int half, int ks) { return lds_read_128(kcur[ks] + half * BLK * LP); };
  // V^T fragment (k-step ks2 in {0,1} of half-tile `half`, head-dim block db) of the tile vcur points at.
  auto v_frag = [&](int half, int ks2, int db) -> s16x8 {
    s16x4 lo = lds_read_tr(vlo[db] + half * BLK * LP + 16 * ks2 * LP);
    s16x4 hi = lds_read_tr(vhi[db] + half * BLK * LP + 16 * ks2 * LP);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;
  float m_ref = -INFINITY;  // maximum the probabilities are formed against (raw scores; PRE: base-2 exponents)
  float l_run = 0.f;        // this lane's share of the running sum (its half of the key rows)
  const int qrow = q0w + c;
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  auto apply_mask = [&](f32x16 &s, int kv0) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int kv = kv0 + 8 * (i >> 2) + 4 * h + (i & 3);
      if (kv > qrow || kv >= seqlen_k) s[i] = -INFINITY;
    }
  };
  auto row_max = [&](const f32x16 &s) {
    float m = s[0];
#pragma unroll
    for (int i = 1; i < 16; i++) m = fmaxf(m, s[i]);
    return max_over_halves(m);
  };
  // K_0 and Q have landed once at most the loads of V_0 (and K_1) are outstanding: loads complete
  // in the order they were issued.
  constexpr int LOADS_PER_TILE = TileLoader<DP, BKV, kFwdWaves, PAD>::LOADS;
  static_assert(2 * LOADS_PER_TILE < 64, "vmcnt field");
  if (n_tiles > 1) wait_vmem<2 * LOADS_PER_TILE>(); else wait_vmem<LOADS_PER_TILE>();
  __syncthreads();

  // Q^T fragments (B operand of S^T = K Q^T): lane (c, h) holds Q[q0w + c][16 ks + 8 h + j].
  s16x8 qf[KS];
  {
    const lds_cptr qrows = lds0 + ((wave >> 1) ? (int)(Q_HI / 2) : (int)(Q_LO / 2));
    const int r = 32 * (wave & 1) + c;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = lds_read_128(qrows + swz_off<LP>(r, 2 * ks + h));
    if (PRE) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) qf[ks] = scale8<T>(qf[ks], scale_log2);
    }
  }

  // ---- prologue: S_0, its row maximum, e_0 = exp2(scale*S_0 - scale*m), ring <- K fragments of
  // block 1 ---------------------------------------------------------------------------------
  s16x8 ring[KS];
  f32x16 sc;  // the score block in flight (S_{j+1} during step j)
  f32x16 e;   // unnormalised probabilities of the block whose P V product comes next
  {
#pragma unroll
    for (int ks = 0; ks < KS; ks++) ring[ks] = k_frag(0, ks);
    sc = zero;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) sc = Elem<T>::mfma(ring[ks], qf[ks], sc);
    if (0 >= n_full) apply_mask(sc, 0);
    m_ref = row_max(sc);  // finite: every query row sees key 0
    const float mc = m_ref * scale_log2;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      e[i] = PRE ? fast_exp2(sc[i] - m_ref) : fast_exp2(sc[i] * scale_log2 - mc);
      l_run += e[i];
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) ring[ks] = k_frag(1, ks);
    // From here on kcur addresses K tile 1 (the tile after the current one).
#pragma unroll
    for (int ks = 0; ks < KS; ks++) kcur[ks] += L::TILE_ELEMS;
  }
  // V_0 and K_1 have landed, and every wave has taken its Q fragments out of the two stages that
  // the first tile's loads (K_2, V_1) are about to overwrite.
  wait_vmem_all();
  __syncthreads();

  // PRE: the C operand every later score chain starts from.
  f32x16 negm = zero;
  if (PRE) negm = splat16(-m_ref);

  // One block step.  On entry e holds the probabilities of block j (formed against m_ref) and the
  // ring the K fragments of block j+1.
  //     X: S_{j+1}^T = K_{j+1} Q^T   beside   pack P_j                                  ring <- V_j^T
  //     Y: O^T += V_j^T P_j^T        beside   exponentials of S_{j+1} and their row sums   ring <- K_{j+2}
  // The exponentials, which do not overlap with MFMAs of their own wave and are the most expensive
  // vector instructions here, sit in the phase whose MFMAs need the fewest LDS reads, which evens
  // out the two phases.  HALF (= j & 1) selects the half-tile: V_j is half HALF of the current V
  // tile and K_{j+2} is half HALF of the next K tile.
  //
  // The step is hand-interleaved: each unit is one MFMA, the LDS reads that refill the ring slot
  // it just freed, and a few vector instructions; a scheduling fence after every unit keeps the
  // compiler from regrouping them (which would lengthen live ranges past the register file).
  // S_{j+1} and the K fragments of block j+2 are produced even when those blocks are not this
  // wave's (the values are then never used), so that there is a single code path.
  //
  // The new probabilities are formed against the maximum in use; if S_{j+1} turns out to exceed
  // it by more than the slack (rare once the maximum has settled), the running state is rescaled
  // after the step's MFMAs and the probabilities are formed again.
  //
  // Tile loads (SPREAD): the global->LDS loads of K tile t+2 and V tile t+1 are issued one at a
  // time between the units of tile t's first step.  Issued back to back by all waves at once they
  // queue up in the memory pipeline, and a wave whose load cannot issue cannot issue its MFMAs
  // either.
  constexpr int LOADS = TileLoader<DP, BKV, kFwdWaves, PAD>::LOADS;
  constexpr int LOAD_EVERY = KS / LOADS;
  auto step = [&](int j, auto half_tag, auto spread_tag) {
    constexpr int HALF = decltype(half_tag)::value;
    constexpr bool SPREAD = decltype(spread_tag)::value;
    // SPREAD steps and the step after them lie at least two tiles before the wave's diagonal:
    // blocks j and j + 1 are always the wave's own there, and the tests below fold away.
    constexpr bool INNER = decltype(spread_tag)::value || decltype(half_tag)::inner;
    if (!INNER && j >= n_mine) {
      if (SPREAD) {  // not reached: the skipped blocks lie in the last two tiles, which load nothing
        issue_k(j / 2 + 2);
        issue_v(j / 2 + 1);
      }
      return;
    }
    const int kt = j / 2 + 2, vt = j / 2 + 1;  // tiles loaded during this step (SPREAD)
    const unsigned kdst = lds_base + 2u * (unsigned)(L::K_BASE + (kt % L::K_STAGES) * L::TILE_ELEMS);
    const unsigned vdst = lds_base + 2u * (unsigned)(L::V_BASE + (vt % L::V_STAGES) * L::TILE_ELEMS);
    typedef unsigned u32x4v __attribute__((ext_vector_type(4)));
    u32x4v w[2];  // packed probabilities, two per word: w[0] = k-step 0, w[1] = k-step 1
    if (!PRE) sc = zero;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      sc = Elem<T>::mfma(ring[ks], qf[ks], (PRE && ks == 0) ? negm : sc);
      if (SPREAD && ks % LOAD_EVERY == 0 && ks / LOAD_EVERY < LOADS) vload.issue_one(vt * BKV, vdst, ks / LOAD_EVERY);
      ring[ks] = v_frag(HALF, ks / DB, ks % DB);
#pragma unroll
      for (int i = part(8, KS, ks); i < part(8, KS, ks + 1); i++)  // probability pair (2i, 2i+1) of the block
        w[i / 4][i % 4] = Elem<T>::pack2(e[2 * i], e[2 * i + 1]);
      // Pin the arithmetic to this unit: without a use here the optimiser sinks it next to the
      // MFMAs that consume it.
      if (ks == KS / 2 - 1) asm volatile("" : "+v"(w[0]));
      if (ks == KS - 1) asm volatile("" : "+v"(w[1]));
      __builtin_amdgcn_sched_barrier(0);
    }
    // S_{j+1} of a SPREAD step is the second half of a tile that ends before the workgroup's first
    // query row: never masked.  (The step after it may produce the first block of the diagonal.)
    if (!SPREAD && j + 1 >= n_full) apply_mask(sc, (j + 1) * BLK);
    const s16x8 pf[2] = {__builtin_bit_cast(s16x8, w[0]), __builtin_bit_cast(s16x8, w[1])};
    const float mc = m_ref * scale_log2;
    float lsum[2] = {0.f, 0.f};  // this lane's sum of the new probabilities, in two chains
#pragma unroll
    for (int ks2 = 0; ks2 < 2; ks2++) {
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const int slot = ks2 * DB + db;
        oacc[db] = Elem<T>::mfma(ring[slot], pf[ks2], oacc[db]);
        if (SPREAD && slot % LOAD_EVERY == 0 && slot / LOAD_EVERY < LOADS) kload.issue_one(kt * BKV, kdst, slot / LOAD_EVERY);
        ring[slot] = k_frag(HALF, slot);
#pragma unroll
        for (int i = part(16, KS, slot); i < part(16, KS, slot + 1); i++) {
          e[i] = PRE ? fast_exp2(sc[i]) : fast_exp2(sc[i] * scale_log2 - mc);
          lsum[i & 1] += e[i];
        }
        asm volatile("" : "+v"(lsum[0]), "+v"(lsum[1]));
        asm volatile("" : "+v"(e));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (INNER || j + 1 < n_mine) {
      // No maximum is taken on this path: a lane's sum of sixteen probabilities bounds each of
      // them, so a sum above kSumTrigger (or one that overflowed to +inf) is what sends the wave
      // to the rescale below.
      float lblk = lsum[0] + lsum[1];
      const bool grow = !(lblk <= kSumTrigger);
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        // PRE: sc holds the exponents relative to m_ref; raise m_ref by the largest positive excess.
        const float up = fmaxf(row_max(sc), 0.f);
        const float m_new = PRE ? m_ref + up : fmaxf(m_ref, row_max(sc));
        const float alpha = PRE ? fast_exp2(-up) : fast_exp2((m_ref - m_new) * scale_log2);
        m_ref = m_new;
        if (PRE) negm = splat16(-m_ref);
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
        const float mc2 = m_new * scale_log2;
        lblk = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          e[i] = PRE ? fast_exp2(sc[i] - up) : fast_exp2(sc[i] * scale_log2 - mc2);
          lblk += e[i];
        }
      }
      l_run += lblk;
    }
  };

  // End of a tile: every wave is done with V_t and the K fragments of tile t+1 are in flight or
  // in registers; K_{t+2} and V_{t+1} (issued during this tile) have landed.  Then the fragment
  // pointers advance to K tile t+2 and V tile t+1 (stages are used round-robin).
  auto end_tile = [&](int t) {
    wait_vmem_all();
    tile_barrier();
    const int dk = ((t + 2) % L::K_STAGES == 0) ? -(L::K_STAGES - 1) * L::TILE_ELEMS : L::TILE_ELEMS;
    const int dv = ((t + 1) % L::V_STAGES == 0) ? -(L::V_STAGES - 1) * L::TILE_ELEMS : L::TILE_ELEMS;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) kcur[ks] += dk;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      vlo[db] += dv;
      vhi[db] += dv;
    }
  };
  int t = 0;
  // Tiles whose loads are whole tiles inside the keys: spread over the first step.
  const int n_spread = min(n_tiles, n_inside) - 2;
  for (; t < n_spread; t++) {
    step(2 * t, HalfTag<0, true>{}, std::true_type{});
    step(2 * t + 1, HalfTag<1, true>{}, std::false_type{});
    end_tile(t);
  }
  // The last tiles: whatever is left to load (possibly a ragged tile) is issued at once.
  for (; t < n_tiles; t++) {
    if (t + 2 < n_tiles) issue_k(t + 2);
    if (t + 1 < n_tiles) issue_v(t + 1);
    step(2 * t, HalfTag<0, false>{}, std::false_type{});
    step(2 * t + 1, HalfTag<1, false>{}, std::false_type{});
    end_tile(t);
  }
  const float l_tot = sum_over_halves(l_run);
  const float inv_l = 1.f / l_tot;
  if (h == 0 && q0w + c < p.seqlen_q) LSE[q0w + c] = m_ref * (PRE ? kLn2 : p.scale) + __logf(l_tot);
  if (qt == p.n_qtiles - 1) {
    for (int r = p.seqlen_q + tid; r < p.seqlen_q_rounded; r += NTHREADS) LSE[r] = 0.f;
  }
  // The patch overlays the stages; the loop's last barrier already ordered it after all reads.
  short *patch = smem + wave * 32 * (DP + 8);
  store_transposed_acc<T, DP>(oacc, inv_l, patch, O + (int64_t)q0w * p.o.stride_seq,
                              p.o.stride_seq, p.seqlen_q - q0w, hdim, true);
}

}  // namespace fa2
