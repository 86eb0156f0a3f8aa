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
//  * K and V tiles are double-buffered in LDS; the next tile's global loads are in flight while
//    the current tile is being multiplied.
//  * Unlike the reference (mask applied to every tile, lines 139-147) the mask is evaluated only
//    on tiles that touch the diagonal or the end of the key sequence, and sub-blocks entirely
//    above the diagonal are skipped.
//  * The running maximum `m` is the usual one; the reference floors it with the running lse
//    (line 150), which only changes rounding.
#pragma once

#include "fa2_common.cuh"

namespace fa2 {

struct FwdParams {
  Tensor4 q, k, v, o;
  float *lse;
  int batch, nheads, seqlen_q, seqlen_k, headdim, seqlen_q_rounded;
  int n_qtiles;
  float scale;       // softmax scale (natural units)
  float scale_log2;  // scale * log2(e)
  int vec;           // 16-byte global accesses are legal for every tensor
};

constexpr int kFwdWaves = 4;
constexpr int kFwdBlockQ = 32 * kFwdWaves;

template <int DP, int BKV>
struct FwdLayout {
  static constexpr int KLD = DP + 8;   // K tile row pitch: conflict-free 16-byte row reads
  static constexpr int VLD = DP + 8;   // V tile row pitch (read with transposing loads)
  static constexpr int K_ELEMS = BKV * KLD;
  static constexpr int V_ELEMS = BKV * VLD;
  static constexpr int STAGE_ELEMS = K_ELEMS + V_ELEMS;
  static constexpr int PATCH_ELEMS = kFwdWaves * 32 * (DP + 8);
  static constexpr int TOTAL_ELEMS =
      (2 * STAGE_ELEMS > PATCH_ELEMS) ? 2 * STAGE_ELEMS : PATCH_ELEMS;
};

template <typename T, int DP, int BKV>
__global__ __launch_bounds__(64 * kFwdWaves, 2) void fwd_kernel(const FwdParams p) {
  using L = FwdLayout<DP, BKV>;
  constexpr int KS = DP / 16;    // k-steps of Q K^T
  constexpr int DB = DP / 32;    // 32-row blocks of O^T
  constexpr int MB = BKV / 32;   // 32-row blocks of S^T
  constexpr int KS2 = BKV / 16;  // k-steps of P V
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
  const int bh = blockIdx.x % BH;
  const int qt = p.n_qtiles - 1 - blockIdx.x / BH;
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const int q0 = qt * kFwdBlockQ;
  const int q0w = q0 + 32 * wave;
  const bool vec = p.vec != 0;

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
    for (int ks = 0; ks < KS; ks++) qf[ks] = load_chunk(rp, 16 * ks + 8 * h, p.headdim, ok, vec);
  }

  const int kv_end = min(q0 + kFwdBlockQ, p.seqlen_k);
  const int n_tiles = (kv_end + BKV - 1) / BKV;

  s16x8 kreg[CPT], vreg[CPT];
  auto load_tile = [&](int kvt) {
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      const int id = tid + NTHREADS * i;
      const int r = id / CPR, cc = id % CPR;
      const int kv = kvt + r;
      const bool ok = kv < p.seqlen_k;
      kreg[i] = load_chunk(K + (int64_t)kv * p.k.stride_seq, cc * 8, p.headdim, ok, vec);
      vreg[i] = load_chunk(V + (int64_t)kv * p.v.stride_seq, cc * 8, p.headdim, ok, vec);
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
  float m_run = -INFINITY;  // running max of the raw (unscaled) scores of this lane's query
  float l_run = 0.f;        // this lane's share of the running sum (its half of the key rows)

  load_tile(0);
  store_tile(0);
  __syncthreads();

  // Per-lane LDS offsets that do not depend on the tile.
  const int k_frag_off = c * L::KLD + 8 * h;                                  // + 32mb*KLD + 16ks
  const int v_frag_off = (4 * h + (i16 >> 2)) * L::VLD + 16 * g2 + 4 * (i16 & 3);  // + 16ks2*VLD + 32db

  for (int t = 0; t < n_tiles; t++) {
    const int buf = t & 1;
    const int kvt = t * BKV;
    const bool more = (t + 1) < n_tiles;
    if (more) load_tile(kvt + BKV);

    // Key sub-blocks (32 rows) of this tile that reach this wave's query range at all.
    int nact = (q0w + 31 - kvt) / 32 + 1;
    nact = (q0w + 31 < kvt) ? 0 : min(nact, MB);

    if (nact > 0) {
      const short *sk = smem + buf * L::STAGE_ELEMS;
      const short *sv = sk + L::K_ELEMS;

      f32x16 s[MB];
#pragma unroll
      for (int mb = 0; mb < MB; mb++) {
#pragma unroll
        for (int i = 0; i < 16; i++) s[mb][i] = 0.f;
        if (mb < nact) {
#pragma unroll
          for (int ks = 0; ks < KS; ks++) {
            s16x8 a = *reinterpret_cast<const s16x8 *>(sk + k_frag_off + 32 * mb * L::KLD + 16 * ks);
            s[mb] = Elem<T>::mfma(a, qf[ks], s[mb]);
          }
        }
      }

      // Mask: needed when the tile crosses the diagonal of this wave's rows or the key end.
      const bool need_mask = (kvt + 32 * nact - 1 > q0w) || (kvt + 32 * nact > p.seqlen_k);
      if (need_mask) {
        const int qrow = q0w + c;
#pragma unroll
        for (int mb = 0; mb < MB; mb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int kv = kvt + 32 * mb + 8 * (i >> 2) + 4 * h + (i & 3);
            if (kv > qrow || kv >= p.seqlen_k) s[mb][i] = -INFINITY;
          }
      }
#pragma unroll
      for (int mb = 0; mb < MB; mb++)
        if (mb >= nact) {
#pragma unroll
          for (int i = 0; i < 16; i++) s[mb][i] = -INFINITY;
        }

      float mloc = -INFINITY;
#pragma unroll
      for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int i = 0; i < 16; i++) mloc = fmaxf(mloc, s[mb][i]);
      mloc = max_over_halves(mloc);
      const float m_new = fmaxf(m_run, mloc);
      // Every query column of an active tile sees at least key kvt, so m_new is finite here.
      const float mc = m_new * p.scale_log2;
      const float alpha = fast_exp2(m_run * p.scale_log2 - mc);
      m_run = m_new;

      float lsum = 0.f;
      s16x8 pf[KS2];
#pragma unroll
      for (int mb = 0; mb < MB; mb++) {
        f32x16 e;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          e[i] = fast_exp2(s[mb][i] * p.scale_log2 - mc);
          lsum += e[i];
        }
        f32x8 lo = {e[0], e[1], e[2], e[3], e[4], e[5], e[6], e[7]};
        f32x8 hi = {e[8], e[9], e[10], e[11], e[12], e[13], e[14], e[15]};
        pf[2 * mb] = Elem<T>::pack8(lo);
        pf[2 * mb + 1] = Elem<T>::pack8(hi);
      }
      l_run = l_run * alpha + lsum;

#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;

#pragma unroll
      for (int ks2 = 0; ks2 < KS2; ks2++) {
        if ((ks2 >> 1) < nact) {
#pragma unroll
          for (int db = 0; db < DB; db++) {
            s16x8 a = lds_read_tr_frag(sv + v_frag_off + 16 * ks2 * L::VLD + 32 * db, L::VLD);
            oacc[db] = Elem<T>::mfma(a, pf[ks2], oacc[db]);
          }
        }
      }
    }

    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  // Epilogue: normalise, write lse and O.
  const float l_tot = sum_over_halves(l_run);
  const float inv_l = 1.f / l_tot;
  if (h == 0 && q0w + c < p.seqlen_q) LSE[q0w + c] = m_run * p.scale + __logf(l_tot);
  if (qt == p.n_qtiles - 1) {
    for (int r = p.seqlen_q + tid; r < p.seqlen_q_rounded; r += NTHREADS) LSE[r] = 0.f;
  }
  // All waves passed the loop's final barrier, so the K/V stages are free to reuse.
  short *patch = smem + wave * 32 * (DP + 8);
  store_transposed_acc<T, DP>(oacc, inv_l, patch, O + (int64_t)q0w * p.o.stride_seq,
                              p.o.stride_seq, p.seqlen_q - q0w, p.headdim, vec);
}

}  // namespace fa2
