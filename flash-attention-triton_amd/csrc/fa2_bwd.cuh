// Causal FlashAttention-2 backward for gfx950.
//
// The reference backward (src/flash_attention_triton/_triton_kernels_v2.py:192-352) walks, for
// one key/value tile j, all query tiles i at or below the diagonal and does
//   S = Q_i K_j^T,  P = exp(scale*S - lse_i),  dP = dO_i V_j^T,  dS = P*(dP - delta_i)*scale,
//   dK_j += dS^T Q_i,  dV_j += P^T dO_i,  dQ_i += dS K_j
// with dQ either atomically added (sequence-parallel) or read-modify-written by a single
// sequential program per head (deterministic).  Here the work is split so that every output is
// owned by exactly one wave and written once:
//
//  * bwd_dkdv_kernel: one workgroup per key/value tile of 128 rows, each of its 4 waves owning 32
//    key columns (K and V fragments stay in registers); Q and dO tiles stream through LDS.
//    S and dP come out of the MFMA with one key column per lane, which is the B-operand layout
//    dV^T = dO^T P and dK^T = Q^T dS need; dO^T and Q^T fragments are fetched from the row-major
//    tiles with the transposing LDS read.
//  * bwd_dq_kernel: one workgroup per query tile of 128 rows, each wave owning 32 query columns
//    (Q and dO fragments in registers); K and V tiles stream through LDS in ascending order.  It
//    recomputes S^T and dP^T and accumulates dQ^T = K^T dS^T in registers, in a fixed order and
//    without atomics, so dQ is bit-reproducible.
//  * bwd_preprocess_kernel: delta = rowsum(O * dO), the reference's
//    _backward_preprocess_do_o_dot (_triton_kernels_v2.py:532-608).
#pragma once

#include <type_traits>

#include "fa2_common.cuh"

namespace fa2 {

struct BwdParams {
  Tensor4 q, k, v, d_o, dq, dk, dv;
  Tensor4 o;         // only read by the dQ kernel when it also forms delta
  float *delta_out;  // where that kernel writes delta (the same buffer `delta` points to)
  const float *lse;
  const float *delta;
  int batch, nheads, seqlen_q, seqlen_k, headdim, seqlen_q_rounded;
  int n_tiles;  // key tiles (dK/dV kernel) or query tiles (dQ kernel)
  float scale, scale_log2;
  int vec;
};

struct PreParams {
  Tensor4 o, d_o;
  float *delta;
  int batch, nheads, seqlen_q, headdim, seqlen_q_rounded;
  int vec;
};

// ------------------------------------------------------------------------------------------
// delta = rowsum(O * dO).  16 lanes per row, 16 rows per workgroup; rows in
// [seqlen_q, seqlen_q_rounded) are written as zero.
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_preprocess_kernel(const PreParams p) {
  const int tid = threadIdx.x;
  const int sub = tid & 15;
  const int row = blockIdx.x * 16 + (tid >> 4);
  const int bh = blockIdx.y;
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const bool vec = p.vec != 0;
  float acc = 0.f;
  if (row < p.seqlen_q) {
    const short *orow = (const short *)p.o.ptr + b * p.o.stride_batch + hd * p.o.stride_head +
                        (int64_t)row * p.o.stride_seq;
    const short *grow = (const short *)p.d_o.ptr + b * p.d_o.stride_batch +
                        hd * p.d_o.stride_head + (int64_t)row * p.d_o.stride_seq;
    for (int d0 = sub * 8; d0 < p.headdim; d0 += 128) {
      s16x8 a = load_chunk(orow, d0, p.headdim, true, vec);
      s16x8 g = load_chunk(grow, d0, p.headdim, true, vec);
#pragma unroll
      for (int j = 0; j < 8; j++) acc += Elem<T>::to_float(a[j]) * Elem<T>::to_float(g[j]);
    }
  }
#pragma unroll
  for (int off = 8; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 16);
  if (sub == 0 && row < p.seqlen_q_rounded)
    p.delta[(int64_t)bh * p.seqlen_q_rounded + row] = acc;
}

// ------------------------------------------------------------------------------------------
// dQ kernel (query-tile parallel, fixed accumulation order).
// ------------------------------------------------------------------------------------------
constexpr int kDqWaves = 4;
constexpr int kDqBlockQ = 32 * kDqWaves;

template <int DP, int BKV>
struct DqLayout {
  static constexpr int KLD = DP + 8;
  static constexpr int VLD = DP + 8;
  static constexpr int K_ELEMS = BKV * KLD;
  static constexpr int V_ELEMS = BKV * VLD;
  static constexpr int STAGE_ELEMS = K_ELEMS + V_ELEMS;
  static constexpr int PATCH_ELEMS = kDqWaves * 32 * (DP + 8);
  static constexpr int TOTAL_ELEMS =
      (2 * STAGE_ELEMS > PATCH_ELEMS) ? 2 * STAGE_ELEMS : PATCH_ELEMS;
};

template <typename T, int DP, int BKV>
__global__ __launch_bounds__(64 * kDqWaves, (DP <= 96 ? 2 : 1)) void bwd_dq_kernel(const BwdParams p) {
  using L = DqLayout<DP, BKV>;
  constexpr int KS = DP / 16, DB = DP / 32, MB = BKV / 32, KS2 = BKV / 16, CPR = DP / 8;
  constexpr int NTHREADS = 64 * kDqWaves;
  constexpr int CPT = (BKV * CPR) / NTHREADS;
  static_assert((BKV * CPR) % NTHREADS == 0, "tile must split evenly over the workgroup");

  __shared__ __attribute__((aligned(16))) short smem[L::TOTAL_ELEMS];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, g2 = (lane >> 4) & 1;

  const int BH = p.batch * p.nheads;
  int bh, rank;
  map_workgroup(blockIdx.x, BH, p.n_tiles, bh, rank);
  const int qt = p.n_tiles - 1 - rank;  // the last query tile sees the most keys
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const int q0 = qt * kDqBlockQ;
  const int q0w = q0 + 32 * wave;
  const bool vec = p.vec != 0;

  const short *Q = (const short *)p.q.ptr + b * p.q.stride_batch + hd * p.q.stride_head;
  const short *K = (const short *)p.k.ptr + b * p.k.stride_batch + hd * p.k.stride_head;
  const short *V = (const short *)p.v.ptr + b * p.v.stride_batch + hd * p.v.stride_head;
  const short *DO = (const short *)p.d_o.ptr + b * p.d_o.stride_batch + hd * p.d_o.stride_head;
  short *DQ = (short *)p.dq.ptr + b * p.dq.stride_batch + hd * p.dq.stride_head;

  // B operands: lane (c, h) holds row q0w + c of Q and of dO, columns 16 ks + 8 h + j.
  s16x8 qf[KS], gf[KS];
  float lse2 = 0.f, delta = 0.f;
  {
    const int row = q0w + c;
    const bool ok = row < p.seqlen_q;
    const short *qp = Q + (int64_t)row * p.q.stride_seq;
    const short *gp = DO + (int64_t)row * p.d_o.stride_seq;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      qf[ks] = load_chunk(qp, 16 * ks + 8 * h, p.headdim, ok, vec);
      gf[ks] = load_chunk(gp, 16 * ks + 8 * h, p.headdim, ok, vec);
    }
    if (ok) {
      lse2 = p.lse[(int64_t)bh * p.seqlen_q_rounded + row] * kLog2e;
      delta = p.delta[(int64_t)bh * p.seqlen_q_rounded + row];
    }
  }

  const int kv_end = min(q0 + kDqBlockQ, p.seqlen_k);
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

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) dqacc[db][i] = 0.f;

  load_tile(0);
  store_tile(0);
  __syncthreads();

  const int row_frag_off = c * L::KLD + 8 * h;  // KLD == VLD
  const int tr_frag_off = (4 * h + (i16 >> 2)) * L::KLD + 16 * g2 + 4 * (i16 & 3);
  static_assert(L::KLD == L::VLD, "shared fragment offsets assume equal pitches");

  for (int t = 0; t < n_tiles; t++) {
    const int buf = t & 1;
    const int kvt = t * BKV;
    const bool more = (t + 1) < n_tiles;
    if (more) load_tile(kvt + BKV);

    int nact = (q0w + 31 - kvt) / 32 + 1;
    nact = (q0w + 31 < kvt) ? 0 : min(nact, MB);

    if (nact > 0) {
      const short *sk = smem + buf * L::STAGE_ELEMS;
      const short *sv = sk + L::K_ELEMS;
      const bool need_mask = (kvt + 32 * nact - 1 > q0w) || (kvt + 32 * nact > p.seqlen_k);
      const int qrow = q0w + c;

      s16x8 dsf[KS2];
#pragma unroll
      for (int mb = 0; mb < MB; mb++) {
        f32x16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          s[i] = 0.f;
          dp[i] = 0.f;
        }
        if (mb < nact) {
#pragma unroll
          for (int ks = 0; ks < KS; ks++) {
            s16x8 a = *reinterpret_cast<const s16x8 *>(sk + row_frag_off + 32 * mb * L::KLD + 16 * ks);
            s = Elem<T>::mfma(a, qf[ks], s);
          }
#pragma unroll
          for (int ks = 0; ks < KS; ks++) {
            s16x8 a = *reinterpret_cast<const s16x8 *>(sv + row_frag_off + 32 * mb * L::VLD + 16 * ks);
            dp = Elem<T>::mfma(a, gf[ks], dp);
          }
        }
        f32x16 ds;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          float pr = fast_exp2(s[i] * p.scale_log2 - lse2);
          if (need_mask) {
            const int kv = kvt + 32 * mb + 8 * (i >> 2) + 4 * h + (i & 3);
            if (kv > qrow || kv >= p.seqlen_k) pr = 0.f;
          }
          ds[i] = pr * (dp[i] - delta);
        }
        if (mb >= nact) {
#pragma unroll
          for (int i = 0; i < 16; i++) ds[i] = 0.f;
        }
        f32x8 lo = {ds[0], ds[1], ds[2], ds[3], ds[4], ds[5], ds[6], ds[7]};
        f32x8 hi = {ds[8], ds[9], ds[10], ds[11], ds[12], ds[13], ds[14], ds[15]};
        dsf[2 * mb] = Elem<T>::pack8(lo);
        dsf[2 * mb + 1] = Elem<T>::pack8(hi);
      }

#pragma unroll
      for (int ks2 = 0; ks2 < KS2; ks2++) {
        if ((ks2 >> 1) < nact) {
#pragma unroll
          for (int db = 0; db < DB; db++) {
            s16x8 a = lds_read_tr_frag(sk + tr_frag_off + 16 * ks2 * L::KLD + 32 * db, L::KLD);
            dqacc[db] = Elem<T>::mfma(a, dsf[ks2], dqacc[db]);
          }
        }
      }
    }

    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  short *patch = smem + wave * 32 * (DP + 8);
  store_transposed_acc<T, DP>(dqacc, p.scale, patch, DQ + (int64_t)q0w * p.dq.stride_seq,
                              p.dq.stride_seq, p.seqlen_q - q0w, p.headdim, vec);
}

// ------------------------------------------------------------------------------------------
// dK/dV kernel (key-tile parallel).
// ------------------------------------------------------------------------------------------
constexpr int kDkvWaves = 4;
constexpr int kDkvBlockKV = 32 * kDkvWaves;

template <int DP, int BQ>
struct DkvLayout {
  static constexpr int QLD = DP + 8;
  static constexpr int Q_ELEMS = BQ * QLD;
  // One stage: Q tile, dO tile, then lse*log2e and delta as floats (2 shorts each).
  static constexpr int STAGE_ELEMS = 2 * Q_ELEMS + 4 * BQ;
  static constexpr int PATCH_ELEMS = kDkvWaves * 32 * (DP + 8);
  static constexpr int TOTAL_ELEMS =
      (2 * STAGE_ELEMS > PATCH_ELEMS) ? 2 * STAGE_ELEMS : PATCH_ELEMS;
};

template <typename T, int DP, int BQ>
__global__ __launch_bounds__(64 * kDkvWaves, 1) void bwd_dkdv_kernel(const BwdParams p) {
  using L = DkvLayout<DP, BQ>;
  constexpr int KS = DP / 16, DB = DP / 32, MQ = BQ / 32, CPR = DP / 8;
  // At 256 columns the two accumulators (2 x 128 registers) no longer fit beside the K and V
  // fragments (another 128): the head dimension is then covered in two passes over the query tiles,
  // each accumulating half of the columns of dK and dV (S and dP are formed again in the second
  // pass).  Measured at B=2, H=8, N=4096: 811 us against 2273 us with one pass and 1 KiB of
  // spills per lane; at 192 columns one pass is the faster (295 us against 640 us).
  constexpr int NPASS = DP > 192 ? 2 : 1;
  constexpr int DBP = DB / NPASS;  // 32-column blocks of dK / dV per pass
  static_assert(DB % NPASS == 0, "passes must split the head dimension evenly");
  constexpr int NTHREADS = 64 * kDkvWaves;
  constexpr int CPT = (BQ * CPR) / NTHREADS;
  static_assert((BQ * CPR) % NTHREADS == 0, "tile must split evenly over the workgroup");
  static_assert(BQ <= NTHREADS, "one thread per row loads lse and delta");

  __shared__ __attribute__((aligned(16))) short smem[L::TOTAL_ELEMS];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, g2 = (lane >> 4) & 1;

  // Key tile 0 has the longest query range: issue tiles in ascending order (heaviest first).
  const int BH = p.batch * p.nheads;
  int bh, kt;  // key tile 0 has the longest query range: rank == key tile
  map_workgroup(blockIdx.x, BH, p.n_tiles, bh, kt);
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const int kv0 = kt * kDkvBlockKV;
  const int kv0w = kv0 + 32 * wave;
  const bool vec = p.vec != 0;

  const short *Q = (const short *)p.q.ptr + b * p.q.stride_batch + hd * p.q.stride_head;
  const short *K = (const short *)p.k.ptr + b * p.k.stride_batch + hd * p.k.stride_head;
  const short *V = (const short *)p.v.ptr + b * p.v.stride_batch + hd * p.v.stride_head;
  const short *DO = (const short *)p.d_o.ptr + b * p.d_o.stride_batch + hd * p.d_o.stride_head;
  short *DK = (short *)p.dk.ptr + b * p.dk.stride_batch + hd * p.dk.stride_head;
  short *DV = (short *)p.dv.ptr + b * p.dv.stride_batch + hd * p.dv.stride_head;
  const float *LSE = p.lse + (int64_t)bh * p.seqlen_q_rounded;
  const float *DELTA = p.delta + (int64_t)bh * p.seqlen_q_rounded;

  // B operands: lane (c, h) holds row kv0w + c of K and of V, columns 16 ks + 8 h + j.
  s16x8 kf[KS], vf[KS];
  {
    const int row = kv0w + c;
    const bool ok = row < p.seqlen_k;
    const short *kp = K + (int64_t)row * p.k.stride_seq;
    const short *vp = V + (int64_t)row * p.v.stride_seq;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      kf[ks] = load_chunk(kp, 16 * ks + 8 * h, p.headdim, ok, vec);
      vf[ks] = load_chunk(vp, 16 * ks + 8 * h, p.headdim, ok, vec);
    }
  }

  // First query tile that can see this key tile (row >= col), aligned down to BQ.
  const int q_begin = (kv0 / BQ) * BQ;
  const int n_tiles = (p.seqlen_q > q_begin) ? (p.seqlen_q - q_begin + BQ - 1) / BQ : 0;

  s16x8 qreg[CPT], greg[CPT];
  float lse_reg = 0.f, delta_reg = 0.f;
  auto load_tile = [&](int qt0) {
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      const int id = tid + NTHREADS * i;
      const int r = id / CPR, cc = id % CPR;
      const int row = qt0 + r;
      const bool ok = row < p.seqlen_q;
      qreg[i] = load_chunk(Q + (int64_t)row * p.q.stride_seq, cc * 8, p.headdim, ok, vec);
      greg[i] = load_chunk(DO + (int64_t)row * p.d_o.stride_seq, cc * 8, p.headdim, ok, vec);
    }
    if (tid < BQ) {
      const int row = qt0 + tid;
      const bool ok = row < p.seqlen_q;
      lse_reg = ok ? LSE[row] * kLog2e : 0.f;
      delta_reg = ok ? DELTA[row] : 0.f;
    }
  };
  auto store_tile = [&](int buf) {
    short *sq = smem + buf * L::STAGE_ELEMS;
    short *sg = sq + L::Q_ELEMS;
    float *sl = reinterpret_cast<float *>(sg + L::Q_ELEMS);
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      const int id = tid + NTHREADS * i;
      const int r = id / CPR, cc = id % CPR;
      *reinterpret_cast<s16x8 *>(sq + r * L::QLD + cc * 8) = qreg[i];
      *reinterpret_cast<s16x8 *>(sg + r * L::QLD + cc * 8) = greg[i];
    }
    if (tid < BQ) {
      sl[tid] = lse_reg;
      sl[BQ + tid] = delta_reg;
    }
  };

  const int row_frag_off = c * L::QLD + 8 * h;
  const int tr_frag_off = (4 * h + (i16 >> 2)) * L::QLD + 16 * g2 + 4 * (i16 & 3);
  const int kvcol = kv0w + c;

  for (int pass = 0; pass < NPASS; pass++) {
  const int col0 = pass * DBP * 32;  // first dK / dV column of this pass
  f32x16 dkacc[DBP], dvacc[DBP];
#pragma unroll
  for (int db = 0; db < DBP; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) {
      dkacc[db][i] = 0.f;
      dvacc[db][i] = 0.f;
    }

  if (n_tiles > 0) {
    load_tile(q_begin);
    store_tile(0);
  }
  __syncthreads();

  for (int t = 0; t < n_tiles; t++) {
    const int buf = t & 1;
    const int qt0 = q_begin + t * BQ;
    const bool more = (t + 1) < n_tiles;
    // The next tile travels through registers while this one is worked on, except at 256
    // columns, where those registers are not to be had: there it is fetched after the MFMAs.
    constexpr bool EARLY_LOAD = DP <= 192;
    if (EARLY_LOAD && more) load_tile(qt0 + BQ);

    const short *sq = smem + buf * L::STAGE_ELEMS;
    const short *sg = sq + L::Q_ELEMS;
    const float *sl = reinterpret_cast<const float *>(sg + L::Q_ELEMS);

#pragma unroll
    for (int mq = 0; mq < MQ; mq++) {
      const int qb = qt0 + 32 * mq;  // first query row of this 32-row block
      // Skip blocks whose every row lies above this wave's first key column.
      if (qb + 31 >= kv0w) {
        f32x16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          s[i] = 0.f;
          dp[i] = 0.f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          s16x8 a = *reinterpret_cast<const s16x8 *>(sq + row_frag_off + 32 * mq * L::QLD + 16 * ks);
          s = Elem<T>::mfma(a, kf[ks], s);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          s16x8 a = *reinterpret_cast<const s16x8 *>(sg + row_frag_off + 32 * mq * L::QLD + 16 * ks);
          dp = Elem<T>::mfma(a, vf[ks], dp);
        }
        const bool need_mask = (qb < kv0w + 31);
        f32x16 pr, ds;
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const f32x4 l4 = *reinterpret_cast<const f32x4 *>(sl + 32 * mq + 8 * g + 4 * h);
          const f32x4 d4 = *reinterpret_cast<const f32x4 *>(sl + BQ + 32 * mq + 8 * g + 4 * h);
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const int i = 4 * g + e;
            float x = fast_exp2(s[i] * p.scale_log2 - l4[e]);
            if (need_mask) {
              const int qrow = qb + 8 * g + 4 * h + e;
              if (kvcol > qrow) x = 0.f;
            }
            pr[i] = x;
            ds[i] = x * (dp[i] - d4[e]);
          }
        }
        f32x8 plo = {pr[0], pr[1], pr[2], pr[3], pr[4], pr[5], pr[6], pr[7]};
        f32x8 phi = {pr[8], pr[9], pr[10], pr[11], pr[12], pr[13], pr[14], pr[15]};
        f32x8 dlo = {ds[0], ds[1], ds[2], ds[3], ds[4], ds[5], ds[6], ds[7]};
        f32x8 dhi = {ds[8], ds[9], ds[10], ds[11], ds[12], ds[13], ds[14], ds[15]};
        s16x8 pf[2] = {Elem<T>::pack8(plo), Elem<T>::pack8(phi)};
        s16x8 dsf[2] = {Elem<T>::pack8(dlo), Elem<T>::pack8(dhi)};
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
#pragma unroll
          for (int db = 0; db < DBP; db++) {
            const int off = tr_frag_off + (32 * mq + 16 * tt) * L::QLD + col0 + 32 * db;
            s16x8 ag = lds_read_tr_frag(sg + off, L::QLD);
            dvacc[db] = Elem<T>::mfma(ag, pf[tt], dvacc[db]);
            s16x8 aq = lds_read_tr_frag(sq + off, L::QLD);
            dkacc[db] = Elem<T>::mfma(aq, dsf[tt], dkacc[db]);
          }
        }
      }
    }

    if (!EARLY_LOAD && more) load_tile(qt0 + BQ);
    if (more) store_tile(buf ^ 1);
    __syncthreads();
  }

  // Columns [col0, col0 + 32 DBP) of this wave's 32 rows of dV and dK.  The patch overlays the
  // stages: the loop's last barrier ordered it after all reads, and the barrier below orders the
  // next pass's tile stores after it.
  short *patch = smem + wave * 32 * (DP + 8);
  store_transposed_acc<T, 32 * DBP>(dvacc, 1.0f, patch, DV + (int64_t)kv0w * p.dv.stride_seq + col0,
                                    p.dv.stride_seq, p.seqlen_k - kv0w, p.headdim - col0, vec);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  store_transposed_acc<T, 32 * DBP>(dkacc, p.scale, patch, DK + (int64_t)kv0w * p.dk.stride_seq + col0,
                                    p.dk.stride_seq, p.seqlen_k - kv0w, p.headdim - col0, vec);
  if (pass + 1 < NPASS) __syncthreads();
  }
}



// ------------------------------------------------------------------------------------------
// Fast paths (head dimension equal to the padded one, 16-byte aligned rows): the streamed tiles
// go straight from global memory into swizzled, unpadded LDS with LDS-direct loads, two stages
// deep, one workgroup barrier per tile.  See fa2_common.cuh for the swizzle and TileLoader.
// ------------------------------------------------------------------------------------------
__device__ __forceinline__ void bwd_wait_vmem_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// K tiles in three stages and V tiles in two, like the forward: tile t brings in K tile t+2 and V
// tile t+1, so that the K rows of the next tile are there when the last block of a tile fetches them.
template <int DP, int BKV>
struct DqDirectLayout {
  static constexpr int TILE_ELEMS = BKV * DP;
  static constexpr int K_STAGES = 3, V_STAGES = 2;
  static constexpr int K_BASE = 0;
  static constexpr int V_BASE = K_STAGES * TILE_ELEMS;
  static constexpr int STAGE_ELEMS = (K_STAGES + V_STAGES) * TILE_ELEMS;
  static constexpr int PATCH_ELEMS = kDqWaves * 32 * (DP + 8);
  static constexpr int TOTAL_ELEMS = (STAGE_ELEMS > PATCH_ELEMS) ? STAGE_ELEMS : PATCH_ELEMS;
};

// With FUSE_DELTA the kernel also computes delta = rowsum(O * dO) for its query rows (it holds
// the dO rows anyway), uses it and writes it out for the dK/dV kernel, which then has to be
// launched after this one; the separate preprocess launch disappears.
template <typename T, int DP, int BKV, bool FUSE_DELTA>
__global__ __launch_bounds__(64 * kDqWaves, 2) void bwd_dq_direct_kernel(const BwdParams p) {
  using L = DqDirectLayout<DP, BKV>;
  constexpr int KS = DP / 16, DB = DP / 32;
  constexpr int BLK = 32;
  static_assert(BKV == 2 * BLK, "written for 64-row key tiles of two 32-row blocks");

  __shared__ __attribute__((aligned(1024))) short smem[L::TOTAL_ELEMS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, g2 = (lane >> 4) & 1;

  const int BH = p.batch * p.nheads;
  int bh, rank;
  map_workgroup(blockIdx.x, BH, p.n_tiles, bh, rank);
  const int qt = p.n_tiles - 1 - rank;  // the last query tile sees the most keys
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const int q0 = qt * kDqBlockQ;
  const int q0w = q0 + 32 * wave;

  const short *Q = (const short *)p.q.ptr + b * p.q.stride_batch + hd * p.q.stride_head;
  const short *K = (const short *)p.k.ptr + b * p.k.stride_batch + hd * p.k.stride_head;
  const short *V = (const short *)p.v.ptr + b * p.v.stride_batch + hd * p.v.stride_head;
  const short *DO = (const short *)p.d_o.ptr + b * p.d_o.stride_batch + hd * p.d_o.stride_head;
  short *DQ = (short *)p.dq.ptr + b * p.dq.stride_batch + hd * p.dq.stride_head;

  const TileLoader<DP, BKV, kDqWaves> kload(K, p.k.stride_seq), vload(V, p.v.stride_seq);
  const int seqlen_k = p.seqlen_k;
  const float scale_log2 = p.scale_log2;

  const int kv_end = min(q0 + kDqBlockQ, seqlen_k);
  const int n_tiles = (kv_end + BKV - 1) / BKV;
  const int n_mine = min((kv_end + BLK - 1) / BLK, q0w / BLK + 1);  // 32-key blocks of this wave
  const int n_full = min(q0w + 1, seqlen_k) / BLK;                   // leading blocks without mask
  const int n_inside = seqlen_k / BKV;

  const unsigned lds_base = lds_u32(smem);  // LDS byte address of smem
  auto issue_k = [&](int t) {
    const unsigned dst = lds_base + 2u * (unsigned)(L::K_BASE + (t % L::K_STAGES) * L::TILE_ELEMS);
    if (t < n_inside) kload.issue(t * BKV, dst); else kload.issue_clamped(t * BKV, seqlen_k, dst);
  };
  auto issue_v = [&](int t) {
    const unsigned dst = lds_base + 2u * (unsigned)(L::V_BASE + (t % L::V_STAGES) * L::TILE_ELEMS);
    if (t < n_inside) vload.issue(t * BKV, dst); else vload.issue_clamped(t * BKV, seqlen_k, dst);
  };
  // K_0, V_0 and K_1 are loaded here; after that tile t brings in K_{t+2} and V_{t+1}.
  issue_k(0);
  issue_v(0);
  if (n_tiles > 1) issue_k(1);

  // B operands: lane (c, h) holds row q0w + c of Q and of dO, columns 16 ks + 8 h + j.
  s16x8 qf[KS], gf[KS];
  float lse2 = 0.f, delta = 0.f;
  {
    const int row = q0w + c;
    const bool ok = row < p.seqlen_q;
    const short *qp = Q + (int64_t)row * p.q.stride_seq;
    const short *gp = DO + (int64_t)row * p.d_o.stride_seq;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      qf[ks] = load_chunk(qp, 16 * ks + 8 * h, DP, ok, true);
      gf[ks] = load_chunk(gp, 16 * ks + 8 * h, DP, ok, true);
    }
    if (ok) lse2 = p.lse[(int64_t)bh * p.seqlen_q_rounded + row] * kLog2e;
    if (FUSE_DELTA) {
      const short *op = (const short *)p.o.ptr + b * p.o.stride_batch + hd * p.o.stride_head +
                        (int64_t)row * p.o.stride_seq;
      float part = 0.f;  // this lane's half of the row: columns 16 ks + 8 h + j
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const s16x8 of = load_chunk(op, 16 * ks + 8 * h, DP, ok, true);
#pragma unroll
        for (int j = 0; j < 8; j++) part += Elem<T>::to_float(of[j]) * Elem<T>::to_float(gf[ks][j]);
      }
      delta = sum_over_halves(part);  // 0 for rows beyond the sequence (loads return zeros)
      float *dout = p.delta_out + (int64_t)bh * p.seqlen_q_rounded;
      if (h == 0 && ok) dout[row] = delta;
      if (qt == p.n_tiles - 1)  // rows [seqlen_q, seqlen_q_rounded) are defined to be zero
        for (int r = p.seqlen_q + tid; r < p.seqlen_q_rounded; r += 64 * kDqWaves) dout[r] = 0.f;
    } else if (ok) {
      delta = p.delta[(int64_t)bh * p.seqlen_q_rounded + row];
    }
  }

  // Swizzled fragment addresses (32-bit LDS pointers).  knext: K rows of the tile the next block
  // lies in; vrow: V rows of the current tile; klo/khi: transposed K fragments of the current tile.
  const lds_cptr lds0 = to_lds(smem);
  lds_cptr knext[KS], vrow[KS], klo[DB], khi[DB];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    knext[ks] = lds0 + L::K_BASE + swz_off<DP>(c, 2 * ks + h);
    vrow[ks] = lds0 + L::V_BASE + swz_off<DP>(c, 2 * ks + h);
  }
  {
    const int rowlo = 4 * h + (i16 >> 2);
    const int sub = (i16 & 1) * 4;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      const int chunk = 4 * db + 2 * g2 + ((i16 & 3) >> 1);
      klo[db] = lds0 + L::K_BASE + swz_off<DP>(rowlo, chunk) + sub;
      khi[db] = lds0 + L::K_BASE + swz_off<DP>(rowlo + 8, chunk) + sub;
    }
  }

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) dqacc[db][i] = 0.f;
  const int qrow = q0w + c;
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  bwd_wait_vmem_all();
  __syncthreads();

  // Ring of A fragments, preloaded with the K rows of block 0.
  s16x8 ring[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) ring[ks] = lds_read_128(knext[ks]);

  // One 32-key block j = 2 t + HALF, three GEMMs of KS MFMAs, each unit = one MFMA, the LDS reads
  // that refill the ring slot it freed, and a share of the vector work:
  //     A: S^T = K Q^T            ring <- V rows              (loads of V tile t+1 when SPREAD)
  //     B: dP^T = V dO^T          ring <- K^T fragments       exponentials of S; loads of K tile t+2
  //     C: dQ^T += K^T dS^T       ring <- next block's K rows second half of the dS arithmetic
  constexpr int LOADS = TileLoader<DP, BKV, kDqWaves>::LOADS;
  constexpr int LOAD_EVERY = KS / LOADS;
  auto block = [&](int j, auto half_tag, auto spread_tag) __attribute__((always_inline)) {
    constexpr int HALF = decltype(half_tag)::value;
    constexpr bool SPREAD = decltype(spread_tag)::value;
    const int kt = j / 2 + 2, vt = j / 2 + 1;  // tiles loaded during this block (SPREAD)
    if (j >= n_mine) {
      if (SPREAD) {  // not reached: skipped blocks lie in the last two tiles, which load nothing
        issue_k(kt);
        issue_v(vt);
      }
      return;
    }
    const unsigned kdst = lds_base + 2u * (unsigned)(L::K_BASE + (kt % L::K_STAGES) * L::TILE_ELEMS);
    const unsigned vdst = lds_base + 2u * (unsigned)(L::V_BASE + (vt % L::V_STAGES) * L::TILE_ELEMS);
    constexpr int HOFF = HALF * BLK * DP;
    f32x16 s = zero, dp = zero;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      s = Elem<T>::mfma(ring[ks], qf[ks], s);
      if (SPREAD && ks % LOAD_EVERY == 0) vload.issue_one(vt * BKV, vdst, ks / LOAD_EVERY);
      ring[ks] = lds_read_128(vrow[ks] + HOFF);
      __builtin_amdgcn_sched_barrier(0);
    }
    const bool need_mask = j >= n_full;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      dp = Elem<T>::mfma(ring[ks], gf[ks], dp);
      if (SPREAD && ks % LOAD_EVERY == 0) kload.issue_one(kt * BKV, kdst, ks / LOAD_EVERY);
      {
        s16x4 a0 = lds_read_tr(klo[ks % DB] + HOFF + 16 * (ks / DB) * DP);
        s16x4 a1 = lds_read_tr(khi[ks % DB] + HOFF + 16 * (ks / DB) * DP);
        ring[ks] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
#pragma unroll
      for (int u = 0; u < 16 / KS; u++) {
        const int i = (16 / KS) * ks + u;
        float pr = fast_exp2(s[i] * scale_log2 - lse2);
        if (need_mask) {
          const int kv = j * BLK + 8 * (i >> 2) + 4 * h + (i & 3);
          if (kv > qrow || kv >= seqlen_k) pr = 0.f;
        }
        s[i] = pr;
      }
      asm volatile("" : "+v"(s));
      __builtin_amdgcn_sched_barrier(0);
    }
    // dS of the first 16 keys before the dQ MFMAs that need them, the rest beside those MFMAs.
    f32x8 lo, hi;
#pragma unroll
    for (int i = 0; i < 8; i++) lo[i] = s[i] * (dp[i] - delta);
    s16x8 dsf[2];
    dsf[0] = Elem<T>::pack8(lo);
#pragma unroll
    for (int slot = 0; slot < KS; slot++) {
      constexpr int HALF_SLOTS = KS / 2;
      const int ks2 = slot / DB, db = slot % DB;
      dqacc[db] = Elem<T>::mfma(ring[slot], dsf[ks2], dqacc[db]);
      ring[slot] = lds_read_128(knext[slot] + (HALF == 0 ? BLK * DP : 0));
      if (slot < HALF_SLOTS) {
#pragma unroll
        for (int u = 0; u < 8 / HALF_SLOTS; u++) {
          const int i = (8 / HALF_SLOTS) * slot + u;
          hi[i] = s[8 + i] * (dp[8 + i] - delta);
        }
        asm volatile("" : "+v"(hi));
        if (slot == HALF_SLOTS - 1) dsf[1] = Elem<T>::pack8(hi);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // End of a tile: every wave is done with V_t and with K_t; K_{t+2} and V_{t+1} (issued during
  // this tile) have landed.  The fragment pointers advance (stages are used round-robin).
  auto k_step = [&](int t) { return ((t + 1) % L::K_STAGES == 0) ? -(L::K_STAGES - 1) * L::TILE_ELEMS : L::TILE_ELEMS; };
  auto end_tile = [&](int t) {
    bwd_wait_vmem_all();
    __syncthreads();
    const int dk = k_step(t);
    const int dv = ((t + 1) % L::V_STAGES == 0) ? -(L::V_STAGES - 1) * L::TILE_ELEMS : L::TILE_ELEMS;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) vrow[ks] += dv;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      klo[db] += dk;
      khi[db] += dk;
    }
  };
  auto tile = [&](int t, auto spread_tag) __attribute__((always_inline)) {
    block(2 * t, std::integral_constant<int, 0>{}, spread_tag);
    // knext -> K tile t+1 before the second block prefetches from it.
    const int dk = k_step(t);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) knext[ks] += dk;
    block(2 * t + 1, std::integral_constant<int, 1>{}, std::false_type{});
    end_tile(t);
  };
  int t = 0;
  const int n_spread = min(n_tiles, n_inside) - 2;
  for (; t < n_spread; t++) tile(t, std::true_type{});
  for (; t < n_tiles; t++) {
    if (t + 2 < n_tiles) issue_k(t + 2);
    if (t + 1 < n_tiles) issue_v(t + 1);
    tile(t, std::false_type{});
  }

  short *patch = smem + wave * 32 * (DP + 8);
  store_transposed_acc<T, DP>(dqacc, p.scale, patch, DQ + (int64_t)q0w * p.dq.stride_seq,
                              p.dq.stride_seq, p.seqlen_q - q0w, DP, true);
}

// MFMA whose accumulator is held in vector registers.  At one wave per SIMD the compiler gives every
// MFMA result an accumulation register and copies it out (v_accvgpr_read) before vector
// instructions can use it; S and dP are consumed by vector instructions right away, so their
// chains are written out by hand with vector-register accumulators (dK and dV, which are only
// read at the very end, stay in accumulation registers).  The compiler does not know these are
// MFMAs: `settle` supplies the wait states an 8-pass MFMA result needs before vector
// instructions may read it (11; the s_nop gives 12) and ties them to the value.
template <typename T>
struct VgprMfma;
template <>
struct VgprMfma<__bf16> {
  static __device__ __forceinline__ void first(f32x16 &d, s16x8 a, s16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void next(f32x16 &d, s16x8 a, s16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
  }
};
template <>
struct VgprMfma<_Float16> {
  static __device__ __forceinline__ void first(f32x16 &d, s16x8 a, s16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void next(f32x16 &d, s16x8 a, s16x8 b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
  }
};
__device__ __forceinline__ void settle(f32x16 &d) { asm volatile("s_nop 11" : "+v"(d)); }

template <int DP, int BQ>
struct DkvDirectLayout {
  static constexpr int TILE_ELEMS = BQ * DP;
  // One stage: Q tile, dO tile, then lse*log2e and delta as floats (2 shorts each).
  static constexpr int STAGE_ELEMS = 2 * TILE_ELEMS + 4 * BQ;
  static constexpr int STAGES = 3;
  static constexpr int PATCH_ELEMS = kDkvWaves * 32 * (DP + 8);
  static constexpr int TOTAL_ELEMS =
      (STAGES * STAGE_ELEMS > PATCH_ELEMS) ? STAGES * STAGE_ELEMS : PATCH_ELEMS;
};

template <typename T, int DP, int BQ>
__global__ __launch_bounds__(64 * kDkvWaves, (DP <= 64 ? 2 : 1)) void bwd_dkdv_direct_kernel(const BwdParams p) {
  using L = DkvDirectLayout<DP, BQ>;
  constexpr int KS = DP / 16, DB = DP / 32;
  constexpr int NTHREADS = 64 * kDkvWaves;
  static_assert(BQ == 64 && KS == 2 * DB, "schedule is written for 64-row query tiles of two blocks");
  static_assert(BQ <= NTHREADS, "one thread per row loads lse and delta");
  static_assert((L::STAGE_ELEMS * 2) % 256 == 0, "stages must start on a 256-byte LDS bank line");

  __shared__ __attribute__((aligned(1024))) short smem[L::TOTAL_ELEMS];
  FA2_STAMP(0);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, g2 = (lane >> 4) & 1;

  // Key tile 0 has the longest query range: issue tiles in ascending order (heaviest first).
  const int BH = p.batch * p.nheads;
  int bh, kt;  // key tile 0 has the longest query range: rank == key tile
  map_workgroup(blockIdx.x, BH, p.n_tiles, bh, kt);
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const int kv0 = kt * kDkvBlockKV;
  const int kv0w = kv0 + 32 * wave;

  const short *Q = (const short *)p.q.ptr + b * p.q.stride_batch + hd * p.q.stride_head;
  const short *K = (const short *)p.k.ptr + b * p.k.stride_batch + hd * p.k.stride_head;
  const short *V = (const short *)p.v.ptr + b * p.v.stride_batch + hd * p.v.stride_head;
  const short *DO = (const short *)p.d_o.ptr + b * p.d_o.stride_batch + hd * p.d_o.stride_head;
  short *DK = (short *)p.dk.ptr + b * p.dk.stride_batch + hd * p.dk.stride_head;
  short *DV = (short *)p.dv.ptr + b * p.dv.stride_batch + hd * p.dv.stride_head;
  const float *LSE = p.lse + (int64_t)bh * p.seqlen_q_rounded;
  const float *DELTA = p.delta + (int64_t)bh * p.seqlen_q_rounded;

  const TileLoader<DP, BQ, kDkvWaves> qload(Q, p.q.stride_seq), gload(DO, p.d_o.stride_seq);
  const int seqlen_q = p.seqlen_q;
  const float scale_log2 = p.scale_log2;

  // First query tile that can see this key tile (row >= col), aligned down to BQ.
  const int q_begin = (kv0 / BQ) * BQ;
  const int n_tiles = (seqlen_q > q_begin) ? (seqlen_q - q_begin + BQ - 1) / BQ : 0;
  const int n_inside = (seqlen_q - q_begin) / BQ;  // tiles whose every row exists
  // Tiles that touch the diagonal of this key tile (their blocks need the causal mask).
  const int n_diag = min(n_tiles, (kv0 + kDkvBlockKV - q_begin + BQ - 1) / BQ);

  const unsigned lds_base = lds_u32(smem);  // LDS byte address of smem
  auto issue_tile = [&](int t) {
    const unsigned dst = lds_base + 2u * (unsigned)((t % L::STAGES) * L::STAGE_ELEMS);
    const int row0 = q_begin + t * BQ;
    if (t < n_inside) {
      qload.issue(row0, dst);
      gload.issue(row0, dst + 2u * L::TILE_ELEMS);
    } else {
      qload.issue_clamped(row0, seqlen_q, dst);
      gload.issue_clamped(row0, seqlen_q, dst + 2u * L::TILE_ELEMS);
    }
  };
  // lse*log2e and delta of a tile go through registers into the stage's statistics area (rows
  // beyond the sequence get 0: their probabilities are zeroed by the row mask).
  float lse_reg = 0.f, delta_reg = 0.f;
  auto load_stats = [&](int t) {
    if (tid < BQ) {
      const int row = q_begin + t * BQ + tid;
      const bool ok = row < seqlen_q;
      lse_reg = ok ? LSE[row] * kLog2e : 0.f;
      delta_reg = ok ? DELTA[row] : 0.f;
    }
  };
  auto store_stats = [&](int t) {
    float *sl = reinterpret_cast<float *>(smem + (t % L::STAGES) * L::STAGE_ELEMS + 2 * L::TILE_ELEMS);
    if (tid < BQ) {
      sl[tid] = lse_reg;
      sl[BQ + tid] = delta_reg;
    }
  };
  // Prologue: every global load of the first three tiles and of this wave's K and V rows is
  // issued before anything waits, so that the workgroup pays one memory latency, not one per
  // tile.
#pragma unroll
  for (int t = 0; t < L::STAGES; t++)
    if (t < n_tiles) issue_tile(t);

  // B operands: lane (c, h) holds row kv0w + c of K and of V, columns 16 ks + 8 h + j.
  s16x8 kf[KS], vf[KS];
  {
    const int row = kv0w + c;
    const bool ok = row < p.seqlen_k;
    const short *kp = K + (int64_t)row * p.k.stride_seq;
    const short *vp = V + (int64_t)row * p.v.stride_seq;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      kf[ks] = load_chunk(kp, 16 * ks + 8 * h, DP, ok, true);
      vf[ks] = load_chunk(vp, 16 * ks + 8 * h, DP, ok, true);
    }
  }
  // Statistics of the first three tiles: loaded now, written to LDS just before the first
  // barrier (the write has to wait for every load above, and the set-up below should not).
  float l3[L::STAGES], d3[L::STAGES];
#pragma unroll
  for (int t = 0; t < L::STAGES; t++) {
    load_stats(t);  // rows beyond the sequence (and tiles beyond the last) read as 0
    l3[t] = lse_reg;
    d3[t] = delta_reg;
  }

  // Swizzled fragment addresses (32-bit LDS pointers) into the current tile's stage; the dO tile
  // sits TILE_ELEMS after the Q tile.  qnext runs one block ahead (for the ring prefetch).
  const lds_cptr lds0 = to_lds(smem);
  lds_cptr qnext[KS], qrow[KS], qlo[DB], qhi[DB];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    qrow[ks] = lds0 + swz_off<DP>(c, 2 * ks + h);
    qnext[ks] = qrow[ks];
  }
  {
    const int rowlo = 4 * h + (i16 >> 2);
    const int sub = (i16 & 1) * 4;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      const int chunk = 4 * db + 2 * g2 + ((i16 & 3) >> 1);
      qlo[db] = lds0 + swz_off<DP>(rowlo, chunk) + sub;
      qhi[db] = lds0 + swz_off<DP>(rowlo + 8, chunk) + sub;
    }
  }
  const __attribute__((address_space(3))) float *stat =
      reinterpret_cast<const __attribute__((address_space(3))) float *>(lds0 + 2 * L::TILE_ELEMS) + 4 * h;

  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) {
      dkacc[db][i] = 0.f;
      dvacc[db][i] = 0.f;
    }
  const int kvcol = kv0w + c;

#pragma unroll
  for (int t = 0; t < L::STAGES; t++) {
    lse_reg = l3[t];
    delta_reg = d3[t];
    store_stats(t);
  }
  bwd_wait_vmem_all();
  __syncthreads();

  FA2_STAMP(1);
  // Two rings of A fragments, preloaded with the Q rows and the dO rows of block 0.
  s16x8 ring[KS], ringb[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) ring[ks] = lds_read_128(qrow[ks]);
#pragma unroll
  for (int ks = 0; ks < KS; ks++) ringb[ks] = lds_read_128(qrow[ks] + L::TILE_ELEMS);

  // One 32-row query block.  HALF selects the half-tile; MASKED switches the causal/row masks on.
  // With SPREAD the block also issues the global->LDS loads of tile `lt`, one every fourth unit:
  // issued back to back by all waves after a barrier they queue up in the memory pipeline, and a
  // wave whose load cannot issue cannot issue its MFMAs either.
  auto block = [&](int qb, auto half_tag, auto masked_tag, auto spread_tag, int lt) {
    constexpr int HALF = decltype(half_tag)::value;
    constexpr bool MASKED = decltype(masked_tag)::value;
    constexpr bool SPREAD = decltype(spread_tag)::value;
    constexpr int LOADS = TileLoader<DP, BQ, kDkvWaves>::LOADS;
    static_assert(4 * KS == 8 * LOADS, "one load every fourth unit covers both tiles");
    const unsigned ldst = lds_base + 2u * (unsigned)((lt % L::STAGES) * L::STAGE_ELEMS);
    const int lrow0 = q_begin + lt * BQ;
    auto spread_load = [&](int unit) {  // unit: 0 .. 4 KS - 1 over the four GEMMs
      if (SPREAD && unit % 4 == 0) {
        const int li = unit / 4;
        if (li < LOADS) qload.issue_one(lrow0, ldst, li);
        else gload.issue_one(lrow0, ldst + 2u * L::TILE_ELEMS, li - LOADS);
      }
    };
    constexpr int QOFF = HALF * 32 * DP;          // Q rows of this block inside the tile
    constexpr int GOFF = QOFF + L::TILE_ELEMS;    // dO rows of this block
    typedef const __attribute__((address_space(3))) f32x4 *stat4_ptr;

    // ---- S = Q K^T (ring: Q rows -> dO^T); statistics of the 16 rows this lane holds ---------
    f32x16 s, dp;
    f32x4 l4[4], d4[4];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (ks == 0) VgprMfma<T>::first(s, ring[ks], kf[ks]);
      else VgprMfma<T>::next(s, ring[ks], kf[ks]);
      spread_load(ks);
      {
        s16x4 a0 = lds_read_tr(qlo[ks % DB] + GOFF + 16 * (ks / DB) * DP);
        s16x4 a1 = lds_read_tr(qhi[ks % DB] + GOFF + 16 * (ks / DB) * DP);
        ring[ks] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      constexpr int PER = (4 + KS - 1) / KS;  // row groups of four fetched per unit
#pragma unroll
      for (int u = 0; u < PER; u++) {
        const int g = ks * PER + u;
        if (g < 4) {
          l4[g] = *reinterpret_cast<stat4_ptr>(stat + 32 * HALF + 8 * g);
          d4[g] = *reinterpret_cast<stat4_ptr>(stat + BQ + 32 * HALF + 8 * g);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- dP = dO V^T (ringb: dO rows -> Q^T); exponentials under the MFMAs -------------------
    f32x16 pr;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (ks == 0) VgprMfma<T>::first(dp, ringb[ks], vf[ks]);
      else VgprMfma<T>::next(dp, ringb[ks], vf[ks]);
      spread_load(KS + ks);
      {
        s16x4 a0 = lds_read_tr(qlo[ks % DB] + QOFF + 16 * (ks / DB) * DP);
        s16x4 a1 = lds_read_tr(qhi[ks % DB] + QOFF + 16 * (ks / DB) * DP);
        ringb[ks] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      if (ks == 0) settle(s);  // after the S chain's last MFMA and before the first read of S
#pragma unroll
      for (int u = 0; u < 16 / KS; u++) {
        const int i = (16 / KS) * ks + u;
        float x = fast_exp2(s[i] * scale_log2 - l4[i >> 2][i & 3]);
        if (MASKED) {
          const int qr = qb + 8 * (i >> 2) + 4 * h + (i & 3);
          if (kvcol > qr || qr >= seqlen_q) x = 0.f;
        }
        pr[i] = x;
      }
      asm volatile("" : "+v"(pr));
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x8 plo = {pr[0], pr[1], pr[2], pr[3], pr[4], pr[5], pr[6], pr[7]};
    f32x8 phi = {pr[8], pr[9], pr[10], pr[11], pr[12], pr[13], pr[14], pr[15]};
    const s16x8 pf[2] = {Elem<T>::pack8(plo), Elem<T>::pack8(phi)};
    // ---- dV^T += dO^T P (ring: dO^T -> Q rows of the next block); dS arithmetic under the MFMAs
    f32x16 ds;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      dvacc[ks % DB] = Elem<T>::mfma(ring[ks], pf[ks / DB], dvacc[ks % DB]);
      spread_load(2 * KS + ks);
      ring[ks] = lds_read_128(qnext[ks] + (HALF == 0 ? 32 * DP : 0));
      if (ks == 0) settle(dp);
#pragma unroll
      for (int u = 0; u < 16 / KS; u++) {
        const int i = (16 / KS) * ks + u;
        ds[i] = pr[i] * (dp[i] - d4[i >> 2][i & 3]);
      }
      asm volatile("" : "+v"(ds));
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x8 dlo = {ds[0], ds[1], ds[2], ds[3], ds[4], ds[5], ds[6], ds[7]};
    f32x8 dhi = {ds[8], ds[9], ds[10], ds[11], ds[12], ds[13], ds[14], ds[15]};
    const s16x8 dsf[2] = {Elem<T>::pack8(dlo), Elem<T>::pack8(dhi)};
    // ---- dK^T += Q^T dS (ringb: Q^T -> dO rows of the next block) ------------------------------
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      dkacc[ks % DB] = Elem<T>::mfma(ringb[ks], dsf[ks / DB], dkacc[ks % DB]);
      spread_load(3 * KS + ks);
      ringb[ks] = lds_read_128(qnext[ks] + L::TILE_ELEMS + (HALF == 0 ? 32 * DP : 0));
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Tiles [spread_lo, spread_hi) bring in the tile two after them during their first block; the
  // other tiles' successors are loaded at once after the barrier that frees their stage.
  const int spread_lo = n_diag, spread_hi = n_inside - 2;
  auto tile = [&](int t, auto masked_tag, auto spread_tag) {
    const int qt0 = q_begin + t * BQ;
    // qnext -> next tile's stage before the second block prefetches from it.
    const int d = ((t + 1) % L::STAGES == 0) ? -(L::STAGES - 1) * L::STAGE_ELEMS : L::STAGE_ELEMS;
    block(qt0, std::integral_constant<int, 0>{}, masked_tag, spread_tag, t + 2);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qnext[ks] += d;
    block(qt0 + 32, std::integral_constant<int, 1>{}, masked_tag, std::false_type{}, 0);
    // Tile t+2's statistics were loaded one tile ago; their stage was freed by the last barrier.
    if (t >= 1 && t + 2 < n_tiles) store_stats(t + 2);
    // Everyone is done with stage t % 3; tile t+1 has landed, tile t+2 is in flight.
    bwd_wait_vmem_all();
    __syncthreads();
    if (t + 3 < n_tiles) {
      if (t + 1 < spread_lo || t + 1 >= spread_hi) issue_tile(t + 3);
      load_stats(t + 3);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qrow[ks] += d;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      qlo[db] += d;
      qhi[db] += d;
    }
    stat += d / 2;  // float elements
  };

  int t = 0;
  for (; t < n_diag; t++) tile(t, std::true_type{}, std::false_type{});
  for (; t < spread_hi; t++) tile(t, std::false_type{}, std::true_type{});
  for (; t < n_inside; t++) tile(t, std::false_type{}, std::false_type{});
  for (; t < n_tiles; t++) tile(t, std::true_type{}, std::false_type{});
  FA2_STAMP(2);

  short *patch = smem + wave * 32 * (DP + 8);
  store_transposed_acc<T, DP>(dvacc, 1.0f, patch, DV + (int64_t)kv0w * p.dv.stride_seq,
                              p.dv.stride_seq, p.seqlen_k - kv0w, DP, true);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  store_transposed_acc<T, DP>(dkacc, p.scale, patch, DK + (int64_t)kv0w * p.dk.stride_seq,
                              p.dk.stride_seq, p.seqlen_k - kv0w, DP, true);
  FA2_STAMP(3);
}

}  // namespace fa2
