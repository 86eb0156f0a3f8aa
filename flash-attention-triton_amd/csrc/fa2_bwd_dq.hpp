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

#include "fa2_common.hpp"

namespace fa2 {

// ------------------------------------------------------------------------------------------
// delta = rowsum(O * dO).  16 lanes per row, 16 rows per workgroup; rows in
// [seqlen_q, seqlen_q_rounded) are written as zero.
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void bwd_preprocess_kernel(const PreParams p) {
  const int tid = threadIdx.x;
  const int sub = tid & 15;
  // One-dimensional grid: row tiles of one (batch, head) pair are consecutive workgroups.
  const int tiles = (p.seqlen_q_rounded + 15) / 16;
  const int bh = blockIdx.x / tiles;
  const int row = (blockIdx.x - bh * tiles) * 16 + (tid >> 4);
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
  map_workgroup(blockIdx.x, BH, p.n_tiles, p.head_group, bh, rank);
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
// Fast paths (head dimension equal to the padded one, 16-byte aligned rows): the streamed tiles
// go straight from global memory into swizzled, unpadded LDS with LDS-direct loads, two stages
// deep, one workgroup barrier per tile.  See fa2_common.hpp for the swizzle and TileLoader.
// ------------------------------------------------------------------------------------------

// K tiles in three stages and V tiles in two, like the forward: tile t brings in K tile t+2 and V
// tile t+1, so that the K rows of the next tile are there when the last block of a tile fetches them.
template <int DP, int BKV>
struct DqDirectLayout {
  static constexpr int LP = lds_pitch(DP);  // LDS row pitch
  static constexpr int TILE_ELEMS = BKV * LP;
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
// PAD: the head dimension is a multiple of 8 below DP; the columns beyond it are zeros in LDS and in
// the register fragments, and are not stored.
template <typename T, int DP, int BKV, bool FUSE_DELTA, bool PAD>
__global__ __launch_bounds__(64 * kDqWaves, (DP <= 128 ? 2 : 1)) void bwd_dq_direct_kernel(const BwdParams p) {
  using L = DqDirectLayout<DP, BKV>;
  constexpr int KS = DP / 16, DB = DP / 32, LP = L::LP;
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
  map_workgroup(blockIdx.x, BH, p.n_tiles, p.head_group, bh, rank);
  const int qt = p.n_tiles - 1 - rank;  // the last query tile sees the most keys
  const int b = bh / p.nheads, hd = bh % p.nheads;
  const int q0 = qt * kDqBlockQ;
  const int q0w = q0 + 32 * wave;

  const short *Q = (const short *)p.q.ptr + b * p.q.stride_batch + hd * p.q.stride_head;
  const short *K = (const short *)p.k.ptr + b * p.k.stride_batch + hd * p.k.stride_head;
  const short *V = (const short *)p.v.ptr + b * p.v.stride_batch + hd * p.v.stride_head;
  const short *DO = (const short *)p.d_o.ptr + b * p.d_o.stride_batch + hd * p.d_o.stride_head;
  short *DQ = (short *)p.dq.ptr + b * p.dq.stride_batch + hd * p.dq.stride_head;

  const int hdim = PAD ? p.headdim : DP;
  const TileLoader<DP, BKV, kDqWaves, PAD> kload(K, p.k.stride_seq, hdim / 8), vload(V, p.v.stride_seq, hdim / 8);
  const int seqlen_k = p.seqlen_k;
  const float scale_log2 = p.scale_log2;

  const int kv_end = min(q0 + kDqBlockQ, seqlen_k);
  const int n_tiles = (kv_end + BKV - 1) / BKV;
  const int n_mine = min((kv_end + BLK - 1) / BLK, q0w / BLK + 1);  // 32-key blocks of this wave
  const int n_full = min(q0w + 1, seqlen_k) / BLK;                   // leading blocks without mask
  const int n_inside = seqlen_k / BKV;

  const unsigned lds_base = lds_u32(smem);  // LDS byte address of smem
  if (PAD) {
    zero_lds<64 * kDqWaves>(smem, L::STAGE_ELEMS);
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
      qf[ks] = load_chunk(qp, 16 * ks + 8 * h, hdim, ok, true);
      gf[ks] = load_chunk(gp, 16 * ks + 8 * h, hdim, ok, true);
    }
    if (ok) lse2 = p.lse[(int64_t)bh * p.seqlen_q_rounded + row] * kLog2e;
    if (FUSE_DELTA) {
      const short *op = (const short *)p.o.ptr + b * p.o.stride_batch + hd * p.o.stride_head +
                        (int64_t)row * p.o.stride_seq;
      float part = 0.f;  // this lane's half of the row: columns 16 ks + 8 h + j
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const s16x8 of = load_chunk(op, 16 * ks + 8 * h, hdim, ok, true);
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
    knext[ks] = lds0 + L::K_BASE + swz_off<LP>(c, 2 * ks + h);
    vrow[ks] = lds0 + L::V_BASE + swz_off<LP>(c, 2 * ks + h);
  }
  {
    const int rowlo = 4 * h + (i16 >> 2);
    const int sub = (i16 & 1) * 4;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      const int chunk = 4 * db + 2 * g2 + ((i16 & 3) >> 1);
      klo[db] = lds0 + L::K_BASE + swz_off<LP>(rowlo, chunk) + sub;
      khi[db] = lds0 + L::K_BASE + swz_off<LP>(rowlo + 8, chunk) + sub;
    }
  }

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) dqacc[db][i] = 0.f;
  // Element i of a score block that starts at key kv0 is key kv0 + 4h + 8 (i / 4) + i % 4; it is kept
  // when that key is at most min(query row, last key): one subtraction per block and one compare
  // with a constant per element.
  const int key_limit = min(q0w + c, seqlen_k - 1) - 4 * h;
  const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

  // The dP chain of every block starts from -delta instead of zero (the MFMA's C operand), so that
  // dS = P * dP needs no subtraction.  Costs sixteen registers (255 of 256 in use at 128 columns).
  const f32x16 dp_start = splat16(-delta);

  wait_vmem_all();
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
  constexpr int LOADS = TileLoader<DP, BKV, kDqWaves, PAD>::LOADS;
  constexpr int LOAD_EVERY = KS / LOADS;
  // INNER blocks lie in tiles that end before the workgroup's first query row: they are every
  // wave's own and need no mask, so the two tests fold away.
  auto block = [&](int j, auto half_tag, auto spread_tag, auto inner_tag) __attribute__((always_inline)) {
    constexpr int HALF = decltype(half_tag)::value;
    constexpr bool SPREAD = decltype(spread_tag)::value;
    constexpr bool INNER = decltype(inner_tag)::value;
    const int kt = j / 2 + 2, vt = j / 2 + 1;  // tiles loaded during this block (SPREAD)
    if (!INNER && j >= n_mine) {
      if (SPREAD) {  // not reached: skipped blocks lie in the last two tiles, which load nothing
        issue_k(kt);
        issue_v(vt);
      }
      return;
    }
    const unsigned kdst = lds_base + 2u * (unsigned)(L::K_BASE + (kt % L::K_STAGES) * L::TILE_ELEMS);
    const unsigned vdst = lds_base + 2u * (unsigned)(L::V_BASE + (vt % L::V_STAGES) * L::TILE_ELEMS);
    constexpr int HOFF = HALF * BLK * LP;
    f32x16 s = zero, dp;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      s = Elem<T>::mfma(ring[ks], qf[ks], s);
      if (SPREAD && ks % LOAD_EVERY == 0 && ks / LOAD_EVERY < LOADS) vload.issue_one(vt * BKV, vdst, ks / LOAD_EVERY);
      ring[ks] = lds_read_128(vrow[ks] + HOFF);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (!INNER && j >= n_full) {
      // Diagonal and ragged blocks: masked scores become -inf, their probabilities 0.  The empty asm
      // statement keeps this a branch that interior blocks skip (the test is cheap enough that the
      // optimiser would otherwise run it for every block).
      asm volatile("");
      const int lim = key_limit - j * BLK;
#pragma unroll
      for (int i = 0; i < 16; i++)
        if (8 * (i >> 2) + (i & 3) > lim) s[i] = -INFINITY;
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      dp = Elem<T>::mfma(ring[ks], gf[ks], ks == 0 ? dp_start : dp);
      if (SPREAD && ks % LOAD_EVERY == 0 && ks / LOAD_EVERY < LOADS) kload.issue_one(kt * BKV, kdst, ks / LOAD_EVERY);
      {
        s16x4 a0 = lds_read_tr(klo[ks % DB] + HOFF + 16 * (ks / DB) * LP);
        s16x4 a1 = lds_read_tr(khi[ks % DB] + HOFF + 16 * (ks / DB) * LP);
        ring[ks] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
#pragma unroll
      for (int i = part(16, KS, ks); i < part(16, KS, ks + 1); i++) {
        s[i] = fast_exp2(s[i] * scale_log2 - lse2);
      }
      asm volatile("" : "+v"(s));
      __builtin_amdgcn_sched_barrier(0);
    }
    // dS of the first 16 keys before the dQ MFMAs that need them, the rest beside those MFMAs.
    f32x8 lo, hi;
#pragma unroll
    for (int i = 0; i < 8; i++) lo[i] = s[i] * dp[i];
    s16x8 dsf[2];
    dsf[0] = Elem<T>::pack8(lo);
#pragma unroll
    for (int slot = 0; slot < KS; slot++) {
      constexpr int HALF_SLOTS = KS / 2;
      const int ks2 = slot / DB, db = slot % DB;
      dqacc[db] = Elem<T>::mfma(ring[slot], dsf[ks2], dqacc[db]);
      ring[slot] = lds_read_128(knext[slot] + (HALF == 0 ? BLK * LP : 0));
      if (slot < HALF_SLOTS) {
#pragma unroll
        for (int i = part(8, HALF_SLOTS, slot); i < part(8, HALF_SLOTS, slot + 1); i++)
          hi[i] = s[8 + i] * dp[8 + i];
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
    wait_vmem_all();
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
    block(2 * t, std::integral_constant<int, 0>{}, spread_tag, spread_tag);
    // knext -> K tile t+1 before the second block prefetches from it.
    const int dk = k_step(t);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) knext[ks] += dk;
    block(2 * t + 1, std::integral_constant<int, 1>{}, std::false_type{}, spread_tag);
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
                              p.dq.stride_seq, p.seqlen_q - q0w, hdim, true);
}


}  // namespace fa2
