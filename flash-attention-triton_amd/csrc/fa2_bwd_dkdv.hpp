// dK/dV half of the causal FlashAttention-2 backward for gfx950; the split of the backward into
// a dK/dV kernel and a dQ kernel is described at the top of fa2_bwd_dq.hpp.
#pragma once

#include <type_traits>

#include "fa2_common.hpp"

namespace fa2 {

// ------------------------------------------------------------------------------------------
// dK/dV kernel (key-tile parallel).
// ------------------------------------------------------------------------------------------

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
  map_workgroup(blockIdx.x, BH, p.n_tiles, p.head_group, bh, kt);
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
// deep, one workgroup barrier per tile.  See fa2_common.hpp for the swizzle and TileLoader.
// ------------------------------------------------------------------------------------------
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
  static constexpr int LP = lds_pitch(DP);  // LDS row pitch
  static constexpr int TILE_ELEMS = BQ * LP;
  // One stage: Q tile, dO tile, then lse*log2e and delta as floats (2 shorts each).
  static constexpr int STAGE_ELEMS = 2 * TILE_ELEMS + 4 * BQ;
  static constexpr int STAGES = 3;
  static constexpr int PATCH_ELEMS = kDkvWaves * 32 * (DP + 8);
  // Beyond the stages: room for the workgroup's 128 V rows on their way into registers (its K rows
  // pass through the third stage before the third tile is requested).
  static constexpr int V_ROWS_BASE = STAGES * STAGE_ELEMS;
  static constexpr int TOTAL_ELEMS = V_ROWS_BASE + 2 * TILE_ELEMS;
  static_assert(V_ROWS_BASE >= PATCH_ELEMS, "the output patch overlays the stages");
};

// PAD: the head dimension is a multiple of 8 below DP; the columns beyond it are zeros in LDS and in
// the register fragments, and are not stored.
//
// ATOMIC_DQ: the kernel is the whole backward of the reference's sequence-parallel mode
// (_triton_kernels_v2.py:336-339, 466-494): besides dK and dV of its key tile it forms, for every
// 32-row query block, the block's contribution dS K to dQ (a fifth GEMM) and adds it with fp32
// global atomics into p.dq_accum, which the caller zeroed and converts afterwards.  dS has the key
// index across lanes, the contraction index of that GEMM, so it travels through LDS: every wave
// writes its 32 key rows of dS ([key][query], two buffers used alternately), the workgroup meets at
// a barrier, and wave w multiplies column block w % DB of K by the dS rows of key group w / DB
// (at DB = 4: 32 of the 128 columns each, all 128 keys).  The result leaves the MFMA with the head
// dimension across lanes, so every atomic instruction covers two 128-byte row segments.
template <typename T, int DP, int BQ, bool PAD, bool ATOMIC_DQ = false>
__global__ __launch_bounds__(64 * kDkvWaves, (DP <= 64 && !ATOMIC_DQ ? 2 : 1)) void bwd_dkdv_direct_kernel(const BwdParams p) {
  using L = DkvDirectLayout<DP, BQ>;
  constexpr int KS = DP / 16, DB = DP / 32, LP = L::LP;
  constexpr int NTHREADS = 64 * kDkvWaves;
  static_assert(BQ == 64 && KS == 2 * DB, "schedule is written for 64-row query tiles of two blocks");
  static_assert(BQ <= NTHREADS, "one thread per row loads lse and delta");
  static_assert((L::STAGE_ELEMS * 2) % 256 == 0, "stages must start on a 256-byte LDS bank line");
  static_assert(!ATOMIC_DQ || (kDkvWaves % DB == 0 && !PAD), "the dQ GEMM splits column blocks evenly over the waves");
  // dS exchange area: kDkvBlockKV key rows of 32 queries, pitch 36 halves (72 bytes: rows start on
  // 8-byte words and fall on different banks), two buffers.
  constexpr int DS_PITCH = 36;
  constexpr int DS_BUF_ELEMS = kDkvBlockKV * DS_PITCH;
  constexpr int DS_BASE = (L::TOTAL_ELEMS + 7) / 8 * 8;
  constexpr int KG = ATOMIC_DQ ? kDkvBlockKV * DB / kDkvWaves : 32;  // keys a wave contracts over in the dQ GEMM
  constexpr int KSQ = KG / 16;                                        // its MFMAs per block

  __shared__ __attribute__((aligned(1024))) short smem[ATOMIC_DQ ? DS_BASE + 2 * DS_BUF_ELEMS : L::TOTAL_ELEMS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31, h = lane >> 5;
  const int i16 = lane & 15, g2 = (lane >> 4) & 1;

  // Key tile 0 has the longest query range: issue tiles in ascending order (heaviest first).
  const int BH = p.batch * p.nheads;
  int bh, kt;  // key tile 0 has the longest query range: rank == key tile
  map_workgroup(blockIdx.x, BH, p.n_tiles, p.head_group, bh, kt);
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

  const int hdim = PAD ? p.headdim : DP;
  // (Bases and strides are restated as scalars: with the K and V loaders below in the same kernel the
  // compiler otherwise forms the spread loads' addresses on the vector unit, 24 more vector
  // instructions per tile.)
  const TileLoader<DP, BQ, kDkvWaves, PAD> qload(uniform_ptr(Q), (int64_t)uniform64((uint64_t)p.q.stride_seq), hdim / 8),
      gload(uniform_ptr(DO), (int64_t)uniform64((uint64_t)p.d_o.stride_seq), hdim / 8);
  const int seqlen_q = p.seqlen_q;
  const float scale_log2 = p.scale_log2;

  // First query tile that can see this key tile (row >= col), aligned down to BQ.
  const int q_begin = (kv0 / BQ) * BQ;
  const int n_tiles = (seqlen_q > q_begin) ? (seqlen_q - q_begin + BQ - 1) / BQ : 0;
  const int n_inside = (seqlen_q - q_begin) / BQ;  // tiles whose every row exists
  // Tiles that touch the diagonal of this key tile (their blocks need the causal mask).
  const int n_diag = min(n_tiles, (kv0 + kDkvBlockKV - q_begin + BQ - 1) / BQ);

  const unsigned lds_base = lds_u32(smem);  // LDS byte address of smem
  if (PAD) {
    zero_lds<NTHREADS>(smem, L::TOTAL_ELEMS);
    __syncthreads();
  }
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
  // lse and delta of a tile go through registers into the stage's statistics area.  load_stats
  // only issues the two loads: any arithmetic on a loaded value makes the wave wait for it on the
  // spot (and, loads returning in order, for every tile load issued before it), once per tile and
  // with nothing else to run on the SIMD.  The values are first touched a tile later, in
  // store_stats.  Rows beyond the sequence take the last row's values (finite; the row mask zeroes
  // their probabilities).
  float lse_reg = 0.f, delta_reg = 0.f;
  auto load_stats = [&](int t) {
    if (tid < BQ) {
      const int row = min(q_begin + t * BQ + tid, seqlen_q - 1);
      lse_reg = LSE[row];
      delta_reg = DELTA[row];
    }
  };
  auto store_stats = [&](int t) {
    float *sl = reinterpret_cast<float *>(smem + (t % L::STAGES) * L::STAGE_ELEMS + 2 * L::TILE_ELEMS);
    // The compiler's own wait for the two loads counts the atomics issued since as if everything
    // completed in order; atomics complete ahead of older loads.
    if (ATOMIC_DQ) wait_vmem_all();
    if (tid < BQ) {
      sl[tid] = lse_reg * kLog2e;
      sl[BQ + tid] = -delta_reg;  // negated: it is the accumulator the dP MFMAs start from
    }
  };
  // Prologue: the global loads of the first two tiles and of the workgroup's K and V rows are
  // issued before anything waits, so that the workgroup pays one memory latency.  K and V travel
  // like tiles: LDS-direct loads that cover whole rows, K into the third stage (whose tile is
  // requested once every wave has taken its fragments out; it is first read near the end of tile 1),
  // V behind the stages.  Loaded straight into registers, a wave's sixteen fragment loads touch 32
  // rows each, and a workgroup, alone on its CU, spent 5 of its first 7 microseconds getting its
  // loads accepted by the memory pipeline.  Rows beyond the keys are read from the last key row:
  // finite values whose dK and dV rows are never stored.
  constexpr unsigned K_LO = 2u * (unsigned)(2 * L::STAGE_ELEMS), K_HI = K_LO + 2u * (unsigned)L::TILE_ELEMS;
  constexpr unsigned V_LO = 2u * (unsigned)L::V_ROWS_BASE, V_HI = V_LO + 2u * (unsigned)L::TILE_ELEMS;
  {
    const TileLoader<DP, BQ, kDkvWaves, PAD> kload(K + (int64_t)kv0 * p.k.stride_seq, p.k.stride_seq, hdim / 8),
        vload(V + (int64_t)kv0 * p.v.stride_seq, p.v.stride_seq, hdim / 8);
    const int k_rows = p.seqlen_k - kv0;  // key rows of this tile that exist (>= 1)
    if (n_tiles > 0) issue_tile(0);
    if (k_rows >= BQ) kload.issue(0, lds_base + K_LO); else kload.issue_clamped(0, k_rows, lds_base + K_LO);
    if (k_rows >= 2 * BQ) kload.issue(BQ, lds_base + K_HI); else kload.issue_clamped(BQ, k_rows, lds_base + K_HI);
    if (k_rows >= BQ) vload.issue(0, lds_base + V_LO); else vload.issue_clamped(0, k_rows, lds_base + V_LO);
    if (k_rows >= 2 * BQ) vload.issue(BQ, lds_base + V_HI); else vload.issue_clamped(BQ, k_rows, lds_base + V_HI);
    if (n_tiles > 1) issue_tile(1);
  }
  // B operands of the dQ GEMM: lane (c, h) holds column 32 (wave % DB) + c of K for the keys of key
  // group wave / DB, element j of k-step s being key 16 s + 8 (j / 4) + 4 h + j % 4 of the group (the
  // order in which the transposing LDS reads deliver the dS rows).
  s16x8 kb[KSQ];
  float *dq_rows = nullptr;  // this lane's column of the fp32 dQ accumulator, row 4 h of the sequence
  if (ATOMIC_DQ) {
    const int col = 32 * (wave % DB) + c;
    const int key0 = kv0 + (wave / DB) * KG;
#pragma unroll
    for (int ks = 0; ks < KSQ; ks++)
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const int key = key0 + 16 * ks + 8 * (j >> 2) + 4 * h + (j & 3);
        kb[ks][j] = key < p.seqlen_k ? K[(int64_t)key * p.k.stride_seq + col] : (short)0;
      }
    dq_rows = p.dq_accum + ((int64_t)bh * p.dq_accum_rows + 4 * h) * DP + col;
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
    qrow[ks] = lds0 + swz_off<LP>(c, 2 * ks + h);
    qnext[ks] = qrow[ks];
  }
  {
    const int rowlo = 4 * h + (i16 >> 2);
    const int sub = (i16 & 1) * 4;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      const int chunk = 4 * db + 2 * g2 + ((i16 & 3) >> 1);
      qlo[db] = lds0 + swz_off<LP>(rowlo, chunk) + sub;
      qhi[db] = lds0 + swz_off<LP>(rowlo + 8, chunk) + sub;
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
  // Element i of a block that starts at query row qb is row qb + 4h + 8 (i / 4) + i % 4; it is kept
  // when key column <= row < seqlen_q, tested as one unsigned compare: (row - column) < (seqlen_q - column).
  const int kvcol = kv0w + c;
  const int row_shift = 4 * h - kvcol;  // row - column = qb + 8 (i / 4) + i % 4 + row_shift
  const unsigned row_span = (unsigned)max(seqlen_q - kvcol, 0);

#pragma unroll
  for (int t = 0; t < L::STAGES; t++) {
    lse_reg = l3[t];
    delta_reg = d3[t];
    store_stats(t);
  }
  wait_vmem_all();
  __syncthreads();
  // B operands: lane (c, h) holds row kv0w + c of K and of V, columns 16 ks + 8 h + j.
  s16x8 kf[KS], vf[KS];
  {
    const int r = 32 * (wave & 1) + c;  // row inside the 64-row half the wave's keys lie in
    const lds_cptr krows = lds0 + (int)(((wave >> 1) ? K_HI : K_LO) / 2);
    const lds_cptr vrows = lds0 + (int)(((wave >> 1) ? V_HI : V_LO) / 2);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      kf[ks] = lds_read_128(krows + swz_off<LP>(r, 2 * ks + h));
      vf[ks] = lds_read_128(vrows + swz_off<LP>(r, 2 * ks + h));
    }
  }
  // Every wave has its K fragments: the third stage is free for its tile.
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();
  if (n_tiles > 2) issue_tile(2);
  // Two rings of A fragments, preloaded with the Q rows and the dO rows of block 0.
  s16x8 ring[KS], ringb[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) ring[ks] = lds_read_128(qrow[ks]);
#pragma unroll
  for (int ks = 0; ks < KS; ks++) ringb[ks] = lds_read_128(qrow[ks] + L::TILE_ELEMS);

  // One 32-row query block.  HALF selects the half-tile; MASKED switches the causal/row masks on.
  // With SPREAD the block also issues the global->LDS loads of tile `lt`, one every few units:
  // issued back to back by all waves after a barrier they queue up in the memory pipeline, and a
  // wave whose load cannot issue cannot issue its MFMAs either.
  auto block = [&](int qb, auto half_tag, auto masked_tag, auto spread_tag, int lt) {
    constexpr int HALF = decltype(half_tag)::value;
    constexpr bool MASKED = decltype(masked_tag)::value;
    constexpr bool SPREAD = decltype(spread_tag)::value;
    constexpr int LOADS = TileLoader<DP, BQ, kDkvWaves, PAD>::LOADS;
    constexpr int EVERY = 4 * KS / (2 * LOADS);  // units between loads: both tiles' loads fit the block
    static_assert(EVERY >= 1 && (2 * LOADS - 1) * EVERY < 4 * KS, "the block must have room for both tiles' loads");
    const unsigned ldst = lds_base + 2u * (unsigned)((lt % L::STAGES) * L::STAGE_ELEMS);
    const int lrow0 = q_begin + lt * BQ;
    auto spread_load = [&](int unit) {  // unit: 0 .. 4 KS - 1 over the four GEMMs
      if (SPREAD && unit % EVERY == 0 && unit / EVERY < 2 * LOADS) {
        const int li = unit / EVERY;
        if (li < LOADS) qload.issue_one(lrow0, ldst, li);
        else gload.issue_one(lrow0, ldst + 2u * L::TILE_ELEMS, li - LOADS);
      }
    };
    constexpr int QOFF = HALF * 32 * LP;          // Q rows of this block inside the tile
    constexpr int GOFF = QOFF + L::TILE_ELEMS;    // dO rows of this block
    typedef const __attribute__((address_space(3))) f32x4 *stat4_ptr;

    // ---- S = Q K^T (ring: Q rows -> dO^T); statistics of the 16 rows this lane holds ---------
    f32x16 s, dp;
    f32x4 l4[4], d4[4];  // d4: minus delta of the rows this lane holds
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (ks == 0) VgprMfma<T>::first(s, ring[ks], kf[ks]);
      else VgprMfma<T>::next(s, ring[ks], kf[ks]);
      spread_load(ks);
      {
        s16x4 a0 = lds_read_tr(qlo[ks % DB] + GOFF + 16 * (ks / DB) * LP);
        s16x4 a1 = lds_read_tr(qhi[ks % DB] + GOFF + 16 * (ks / DB) * LP);
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
    const int rel = qb + row_shift;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      // The chain starts from -delta, so that dS = P * dP needs no subtraction.
      if (ks == 0)
        dp = __builtin_shufflevector(__builtin_shufflevector(d4[0], d4[1], 0, 1, 2, 3, 4, 5, 6, 7),
                                     __builtin_shufflevector(d4[2], d4[3], 0, 1, 2, 3, 4, 5, 6, 7), 0, 1, 2,
                                     3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
      VgprMfma<T>::next(dp, ringb[ks], vf[ks]);
      spread_load(KS + ks);
      {
        s16x4 a0 = lds_read_tr(qlo[ks % DB] + QOFF + 16 * (ks / DB) * LP);
        s16x4 a1 = lds_read_tr(qhi[ks % DB] + QOFF + 16 * (ks / DB) * LP);
        ringb[ks] = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      if (ks == 0) settle(s);  // after the S chain's last MFMA and before the first read of S
#pragma unroll
      for (int i = part(16, KS, ks); i < part(16, KS, ks + 1); i++) {
        float x = fast_exp2(s[i] * scale_log2 - l4[i >> 2][i & 3]);
        if (MASKED && (unsigned)(rel + (8 * (i >> 2) + (i & 3))) >= row_span) x = 0.f;
        s[i] = x;  // P takes the place of S
      }
      asm volatile("" : "+v"(s));
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x8 plo = {s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7]};
    f32x8 phi = {s[8], s[9], s[10], s[11], s[12], s[13], s[14], s[15]};
    const s16x8 pf[2] = {Elem<T>::pack8(plo), Elem<T>::pack8(phi)};
    // ---- dV^T += dO^T P (ring: dO^T -> Q rows of the next block); dS arithmetic under the MFMAs
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      dvacc[ks % DB] = Elem<T>::mfma(ring[ks], pf[ks / DB], dvacc[ks % DB]);
      spread_load(2 * KS + ks);
      ring[ks] = lds_read_128(qnext[ks] + (HALF == 0 ? 32 * LP : 0));
      if (ks == 0) settle(dp);
#pragma unroll
      for (int i = part(16, KS, ks); i < part(16, KS, ks + 1); i++) dp[i] = s[i] * dp[i];  // dS takes the place of dP
      asm volatile("" : "+v"(dp));
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x8 dlo = {dp[0], dp[1], dp[2], dp[3], dp[4], dp[5], dp[6], dp[7]};
    f32x8 dhi = {dp[8], dp[9], dp[10], dp[11], dp[12], dp[13], dp[14], dp[15]};
    const s16x8 dsf[2] = {Elem<T>::pack8(dlo), Elem<T>::pack8(dhi)};
    if (ATOMIC_DQ) {
      // This lane's key row of dS: element j of dsf[t] is query 16 t + 8 (j / 4) + 4 h + j % 4.
      short *row = smem + DS_BASE + HALF * DS_BUF_ELEMS + (32 * wave + c) * DS_PITCH + 4 * h;
#pragma unroll
      for (int t2 = 0; t2 < 2; t2++)
#pragma unroll
        for (int g = 0; g < 2; g++) {
          const s16x4 w4 = {dsf[t2][4 * g], dsf[t2][4 * g + 1], dsf[t2][4 * g + 2], dsf[t2][4 * g + 3]};
          *reinterpret_cast<s16x4 *>(row + 16 * t2 + 8 * g) = w4;
        }
    }
    // ---- dK^T += Q^T dS (ringb: Q^T -> dO rows of the next block) ------------------------------
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      dkacc[ks % DB] = Elem<T>::mfma(ringb[ks], dsf[ks / DB], dkacc[ks % DB]);
      spread_load(3 * KS + ks);
      ringb[ks] = lds_read_128(qnext[ks] + L::TILE_ELEMS + (HALF == 0 ? 32 * LP : 0));
      __builtin_amdgcn_sched_barrier(0);
    }
    if (ATOMIC_DQ) {
      // ---- dQ[block] += dS K: every wave's dS rows are in LDS after this barrier (the buffer of
      // the block before is being read by nobody: all waves passed that block's barrier) --------
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      const short *frag = smem + DS_BASE + HALF * DS_BUF_ELEMS +
                          ((wave / DB) * KG + 4 * h + (i16 >> 2)) * DS_PITCH + 16 * g2 + 4 * (i16 & 3);
      f32x16 dqb = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KSQ; ks++) {
        const s16x8 a = lds_read_tr_frag(frag + 16 * ks * DS_PITCH, DS_PITCH);
        dqb = Elem<T>::mfma(a, kb[ks], dqb);
      }
      // Element i is query row qb + 4 h + 8 (i / 4) + i % 4, this lane's column.  Rows up to the end
      // of the last 64-row tile exist in the accumulator; masked rows add zeros.
      float *dst = dq_rows + (int64_t)qb * DP;
#pragma unroll
      for (int i = 0; i < 16; i++)
        __builtin_amdgcn_global_atomic_fadd_f32(
            (__attribute__((address_space(1))) float *)(dst + (8 * (i >> 2) + (i & 3)) * DP), dqb[i]);
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
    wait_vmem_all();
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

  short *patch = smem + wave * 32 * (DP + 8);
  store_transposed_acc<T, DP>(dvacc, 1.0f, patch, DV + (int64_t)kv0w * p.dv.stride_seq,
                              p.dv.stride_seq, p.seqlen_k - kv0w, hdim, true);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  store_transposed_acc<T, DP>(dkacc, p.scale, patch, DK + (int64_t)kv0w * p.dk.stride_seq,
                              p.dk.stride_seq, p.seqlen_k - kv0w, hdim, true);
}

// ---- fp32 dQ accumulator of the sequence-parallel mode ------------------------------------------
// Cleared by a kernel, not a memset node, so that callers may capture the backward in a HIP graph.
__global__ __launch_bounds__(256) void dq_accum_zero_kernel(float *acc, int64_t n4) {
  const f32x4 z = {0.f, 0.f, 0.f, 0.f};
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (int64_t)gridDim.x * 256)
    reinterpret_cast<f32x4 *>(acc)[i] = z;
}

// dq = scale * accumulator, rounded once to the tensor's type (the reference's dq.copy_(dq_accum),
// flash_attention_2.py:277, with the scale the kernel left out).  One thread per 8 columns.
template <typename T>
__global__ __launch_bounds__(256) void dq_accum_convert_kernel(const BwdParams p) {
  const int cpr = p.headdim / 8;  // headdim is a multiple of 32 in this mode
  const int64_t total = (int64_t)p.batch * p.nheads * p.seqlen_q * cpr;
  for (int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x; id < total; id += (int64_t)gridDim.x * 256) {
    const int cc = (int)(id % cpr);
    const int64_t r = id / cpr;
    const int row = (int)(r % p.seqlen_q);
    const int bh = (int)(r / p.seqlen_q);
    const int b = bh / p.nheads, hd = bh % p.nheads;
    const float *src = p.dq_accum + ((int64_t)bh * p.dq_accum_rows + row) * p.headdim + cc * 8;
    const f32x4 lo = *reinterpret_cast<const f32x4 *>(src), hi = *reinterpret_cast<const f32x4 *>(src + 4);
    const f32x8 x = {lo[0] * p.scale, lo[1] * p.scale, lo[2] * p.scale, lo[3] * p.scale,
                     hi[0] * p.scale, hi[1] * p.scale, hi[2] * p.scale, hi[3] * p.scale};
    short *dst = (short *)p.dq.ptr + b * p.dq.stride_batch + hd * p.dq.stride_head + (int64_t)row * p.dq.stride_seq + cc * 8;
    *reinterpret_cast<s16x8 *>(dst) = Elem<T>::pack8(x);
  }
}

}  // namespace fa2
