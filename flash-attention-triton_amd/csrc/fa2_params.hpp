// Kernel parameter blocks and tile constants shared by the host-side C ABI and the device code.
#pragma once

#include <stdint.h>

namespace fa2 {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// One (batch, nheads, seqlen, headdim) tensor: base pointer and strides in elements.
struct Tensor4 {
  void *ptr;
  int64_t stride_batch, stride_head, stride_seq;
};

// Every MFMA kernel runs 4 waves per workgroup, each wave owning 32 rows of the operand that stays
// in registers: 128 query rows (forward, dQ) or 128 key rows (dK/dV) per workgroup.
constexpr int kFwdWaves = 4;
constexpr int kFwdBlockQ = 32 * kFwdWaves;
constexpr int kDqWaves = 4;
constexpr int kDqBlockQ = 32 * kDqWaves;
constexpr int kDkvWaves = 4;
constexpr int kDkvBlockKV = 32 * kDkvWaves;
// Rows of the streamed operand per LDS tile.
constexpr int kFwdBlockKV = 64;
constexpr int kDqBlockKV = 64;
constexpr int kDkvBlockQ = 64;

struct FwdParams {
  Tensor4 q, k, v, o;
  float *lse;
  int batch, nheads, seqlen_q, seqlen_k, headdim, seqlen_q_rounded;
  int n_qtiles;
  int head_group;  // (batch, head) pairs whose tiles are dispatched together (multiple of 8)
  float scale;       // softmax scale (natural units)
  float scale_log2;  // scale * log2(e)
  int vec;           // 16-byte global accesses are legal for every tensor
};

struct BwdParams {
  Tensor4 q, k, v, d_o, dq, dk, dv;
  Tensor4 o;         // only read by the dQ kernel when it also forms delta
  float *delta_out;  // where that kernel writes delta (the same buffer `delta` points to)
  // Sequence-parallel mode only: fp32 (batch * nheads, dq_accum_rows, headdim) accumulator the
  // key-tile kernel adds its dQ contributions to; dq_accum_rows is seqlen_q rounded up to the
  // kernel's 64-row query tile.
  float *dq_accum;
  int dq_accum_rows;
  const float *lse;
  const float *delta;
  int batch, nheads, seqlen_q, seqlen_k, headdim, seqlen_q_rounded;
  int n_tiles;  // key tiles (dK/dV kernel) or query tiles (dQ kernel)
  int head_group;  // (batch, head) pairs whose tiles are dispatched together (multiple of 8)
  float scale, scale_log2;
  int vec;
};

struct PreParams {
  Tensor4 o, d_o;
  float *delta;
  int batch, nheads, seqlen_q, headdim, seqlen_q_rounded;
  int vec;
};

}  // namespace fa2
