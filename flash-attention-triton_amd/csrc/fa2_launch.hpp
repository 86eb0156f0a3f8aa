// Kernel launchers, one translation unit per kernel family so that the library builds in parallel.
// `dp` is the padded head dimension of the table row in use (32, 64, 96, 128, 192 or 256); the
// launchers pick the LDS-direct fast kernel when the tensors allow it and the generic one otherwise.
#pragma once

#include <hip/hip_runtime.h>

#include "fa2_params.hpp"

namespace fa2 {

// Which kernel a launcher picked (reported to callers that label measurements).
enum KernelPath { kPathGeneric = 0, kPathDirect = 1 };

// The fast kernels need a head dimension that is a multiple of 8 (whole 16-byte chunks) up to 128
// (up to 256 in the forward and dQ kernels), 16-byte aligned rows and row offsets inside a tile that
// fit 32 bits.  A head dimension below the table row's padded one runs the padded variant of the
// kernel.
inline bool direct_stride_ok(const Tensor4 &t) { return t.stride_seq < (int64_t(1) << 24); }
inline bool direct_headdim(int dp, int headdim) {
  return headdim % 8 == 0 && headdim <= dp && (dp == 32 || dp == 64 || dp == 96 || dp == 128);
}
// The forward and dQ kernels, which stream K and V, also have fast variants for the rows of 192 and
// 256 columns (one wave per SIMD, all 160 KiB of LDS).
inline bool direct_headdim_kv_stream(int dp, int headdim) {
  return direct_headdim(dp, headdim) || (headdim % 8 == 0 && headdim <= dp && (dp == 192 || dp == 256));
}
inline bool fwd_direct_ok(int dp, const FwdParams &p) {
  return p.vec && direct_headdim_kv_stream(dp, p.headdim) && direct_stride_ok(p.q) && direct_stride_ok(p.k) &&
         direct_stride_ok(p.v);
}
inline bool dq_direct_ok(int dp, const BwdParams &p) {
  return p.vec && direct_headdim_kv_stream(dp, p.headdim) && direct_stride_ok(p.k) && direct_stride_ok(p.v);
}
inline bool dkdv_direct_ok(int dp, const BwdParams &p) {
  return p.vec && direct_headdim(dp, p.headdim) && direct_stride_ok(p.q) && direct_stride_ok(p.d_o) &&
         direct_stride_ok(p.k) && direct_stride_ok(p.v);
}
// The sequence-parallel (atomic dQ) kernels: the fast dK/dV kernel's conditions, a head dimension
// of exactly 32, 64 or 128 and 16-byte aligned dq rows.
inline bool seqpar_atomic_ok(int dp, const BwdParams &p) {
  return dkdv_direct_ok(dp, p) && p.headdim == dp && (dp == 32 || dp == 64 || dp == 128);
}

// Size of the head groups map_workgroup is given, for `heads` (batch, head) pairs and a table group
// size `group`: the heads are split into floor(heads / group) groups of (nearly) equal size, each a
// multiple of 8 so that a head stays on one XCD.  Equal groups, because a small last group would start
// its heaviest tiles late and finish them alone (96 heads as 64 + 32 cost 5 % against one group of 96);
// fewer than two table groups' worth of heads form a single group, walked heaviest tile first over
// the whole grid.
inline int equal_head_groups(int group, int64_t heads) {
  const int64_t n_groups = heads / group > 0 ? heads / group : 1;
  const int64_t per_group = (heads + n_groups - 1) / n_groups;
  return (int)((per_group + 7) / 8 * 8);
}

// bf16 != 0 selects the bf16 kernels, otherwise fp16.
// folded: the LDS-direct forward takes its exponents straight from the score MFMAs (Q fragments
// multiplied by scale * log2(e) and rounded once); the generic forward ignores it.
void launch_fwd(bool bf16, int dp, bool folded, const FwdParams &p, dim3 grid, hipStream_t s);
// The 192- and 256-column LDS-direct forward kernels (dp is 192 or 256), instantiated apart from the others.
void launch_fwd_direct_wide(bool bf16, int dp, bool pad, const FwdParams &p, dim3 grid, dim3 block, hipStream_t s);
void launch_preprocess(bool bf16, const PreParams &p, dim3 grid, hipStream_t s);
// fuse_delta: the fast dQ kernel also forms delta from O and dO (dq_direct_ok must hold).
void launch_dq(bool bf16, int dp, const BwdParams &p, dim3 grid, bool fuse_delta, hipStream_t s);
// With p.dq_accum set the sequence-parallel kernel runs: dK, dV and atomic dQ contributions.
void launch_dkdv(bool bf16, int dp, const BwdParams &p, dim3 grid, hipStream_t s);
void launch_dq_accum_zero(float *acc, int64_t floats, hipStream_t s);
void launch_dq_accum_convert(bool bf16, const BwdParams &p, hipStream_t s);

}  // namespace fa2
