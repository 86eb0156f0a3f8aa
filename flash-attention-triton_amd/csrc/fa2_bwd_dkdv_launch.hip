// Instantiates and launches the dK/dV kernels.
#include <algorithm>

#include "fa2_bwd_dkdv.hpp"
#include "fa2_launch.hpp"

namespace fa2 {
namespace {

template <typename T, bool PAD>
void launch_direct(int dp, const BwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  switch (dp) {
    case 32: hipLaunchKernelGGL((bwd_dkdv_direct_kernel<T, 32, kDkvBlockQ, PAD>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((bwd_dkdv_direct_kernel<T, 64, kDkvBlockQ, PAD>), grid, block, 0, s, p); break;
    case 96: hipLaunchKernelGGL((bwd_dkdv_direct_kernel<T, 96, kDkvBlockQ, PAD>), grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL((bwd_dkdv_direct_kernel<T, 128, kDkvBlockQ, PAD>), grid, block, 0, s, p); break;
  }
}

// The sequence-parallel kernels exist for 32, 64 and 128 columns (column blocks must divide the
// four waves).
template <typename T>
void launch_atomic(int dp, const BwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  switch (dp) {
    case 32: hipLaunchKernelGGL((bwd_dkdv_direct_kernel<T, 32, kDkvBlockQ, false, true>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((bwd_dkdv_direct_kernel<T, 64, kDkvBlockQ, false, true>), grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL((bwd_dkdv_direct_kernel<T, 128, kDkvBlockQ, false, true>), grid, block, 0, s, p); break;
  }
}

template <typename T>
void launch(int dp, const BwdParams &p, dim3 grid, hipStream_t s) {
  const dim3 block(64 * kDkvWaves);
  if (p.dq_accum != nullptr) {  // the caller checked seqpar_atomic_ok
    launch_atomic<T>(dp, p, grid, block, s);
    return;
  }
  if (dkdv_direct_ok(dp, p)) {
    if (p.headdim == dp)
      launch_direct<T, false>(dp, p, grid, block, s);
    else
      launch_direct<T, true>(dp, p, grid, block, s);
    return;
  }
  switch (dp) {
    case 32: hipLaunchKernelGGL((bwd_dkdv_kernel<T, 32, kDkvBlockQ>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((bwd_dkdv_kernel<T, 64, kDkvBlockQ>), grid, block, 0, s, p); break;
    case 96: hipLaunchKernelGGL((bwd_dkdv_kernel<T, 96, kDkvBlockQ>), grid, block, 0, s, p); break;
    case 128: hipLaunchKernelGGL((bwd_dkdv_kernel<T, 128, kDkvBlockQ>), grid, block, 0, s, p); break;
    case 192: hipLaunchKernelGGL((bwd_dkdv_kernel<T, 192, kDkvBlockQ>), grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL((bwd_dkdv_kernel<T, 256, kDkvBlockQ>), grid, block, 0, s, p); break;
  }
}

}  // namespace

void launch_dkdv(bool bf16, int dp, const BwdParams &p, dim3 grid, hipStream_t s) {
  if (bf16)
    launch<__bf16>(dp, p, grid, s);
  else
    launch<_Float16>(dp, p, grid, s);
}

void launch_dq_accum_zero(float *acc, int64_t floats, hipStream_t s) {
  const int64_t n4 = floats / 4;  // the accumulator is a multiple of 32 columns wide
  const unsigned blocks = (unsigned)std::min<int64_t>((n4 + 255) / 256, 4096);
  hipLaunchKernelGGL(dq_accum_zero_kernel, dim3(blocks), dim3(256), 0, s, acc, n4);
}

void launch_dq_accum_convert(bool bf16, const BwdParams &p, hipStream_t s) {
  const int64_t total = (int64_t)p.batch * p.nheads * p.seqlen_q * (p.headdim / 8);
  const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 8192);
  if (bf16)
    hipLaunchKernelGGL((dq_accum_convert_kernel<__bf16>), dim3(blocks), dim3(256), 0, s, p);
  else
    hipLaunchKernelGGL((dq_accum_convert_kernel<_Float16>), dim3(blocks), dim3(256), 0, s, p);
}

}  // namespace fa2
