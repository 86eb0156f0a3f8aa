// Instantiates and launches the dQ kernels and the delta preprocess.
#include "fa2_bwd_dq.hpp"
#include "fa2_launch.hpp"

namespace fa2 {
namespace {

template <typename T, bool FUSE_DELTA, bool PAD>
void launch_direct_pad(int dp, const BwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  switch (dp) {
    case 32: hipLaunchKernelGGL((bwd_dq_direct_kernel<T, 32, kDqBlockKV, FUSE_DELTA, PAD>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((bwd_dq_direct_kernel<T, 64, kDqBlockKV, FUSE_DELTA, PAD>), grid, block, 0, s, p); break;
    case 96: hipLaunchKernelGGL((bwd_dq_direct_kernel<T, 96, kDqBlockKV, FUSE_DELTA, PAD>), grid, block, 0, s, p); break;
    case 128: hipLaunchKernelGGL((bwd_dq_direct_kernel<T, 128, kDqBlockKV, FUSE_DELTA, PAD>), grid, block, 0, s, p); break;
    case 192: hipLaunchKernelGGL((bwd_dq_direct_kernel<T, 192, kDqBlockKV, FUSE_DELTA, PAD>), grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL((bwd_dq_direct_kernel<T, 256, kDqBlockKV, FUSE_DELTA, PAD>), grid, block, 0, s, p); break;
  }
}

template <typename T, bool FUSE_DELTA>
void launch_direct(int dp, const BwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  if (p.headdim == dp)
    launch_direct_pad<T, FUSE_DELTA, false>(dp, p, grid, block, s);
  else
    launch_direct_pad<T, FUSE_DELTA, true>(dp, p, grid, block, s);
}

template <typename T>
void launch(int dp, const BwdParams &p, dim3 grid, bool fuse_delta, hipStream_t s) {
  const dim3 block(64 * kDqWaves);
  if (dq_direct_ok(dp, p)) {
    if (fuse_delta)
      launch_direct<T, true>(dp, p, grid, block, s);
    else
      launch_direct<T, false>(dp, p, grid, block, s);
    return;
  }
  switch (dp) {
    case 32: hipLaunchKernelGGL((bwd_dq_kernel<T, 32, kDqBlockKV>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((bwd_dq_kernel<T, 64, kDqBlockKV>), grid, block, 0, s, p); break;
    case 96: hipLaunchKernelGGL((bwd_dq_kernel<T, 96, kDqBlockKV>), grid, block, 0, s, p); break;
    case 128: hipLaunchKernelGGL((bwd_dq_kernel<T, 128, kDqBlockKV>), grid, block, 0, s, p); break;
    case 192: hipLaunchKernelGGL((bwd_dq_kernel<T, 192, kDqBlockKV>), grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL((bwd_dq_kernel<T, 256, kDqBlockKV>), grid, block, 0, s, p); break;
  }
}

}  // namespace

void launch_dq(bool bf16, int dp, const BwdParams &p, dim3 grid, bool fuse_delta, hipStream_t s) {
  if (bf16)
    launch<__bf16>(dp, p, grid, fuse_delta, s);
  else
    launch<_Float16>(dp, p, grid, fuse_delta, s);
}

void launch_preprocess(bool bf16, const PreParams &p, dim3 grid, hipStream_t s) {
  if (bf16)
    hipLaunchKernelGGL((bwd_preprocess_kernel<__bf16>), grid, dim3(256), 0, s, p);
  else
    hipLaunchKernelGGL((bwd_preprocess_kernel<_Float16>), grid, dim3(256), 0, s, p);
}

}  // namespace fa2
