// Instantiates and launches the dK/dV kernels.
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

template <typename T>
void launch(int dp, const BwdParams &p, dim3 grid, hipStream_t s) {
  const dim3 block(64 * kDkvWaves);
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

}  // namespace fa2
