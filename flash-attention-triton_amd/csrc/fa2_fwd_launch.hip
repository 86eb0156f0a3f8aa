// Instantiates and launches the forward kernels.
#include "fa2_fwd.hpp"
#include "fa2_launch.hpp"

namespace fa2 {
namespace {

template <typename T, bool VEC>
void launch_generic(int dp, const FwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  switch (dp) {
    case 32: hipLaunchKernelGGL((fwd_kernel<T, 32, kFwdBlockKV, VEC>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((fwd_kernel<T, 64, kFwdBlockKV, VEC>), grid, block, 0, s, p); break;
    case 96: hipLaunchKernelGGL((fwd_kernel<T, 96, kFwdBlockKV, VEC>), grid, block, 0, s, p); break;
    case 128: hipLaunchKernelGGL((fwd_kernel<T, 128, kFwdBlockKV, VEC>), grid, block, 0, s, p); break;
    case 192: hipLaunchKernelGGL((fwd_kernel<T, 192, kFwdBlockKV, VEC>), grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL((fwd_kernel<T, 256, kFwdBlockKV, VEC>), grid, block, 0, s, p); break;
  }
}

template <typename T, bool PAD>
void launch_direct(int dp, const FwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  switch (dp) {
    case 32: hipLaunchKernelGGL((fwd_direct_kernel<T, 32, kFwdBlockKV, PAD>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((fwd_direct_kernel<T, 64, kFwdBlockKV, PAD>), grid, block, 0, s, p); break;
    case 96: hipLaunchKernelGGL((fwd_direct_kernel<T, 96, kFwdBlockKV, PAD>), grid, block, 0, s, p); break;
    case 128: hipLaunchKernelGGL((fwd_direct_kernel<T, 128, kFwdBlockKV, PAD>), grid, block, 0, s, p); break;
    case 192: hipLaunchKernelGGL((fwd_direct_kernel<T, 192, kFwdBlockKV, PAD>), grid, block, 0, s, p); break;
    default: hipLaunchKernelGGL((fwd_direct_kernel<T, 256, kFwdBlockKV, PAD>), grid, block, 0, s, p); break;
  }
}

template <typename T>
void launch(int dp, const FwdParams &p, dim3 grid, hipStream_t s) {
  const dim3 block(64 * kFwdWaves);
  if (fwd_direct_ok(dp, p)) {
    if (p.headdim == dp)
      launch_direct<T, false>(dp, p, grid, block, s);
    else
      launch_direct<T, true>(dp, p, grid, block, s);
    return;
  }
  if (p.vec)
    launch_generic<T, true>(dp, p, grid, block, s);
  else
    launch_generic<T, false>(dp, p, grid, block, s);
}

}  // namespace

void launch_fwd(bool bf16, int dp, const FwdParams &p, dim3 grid, hipStream_t s) {
  if (bf16)
    launch<__bf16>(dp, p, grid, s);
  else
    launch<_Float16>(dp, p, grid, s);
}

}  // namespace fa2
