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

// PRE (exponents straight from the score MFMAs) is instantiated up to 128 columns: the sixteen registers
// of the chain's start value are more than the 256-column kernel has left.  The 192- and 256-column
// kernels live in a translation unit of their own (fa2_fwd_launch_wide.hip): compiled beside the
// narrower instantiations the 256-column kernel, which uses all 512 registers, came out with 40-60
// spilled registers and reloads inside its tile loop; alone it spills two, outside the loop.
template <typename T, bool PAD, bool PRE>
void launch_direct(int dp, const FwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  switch (dp) {
    case 32: hipLaunchKernelGGL((fwd_direct_kernel<T, 32, kFwdBlockKV, PAD, PRE>), grid, block, 0, s, p); break;
    case 64: hipLaunchKernelGGL((fwd_direct_kernel<T, 64, kFwdBlockKV, PAD, PRE>), grid, block, 0, s, p); break;
    case 96: hipLaunchKernelGGL((fwd_direct_kernel<T, 96, kFwdBlockKV, PAD, PRE>), grid, block, 0, s, p); break;
    case 128: hipLaunchKernelGGL((fwd_direct_kernel<T, 128, kFwdBlockKV, PAD, PRE>), grid, block, 0, s, p); break;
    default: launch_fwd_direct_wide(std::is_same<T, __bf16>::value, dp, PAD, p, grid, block, s); break;
  }
}

template <typename T>
void launch(int dp, bool folded, const FwdParams &p, dim3 grid, hipStream_t s) {
  const dim3 block(64 * kFwdWaves);
  if (fwd_direct_ok(dp, p)) {
    const bool pad = p.headdim != dp;
    if (folded) {
      if (pad) launch_direct<T, true, true>(dp, p, grid, block, s); else launch_direct<T, false, true>(dp, p, grid, block, s);
    } else {
      if (pad) launch_direct<T, true, false>(dp, p, grid, block, s); else launch_direct<T, false, false>(dp, p, grid, block, s);
    }
    return;
  }
  if (p.vec)
    launch_generic<T, true>(dp, p, grid, block, s);
  else
    launch_generic<T, false>(dp, p, grid, block, s);
}

}  // namespace

void launch_fwd(bool bf16, int dp, bool folded, const FwdParams &p, dim3 grid, hipStream_t s) {
  if (bf16)
    launch<__bf16>(dp, folded, p, grid, s);
  else
    launch<_Float16>(dp, folded, p, grid, s);
}

}  // namespace fa2
