// The LDS-direct forward kernels for 192 and 256 columns (one wave per SIMD, all 512 registers), in a
// translation unit of their own: see launch_direct in fa2_fwd_launch.hip.
#include "fa2_fwd.hpp"
#include "fa2_launch.hpp"

namespace fa2 {
namespace {

// At 256 columns only the padded variant is instantiated, also for a head dimension of exactly 256
// (it then switches no lane off): with the number of columns a run-time value the compiler keeps the
// kernel within its 512 registers, with a constant 256 it spills about forty of them, with reloads
// inside the tile loop, where they queue behind the tile loads (same counter).
template <typename T, bool PAD>
void launch_wide(int dp, const FwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  if (dp == 192)
    hipLaunchKernelGGL((fwd_direct_kernel<T, 192, kFwdBlockKV, PAD, false>), grid, block, 0, s, p);
  else
    hipLaunchKernelGGL((fwd_direct_kernel<T, 256, kFwdBlockKV, true, false>), grid, block, 0, s, p);
}

}  // namespace

void launch_fwd_direct_wide(bool bf16, int dp, bool pad, const FwdParams &p, dim3 grid, dim3 block, hipStream_t s) {
  if (bf16) {
    if (pad) launch_wide<__bf16, true>(dp, p, grid, block, s); else launch_wide<__bf16, false>(dp, p, grid, block, s);
  } else {
    if (pad) launch_wide<_Float16, true>(dp, p, grid, block, s); else launch_wide<_Float16, false>(dp, p, grid, block, s);
  }
}

}  // namespace fa2
