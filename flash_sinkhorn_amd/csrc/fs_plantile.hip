// Launches of the d <= 128 plan-product / c-transform kernel on fp16 planes.
#include "fs_plantile.hpp"

#include "fs_dispatch.hpp"

namespace fs {

template <int DP, int MODE>
static int launch_rb(const LaunchArgs& a, int rb, int blocks, hipStream_t st) {
  if (rb == 2)
    hipLaunchKernelGGL((plan_tile_kernel<DP, 2, MODE>), dim3(blocks), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL((plan_tile_kernel<DP, 1, MODE>), dim3(blocks), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

template <int MODE>
static int launch_dp(const LaunchArgs& a, int dp, int rb, int blocks, hipStream_t st) {
  switch (dp) {
    case 16: return launch_rb<16, MODE>(a, rb, blocks, st);
    case 32: return launch_rb<32, MODE>(a, rb, blocks, st);
    case 64: return launch_rb<64, MODE>(a, rb, blocks, st);
    case 128:
      hipLaunchKernelGGL((plan_tile_kernel<128, 1, MODE>), dim3(blocks), dim3(256), 0, st, a);
      return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
  }
  return FS_ERR_UNSUPPORTED;
}

int launch_plan_tile(const LaunchArgs& a, int mode, int dp, int rb, int blocks, hipStream_t st) {
  if (mode == kMat) return launch_dp<kMat>(a, dp, rb, blocks, st);
  if (mode == kVec) return launch_dp<kVec>(a, dp, rb, blocks, st);
  if (mode == kArgmax) return launch_dp<kArgmax>(a, dp, rb, blocks, st);
  if (mode == kMat5) {  // one row block per wavefront
    switch (dp) {
      case 16: hipLaunchKernelGGL((plan_tile_kernel<16, 1, kMat5>), dim3(blocks), dim3(256), 0, st, a); break;
      case 32: hipLaunchKernelGGL((plan_tile_kernel<32, 1, kMat5>), dim3(blocks), dim3(256), 0, st, a); break;
      case 64: hipLaunchKernelGGL((plan_tile_kernel<64, 1, kMat5>), dim3(blocks), dim3(256), 0, st, a); break;
      case 128: hipLaunchKernelGGL((plan_tile_kernel<128, 1, kMat5>), dim3(blocks), dim3(256), 0, st, a); break;
      default: return FS_ERR_UNSUPPORTED;
    }
    return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
  }
  return FS_ERR_BAD_ARGUMENT;
}

}  // namespace fs
