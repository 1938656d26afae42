// Launch of the large-d GEMM-style log-sum-exp kernel.
#include "fs_lsegemm.hpp"

#include "fs_dispatch.hpp"

namespace fs {

int launch_lse_gemm(const LaunchArgs& a, int mode, int blocks, hipStream_t st) {
  if (mode == kVec)
    hipLaunchKernelGGL(lse_gemm_kernel<1>, dim3(blocks), dim3(512), 0, st, a);
  else if (mode == kArgmax)
    hipLaunchKernelGGL(lse_gemm_kernel<2>, dim3(blocks), dim3(512), 0, st, a);
  else
    hipLaunchKernelGGL(lse_gemm_kernel<0>, dim3(blocks), dim3(512), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

}  // namespace fs
