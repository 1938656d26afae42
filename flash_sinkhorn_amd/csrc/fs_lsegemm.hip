// Launch of the large-d GEMM-style log-sum-exp kernel.
#include "fs_lsegemm.hpp"

#include "fs_dispatch.hpp"

namespace fs {

int launch_lse_gemm(const LaunchArgs& a, bool vec, int blocks, hipStream_t st) {
  if (vec)
    hipLaunchKernelGGL(lse_gemm_kernel<true>, dim3(blocks), dim3(512), 0, st, a);
  else
    hipLaunchKernelGGL(lse_gemm_kernel<false>, dim3(blocks), dim3(512), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

}  // namespace fs
