// Launch of the large-d GEMM-style log-sum-exp kernel.
#include "fs_lsegemm.hpp"

#include "fs_dispatch.hpp"

namespace fs {

int launch_lse_gemm_sweep(const LaunchArgs& a, hipStream_t st) {
  // what the kernel takes for granted
  const Side& s0 = a.side[0];
  const Side& s1 = a.side[1];
  if (a.sel == nullptr || a.col_part == nullptr || s0.part_ms == nullptr || a.sw_splits < 2 ||
      (a.sw_splits & 1) || a.sw_splits > s0.splits || a.sw_chunk <= 0 || a.sw_chunk % kGemmRows != 0 ||
      (long long)(a.sw_splits / 2) * a.sw_chunk < s0.nk ||
      (long long)(a.sw_splits / 2 - 1) * a.sw_chunk >= s0.nk || s0.nq != s1.nk || s0.nk != s1.nq ||
      s0.igroups != (s0.nq + kGemmRows - 1) / kGemmRows || s0.qplanes == nullptr ||
      s0.kplanes == nullptr || s1.kb0 == nullptr)
    return FS_ERR_BAD_ARGUMENT;
  // (a multiple of 8 workgroups: each XCD takes an eighth of the work items)
  const int per_xcd = (s0.igroups * (a.sw_splits / 2) + 7) / 8;
  hipLaunchKernelGGL(lse_gemm_kernel<3>, dim3(8 * per_xcd), dim3(512), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

int launch_lse_gemm(const LaunchArgs& a, int mode, int blocks, hipStream_t st) {
  // what the kernel's mapping of workgroups to work items takes for granted
  if (a.blocks_all != blocks || a.blocks0 > blocks || a.blocks0 != a.side[0].igroups * (a.side[0].splits >> 1))
    return FS_ERR_BAD_ARGUMENT;
  blocks = 8 * ((blocks + 7) / 8);  // each XCD takes an eighth of the work items
  if (mode == kVec)
    hipLaunchKernelGGL(lse_gemm_kernel<1>, dim3(blocks), dim3(512), 0, st, a);
  else if (mode == kArgmax)
    hipLaunchKernelGGL(lse_gemm_kernel<2>, dim3(blocks), dim3(512), 0, st, a);
  else
    hipLaunchKernelGGL(lse_gemm_kernel<0>, dim3(blocks), dim3(512), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

}  // namespace fs
