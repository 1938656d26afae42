// Launches of the large-d plan-matrix kernel and of the value-plane transposition.
#include "fs_plangemm.hpp"

#include "fs_dispatch.hpp"

namespace fs {

template <bool MAT5>
static int launch_cb(const LaunchArgs& a, int cb, int blocks, hipStream_t st) {
  switch (cb) {
    case 2: hipLaunchKernelGGL((plan_gemm_kernel<2, MAT5>), dim3(blocks), dim3(512), 0, st, a); break;
    case 4: hipLaunchKernelGGL((plan_gemm_kernel<4, MAT5>), dim3(blocks), dim3(512), 0, st, a); break;
    case 6: hipLaunchKernelGGL((plan_gemm_kernel<6, MAT5>), dim3(blocks), dim3(512), 0, st, a); break;
    default: return FS_ERR_BAD_ARGUMENT;
  }
  return FS_OK;
}

int launch_plan_gemm(const LaunchArgs& a, bool mat5, int cb, int blocks, hipStream_t st) {
  const int rc = mat5 ? launch_cb<true>(a, cb, blocks, st) : launch_cb<false>(a, cb, blocks, st);
  if (rc != FS_OK) return rc;
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

int launch_mat5_bounds(const float* q2, int nq, int d, const float* k2, long long nk, float* q2norm2,
                       float* kmax2, hipStream_t st) {
  hipLaunchKernelGGL(rownorm2_kernel, dim3((nq + 3) / 4), dim3(256), 0, st, q2, nq, d, q2norm2);
  hipLaunchKernelGGL(vecmax_kernel, dim3(64), dim3(256), 0, st, k2, nk, kmax2);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

int launch_transpose_planes(const float* src, const float* rowscale, unsigned* dst, int rows, int d,
                            int nkb, int ncb, float* partial, float* scale_out, hipStream_t st) {
  hipLaunchKernelGGL(absmax_rows_kernel, dim3(256), dim3(256), 0, st, src, (long long)rows, d,
                     rowscale, partial);
  if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
  const long long units = (long long)nkb * ncb * 2;
  hipLaunchKernelGGL(transpose_planes_f16_kernel, dim3((unsigned)((units + 3) / 4)), dim3(256), 0,
                     st, src, rowscale, dst, rows, d, nkb, ncb, partial, scale_out);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

}  // namespace fs
