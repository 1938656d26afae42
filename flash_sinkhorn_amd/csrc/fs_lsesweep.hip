// Instantiations and dispatch of the one-sweep form of a two-sided log-sum-exp step.
#include "fs_lsesweep.hpp"

#include "fs_dispatch.hpp"

namespace fs {

int launch_finish_sweep(const LaunchArgs& a, hipStream_t st);

template <int DP>
static int launch_sweep_dp(const LaunchArgs& a, hipStream_t st) {
  const Side& s0 = a.side[0];
  // (a multiple of 8 workgroups: each XCD takes an eighth of the work items)
  const int per_xcd = (s0.igroups * a.sw_splits + 7) / 8;
  hipLaunchKernelGGL((lse_sweep_kernel<DP>), dim3(8 * per_xcd), dim3(256), 0, st, a);
  if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
  return launch_finish_sweep(a, st);
}

int launch_finish_sweep(const LaunchArgs& a, hipStream_t st) {
  const int rows = a.side[0].nq + a.side[1].nq;
  hipLaunchKernelGGL((finish_sweep_kernel<0>), dim3((rows + 255) / 256), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

int launch_lse_sweep(const LaunchArgs& a, int dp, hipStream_t st) {
  // what the kernel takes for granted
  const Side& s0 = a.side[0];
  const Side& s1 = a.side[1];
  if (a.sel == nullptr || a.col_part == nullptr || s0.part_ms == nullptr ||
      a.sw_splits < 1 || a.sw_splits > s0.splits || a.sw_chunk % 64 != 0 || a.sw_chunk <= 0 ||
      (long long)a.sw_splits * a.sw_chunk < s0.nk || (long long)(a.sw_splits - 1) * a.sw_chunk >= s0.nk || s0.nq != s1.nk || s0.nk != s1.nq ||
      s0.qplanes == nullptr || s0.kplanes == nullptr || s1.kb0 == nullptr)
    return FS_ERR_BAD_ARGUMENT;
  switch (dp) {
    case 16: return launch_sweep_dp<16>(a, st);
    case 32: return launch_sweep_dp<32>(a, st);
    case 64: return launch_sweep_dp<64>(a, st);
  }
  return FS_ERR_UNSUPPORTED;
}

}  // namespace fs
