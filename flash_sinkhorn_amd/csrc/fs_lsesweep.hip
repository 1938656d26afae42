// Instantiations and dispatch of the one-sweep form of a two-sided log-sum-exp step.
#include "fs_lsesweep.hpp"

#include "fs_dispatch.hpp"

namespace fs {

int launch_finish_sweep(const LaunchArgs& a, hipStream_t st);

static int self_items(const Side& sd, int splits, int chunk) {
  int items = 0;
  for (int s = 0; s < splits; ++s) items += self_groups_of_chunk(s, chunk, sd.nk, sd.igroups);
  return items;
}

template <int DP>
static int launch_sweep_dp(const LaunchArgs& a, hipStream_t st) {
  const Side& s0 = a.side[0];
  // (a multiple of 8 workgroups: each XCD takes an eighth of the work items)
  const int items = a.sweep_self ? a.sw_items : s0.igroups * a.sw_splits;
  const int per_xcd = (items + 7) / 8;
  hipLaunchKernelGGL((lse_sweep_kernel<DP>), dim3(8 * per_xcd), dim3(256), 0, st, a);
  if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
  return launch_finish_sweep(a, st);
}

int launch_finish_sweep(const LaunchArgs& a, hipStream_t st) {
  const bool one = a.sweep_self && a.sw_items == a.sw_items0;  // a single problem of a matrix with itself
  const int rows = a.side[0].nq + (one ? 0 : a.side[1].nq);
  hipLaunchKernelGGL((finish_sweep_kernel<0>), dim3((rows + 255) / 256), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

// what the kernel takes for granted about one side's chunks
static bool chunks_ok(const Side& sd, int splits, int chunk) {
  return sd.part_ms != nullptr && splits >= 1 && splits <= sd.splits && chunk > 0 && chunk % 64 == 0 &&
         (long long)splits * chunk >= sd.nk && (long long)(splits - 1) * chunk < sd.nk &&
         sd.qplanes != nullptr && sd.kplanes != nullptr && sd.kb0 != nullptr;
}

int launch_lse_sweep(const LaunchArgs& a, int dp, hipStream_t st) {
  const Side& s0 = a.side[0];
  const Side& s1 = a.side[1];
  if (a.sel == nullptr || a.col_part == nullptr || !chunks_ok(s0, a.sw_splits, a.sw_chunk)) return FS_ERR_BAD_ARGUMENT;
  if (a.sweep_self) {
    // every side a matrix with itself; side 1 present iff it has items
    if (s0.nq != s0.nk || s0.qplanes != s0.kplanes || s0.igroups != (s0.nq + 255) / 256 ||
        a.sw_items0 != self_items(s0, a.sw_splits, a.sw_chunk) || a.sw_items < a.sw_items0)
      return FS_ERR_BAD_ARGUMENT;
    if (a.sw_items > a.sw_items0 &&
        (a.col_part_b == nullptr || !chunks_ok(s1, a.sw_splits_b, a.sw_chunk_b) || s1.nq != s1.nk ||
         s1.qplanes != s1.kplanes || s1.igroups != (s1.nq + 255) / 256 ||
         a.sw_items - a.sw_items0 != self_items(s1, a.sw_splits_b, a.sw_chunk_b)))
      return FS_ERR_BAD_ARGUMENT;
  } else if (s0.nq != s1.nk || s0.nk != s1.nq || s1.kb0 == nullptr) {
    return FS_ERR_BAD_ARGUMENT;
  }
  switch (dp) {
    case 16: return launch_sweep_dp<16>(a, st);
    case 32: return launch_sweep_dp<32>(a, st);
    case 64: return launch_sweep_dp<64>(a, st);
    case 128: {
      const int items = a.sweep_self ? a.sw_items : s0.igroups * a.sw_splits;
      hipLaunchKernelGGL((lse_sweep128_kernel<0>), dim3(8 * ((items + 7) / 8)), dim3(256), 0, st, a);
      if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
      return launch_finish_sweep(a, st);
    }
  }
  return FS_ERR_UNSUPPORTED;
}

}  // namespace fs
