// Launch of the large-d GEMM-style log-sum-exp kernel.
#include "fs_lsegemm.hpp"

#include "fs_dispatch.hpp"

namespace fs {

// what the one-sweep kernel takes for granted about one side's chunks (splits: partial rows)
static bool sweep_chunks_ok(const Side& sd, int splits, int chunk) {
  return sd.part_ms != nullptr && splits >= 2 && !(splits & 1) && chunk > 0 && chunk % kGemmRows == 0 &&
         (long long)(splits / 2) * chunk >= sd.nk && (long long)(splits / 2 - 1) * chunk < sd.nk &&
         sd.igroups == (sd.nq + kGemmRows - 1) / kGemmRows && sd.qplanes != nullptr &&
         sd.kplanes != nullptr && sd.kb0 != nullptr;
}

static int self_items(const Side& sd, int splits, int chunk) {
  int items = 0;
  for (int s = 0; s < splits / 2; ++s) items += self_groups_of_chunk(s, chunk, sd.nk, sd.igroups);
  return items;
}

int launch_lse_gemm_sweep(const LaunchArgs& a, hipStream_t st) {
  const Side& s0 = a.side[0];
  const Side& s1 = a.side[1];
  if (a.sel == nullptr || a.col_part == nullptr || a.sw_part_mult != 2 ||
      !sweep_chunks_ok(s0, a.sw_splits, a.sw_chunk))
    return FS_ERR_BAD_ARGUMENT;
  int items = s0.igroups * (a.sw_splits / 2);
  if (a.sweep_self) {
    // every side a matrix with itself; side 1 present iff it has items
    if (s0.nq != s0.nk || s0.qplanes != s0.kplanes || a.sw_items0 != self_items(s0, a.sw_splits, a.sw_chunk) ||
        a.sw_items < a.sw_items0)
      return FS_ERR_BAD_ARGUMENT;
    if (a.sw_items > a.sw_items0 &&
        (a.col_part_b == nullptr || !sweep_chunks_ok(s1, a.sw_splits_b, a.sw_chunk_b) || s1.nq != s1.nk ||
         s1.qplanes != s1.kplanes || a.sw_items - a.sw_items0 != self_items(s1, a.sw_splits_b, a.sw_chunk_b)))
      return FS_ERR_BAD_ARGUMENT;
    items = a.sw_items;
  } else if (a.sw_splits > s0.splits || s0.nq != s1.nk || s0.nk != s1.nq || s1.kb0 == nullptr) {
    return FS_ERR_BAD_ARGUMENT;
  }
  // (a multiple of 8 workgroups: each XCD takes an eighth of the work items)
  const int per_xcd = (items + 7) / 8;
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
