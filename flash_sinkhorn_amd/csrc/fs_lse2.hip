// Instantiations and dispatch of the software-pipelined log-sum-exp kernel.
#include "fs_lse2.hpp"
#include "fs_lsecoarse.hpp"
#include "fs_lsecoarse128.hpp"
#include "fs_lsesparse.hpp"

#include "fs_dispatch.hpp"

namespace fs {

template <int DP, int RB, int PREC, bool VEC>
static int launch_cfg(const LaunchArgs& a, int blocks, hipStream_t st) {
  hipLaunchKernelGGL((lse2_kernel<DP, RB, PREC, VEC>), dim3(blocks), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

template <int DP, int PREC, bool VEC>
static int launch_rb(const LaunchArgs& a, int rb, int blocks, hipStream_t st) {
  if constexpr (DP <= 64) {
    if (rb >= 2) return launch_cfg<DP, 2, PREC, VEC>(a, blocks, st);
  }
  return launch_cfg<DP, 1, PREC, VEC>(a, blocks, st);
}

template <int PREC, bool VEC>
static int launch_dp(const LaunchArgs& a, int dp, int rb, int blocks, hipStream_t st) {
  switch (dp) {
    case 16: return launch_rb<16, PREC, VEC>(a, rb, blocks, st);
    case 32: return launch_rb<32, PREC, VEC>(a, rb, blocks, st);
    case 64: return launch_rb<64, PREC, VEC>(a, rb, blocks, st);
    case 128:
      if constexpr (!VEC) return launch_rb<128, PREC, false>(a, rb, blocks, st);
  }
  return FS_ERR_UNSUPPORTED;
}

int launch_absmax(const float* a, long long na, const float* b, long long nb, float* partial,
                  hipStream_t st) {
  hipLaunchKernelGGL(absmax_kernel, dim3(2 * kAbsmaxBlocks), dim3(256), 0, st, a, na, b, nb, partial);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

int launch_fill_zero(unsigned* p, long long n, hipStream_t st) {
  if (n <= 0) return FS_OK;
  const long long grid = (n / 4 + 256) / 256;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)grid), dim3(256), 0, st, p, n);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

int launch_split_planes_f16(const float* src, unsigned* dst, int rows, int d, int dp,
                            const float* partial_max, float* scale_out, float* scale_out2,
                            int chunked, unsigned* clear_state, int* best_keys, unsigned* tiled,
                            hipStream_t st, int start_plain) {
  const long long items = (long long)(rows + kPlanePadRows) * (dp / 4);
  const int grid = (int)((items + 255) / 256);
  hipLaunchKernelGGL(split_planes_f16_kernel, dim3(grid), dim3(256), 0, st, src, dst, rows, d, dp,
                     partial_max, scale_out, scale_out2, chunked, clear_state, best_keys, tiled, start_plain);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

// fp16 planes, log-sum-exp, rows of at most 64 columns: the pipelined kernel with the coarse
// tile test (two blocks of 32 query rows per wavefront: the launch must be planned with rb = 2)
template <int DP>
static int launch_coarse_dp(const LaunchArgs& a, int blocks, hipStream_t st) {
  hipLaunchKernelGGL((lse_coarse_kernel<DP>), dim3(blocks), dim3(256), 0, st, a);
  // with carried margins both forms are enqueued; per side, the one the state words name runs
  if (a.side[0].margins != nullptr)
    hipLaunchKernelGGL((lse_sparse_kernel<DP>), dim3(a.blocks_sparse), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

int launch_row_seeds(const LaunchArgs& a, int dp, int nsides, hipStream_t st) {
  const int sb0 = (a.side[0].nq + 7) / 8;
  const int sb1 = nsides > 1 ? (a.side[1].nq + 7) / 8 : 0;
  LaunchArgs b = a;
  b.sel_pred = 0;
  hipLaunchKernelGGL((coarse_bias_kernel<0>), dim3(sb0 + sb1), dim3(64), 0, st, b, 0, 0, sb0, dp);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

static int launch_coarse(const LaunchArgs& a, int dp, int rb, int blocks, hipStream_t st) {
  if (rb != 2) return FS_ERR_BAD_ARGUMENT;
  // the per-tile records of the key bias, for both sides (tiles past the last key included)
  const int tiles0 = (a.side[0].nk + 63) / 64 + kAuxPadTiles;
  const int tiles1 = blocks > a.blocks0 ? (a.side[1].nk + 63) / 64 + kAuxPadTiles : 0;
  // behind them, per 8 query rows one block that computes where the rows' maxima start
  const bool seeds = a.side[0].seed != nullptr;
  const int sb0 = seeds ? (a.side[0].nq + 7) / 8 : 0;
  const int sb1 = seeds && blocks > a.blocks0 ? (a.side[1].nq + 7) / 8 : 0;
  hipLaunchKernelGGL((coarse_bias_kernel<0>), dim3(tiles0 + tiles1 + sb0 + sb1), dim3(64), 0, st, a,
                     tiles0, tiles0 + tiles1, sb0, dp);
  if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
  switch (dp) {
    case 16: return launch_coarse_dp<16>(a, blocks, st);
    case 32: return launch_coarse_dp<32>(a, blocks, st);
    case 64: return launch_coarse_dp<64>(a, blocks, st);
    case 128:  // no carried margins, no sparse form
      if (a.side[0].margins != nullptr) return FS_ERR_BAD_ARGUMENT;
      hipLaunchKernelGGL((lse_coarse128_kernel<0>), dim3(blocks), dim3(256), 0, st, a);
      return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
  }
  return FS_ERR_UNSUPPORTED;
}

int launch_lse2(const LaunchArgs& a, int dp, int rb, int prec, bool vec, bool coarse, int blocks,
                hipStream_t st) {
  if (coarse && !vec && prec == kH3 && dp <= 128) return launch_coarse(a, dp, rb, blocks, st);
  if (vec) {  // plan-vector product: fp16 planes, rows of at most 64 columns
    return prec == kH3 ? launch_dp<kH3, true>(a, dp, rb, blocks, st) : FS_ERR_UNSUPPORTED;
  }
  switch (prec) {
    case kF32: return launch_dp<kF32, false>(a, dp, rb, blocks, st);
    case kH3: return launch_dp<kH3, false>(a, dp, rb, blocks, st);
  }
  return FS_ERR_BAD_ARGUMENT;
}

}  // namespace fs
