// Instantiations and dispatch of the large-d (column-sliced) kernels.
#include "fs_sliced.hpp"

#include "fs_dispatch.hpp"

namespace fs {

template <int MODE, int NW, int NSL>
static int launch_cfg(const LaunchArgs& a, int blocks, hipStream_t st) {
  constexpr bool stat = (MODE != kMat5);
  if constexpr (NW == 8 && NSL == 6) {
    if (a.nss > 1) {  // rows wider than one workgroup's span
      hipLaunchKernelGGL((sliced_kernel<MODE, NW, NSL, stat, true>), dim3(blocks), dim3(NW * 64), 0,
                         st, a);
      return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
    }
  }
  hipLaunchKernelGGL((sliced_kernel<MODE, NW, NSL, stat, false>), dim3(blocks), dim3(NW * 64), 0, st,
                     a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

template <int MODE>
static int launch_mode(const LaunchArgs& a, int nw, int nsl, int blocks, hipStream_t st) {
  if (nw == 4 && nsl == 2) return launch_cfg<MODE, 4, 2>(a, blocks, st);
  if (nw == 8 && nsl == 2) return launch_cfg<MODE, 8, 2>(a, blocks, st);
  if (nw == 8 && nsl == 4) return launch_cfg<MODE, 8, 4>(a, blocks, st);
  if (nw == 8 && nsl == 6) return launch_cfg<MODE, 8, 6>(a, blocks, st);
  return FS_ERR_UNSUPPORTED;
}

int launch_sliced(int mode, const LaunchArgs& a, int nw, int nsl, int blocks, hipStream_t st) {
  switch (mode) {
    case kLse: return launch_mode<kLse>(a, nw, nsl, blocks, st);
    case kVec: return launch_mode<kVec>(a, nw, nsl, blocks, st);
    case kMat: return launch_mode<kMat>(a, nw, nsl, blocks, st);
    case kMat5: return launch_mode<kMat5>(a, nw, nsl, blocks, st);
  }
  return FS_ERR_BAD_ARGUMENT;
}

}  // namespace fs
