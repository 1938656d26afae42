// Launch functions defined in their own translation units.
#pragma once

#include "fs_common.hpp"

namespace fs {

// Column-sliced kernels for 128 < d <= 1536: nw wavefronts x nsl*32 columns each.
int launch_sliced(int mode, const LaunchArgs& a, int nw, int nsl, int blocks, hipStream_t st);

}  // namespace fs
