// Launch functions defined in their own translation units.
#pragma once

#include "fs_common.hpp"

namespace fs {

// Column-sliced kernels for 128 < d <= 1536: nw wavefronts x nsl*32 columns each.
int launch_sliced(int mode, const LaunchArgs& a, int nw, int nsl, int blocks, hipStream_t st);

// Software-pipelined LSE kernel for d <= 128 with 16-byte aligned rows (dp in {16,32,64,128});
// prec: 0 fp32 operands, 1 two bf16 planes (3 products), 2 three bf16 planes (6 products).
// fp32 rows -> packed bf16 planes [rows][np][dp/2] for the split-bf16 modes of launch_lse2.
int launch_split_planes(const float* src, unsigned* dst, int rows, int d, int dp, int np,
                        hipStream_t st);
int launch_lse2(const LaunchArgs& a, int dp, int rb, int prec, int blocks, hipStream_t st);

}  // namespace fs
