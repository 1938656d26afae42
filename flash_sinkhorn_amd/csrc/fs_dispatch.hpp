// Launch functions defined in their own translation units.
#pragma once

#include "fs_common.hpp"

namespace fs {

// Column-sliced kernels for 128 < d <= 1536: nw wavefronts x nsl*32 columns each.
int launch_sliced(int mode, const LaunchArgs& a, int nw, int nsl, int blocks, hipStream_t st);

// Software-pipelined LSE kernel for d <= 128 with 16-byte aligned rows (dp in {16,32,64,128});
// prec: 0 fp32 operands, 3 two scaled fp16 planes (3 products).
// fp16 planes: absmax over the (at most two) operand matrices -> partial[2][256]; then one
// split per matrix, which also writes the matrix's power-of-two scale to *scale_out and clears
// the variant-choice state at clear_state (kSelWords words; may be null) and resets best_keys
// (one int per row; may be null) to -1.
// n 32-bit words at p (16-byte aligned) set to zero by a kernel (graph-capture safe).
int launch_fill_zero(unsigned* p, long long n, hipStream_t st);
int launch_absmax(const float* a, long long na, const float* b, long long nb, float* partial,
                  hipStream_t st);
// The seed part of coarse_bias_kernel alone: per side with Side::seed set, where each query row's
// running maximum starts (its logit at the key Side::best_key names).
int launch_row_seeds(const LaunchArgs& a, int dp, int nsides, hipStream_t st);
int launch_split_planes_f16(const float* src, unsigned* dst, int rows, int d, int dp,
                            const float* partial_max, float* scale_out, float* scale_out2,
                            int chunked, unsigned* clear_state, int* best_keys, unsigned* tiled,
                            hipStream_t st, int start_plain = 0);
// GEMM-style LSE kernel for 128 < d <= 1536 on chunked fp16 planes; Side::splits counts
// partial rows (twice the workgroup-level key splits).
int launch_lse_gemm(const LaunchArgs& a, int mode, int blocks, hipStream_t st);  // kLse, kVec, kArgmax
// Its one-sweep form (both sides of a two-sided step; side 0's grid with LaunchArgs::sw_splits
// partial rows per query row and sw_chunk keys per workgroup); launch_finish_sweep follows.
int launch_lse_gemm_sweep(const LaunchArgs& a, hipStream_t st);
// Plan-matrix products (mat5: with the second stationary operand) for d > 128 on fp16 planes: cb column blocks per wavefront (2, 4 or 6),
// LaunchArgs::nss column groups.  The value matrix (times an optional per-row scale) is
// brought into operand order by launch_transpose_planes; partial needs 256 floats.
int launch_plan_gemm(const LaunchArgs& a, bool mat5, int cb, int blocks, hipStream_t st);
// mat5: squared row norms of q2 and the largest entry of k2 (= squared row norms of the keys).
int launch_mat5_bounds(const float* q2, int nq, int d, const float* k2, long long nk, float* q2norm2,
                       float* kmax2, hipStream_t st);
int launch_transpose_planes(const float* src, const float* rowscale, unsigned* dst, int rows, int d,
                            int nkb, int ncb, float* partial, float* scale_out, hipStream_t st);
// Plan-matrix (kMat), plan-vector (kVec) products and running arg-max (kArgmax) for d <= 128 on
// two-plane fp16 rows (dp in {16, 32, 64, 128}; rb row blocks per wavefront in {1, 2}, 1 at 128).
int launch_plan_tile(const LaunchArgs& a, int mode, int dp, int rb, int blocks, hipStream_t st);
int launch_lse2(const LaunchArgs& a, int dp, int rb, int prec, bool vec, bool coarse, int blocks,
                hipStream_t st);
// Both sides of a two-sided step from one sweep over the logits (lse_sweep_kernel over side 0's
// grid, then its merge); both run only when the state words at LaunchArgs::sel allow it.
int launch_lse_sweep(const LaunchArgs& a, int dp, hipStream_t st);
// The merge of a one-sweep launch alone (row sums from side 0's partial rows, column sums from
// LaunchArgs::col_part).
int launch_finish_sweep(const LaunchArgs& a, hipStream_t st);

}  // namespace fs
