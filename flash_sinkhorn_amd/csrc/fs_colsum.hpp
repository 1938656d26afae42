// Sums over the 32 query columns of a transposed 32 x 32 logits tile (MFMA accumulator
// layout: lane (li, h) holds query column li and, in register r, key 8 (r / 4) + 4 h + r % 4).
//
// The sum over the 32 lanes of a half-wave goes in steps that pair lanes differing in one bit
// of li and halve the number of registers: of a pair of registers (A, B) a lane with the bit
// clear keeps A + A of its partner, a lane with the bit set B + B of its partner.  For bits 3
// and 2 the partner is the lane's mirror image in its row of 16 / its group of 8 lanes, the two
// kinds of lanes are whole banks of four, and a DPP add with a bank mask writes only one kind:
// two instructions per pair, in place.  The steps for bits 1 and 0 work within a quad: both
// sums, then a select.  After the four steps lane li holds register 8 b0 + 4 b1 + 2 b2 + b3
// (b: the bits of li) summed over its row of 16 lanes; the two rows of a half-wave stay
// separate (whoever collects the sums adds them).
#pragma once

#include <type_traits>

#include "fs_common.hpp"

namespace fs {

// (s_nop: a VALU result read through DPP needs two wait states, which the compiler does not
// insert inside an asm statement; without them the sums came out wrong)
// a: registers (r, r + 1) -> r (+ 1 where bit 3 of li is set)
__device__ __forceinline__ void colsum_step_bit3(float& a, const float& b) {
  asm volatile("s_nop 1\n\t"
               "v_add_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0x3\n\t"
               "v_add_f32_dpp %0, %1, %1 row_mirror row_mask:0xf bank_mask:0xc"
               : "+v"(a) : "v"(b));
}
// a: results (4m, 4m + 2) of the step before -> 4m (+ 2 where bit 2 of li is set)
__device__ __forceinline__ void colsum_step_bit2(float& a, const float& b) {
  asm volatile("s_nop 1\n\t"
               "v_add_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
               "v_add_f32_dpp %0, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xa"
               : "+v"(a) : "v"(b));
}

template <int CTRL>
__device__ __forceinline__ float colsum_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL,
                                                               0xf, 0xf, true));
}
constexpr int kQuadXor2 = 0x4E;  // quad_perm [2,3,0,1]
constexpr int kQuadXor1 = 0xB1;  // quad_perm [1,0,3,2]

// bit 1: the four results of the steps above, by pairs -> two
__device__ __forceinline__ float colsum_bit1(float c0, float c1, int li) {
  const float t = c0 + colsum_dpp<kQuadXor2>(c0);
  const float u = c1 + colsum_dpp<kQuadXor2>(c1);
  return (li & 2) ? u : t;
}
// bit 0: the two results of colsum_bit1 -> this lane's sum
__device__ __forceinline__ float colsum_bit0(float f0, float f1, int li) {
  const float t = f0 + colsum_dpp<kQuadXor1>(f0);
  const float u = f1 + colsum_dpp<kQuadXor1>(f1);
  return (li & 1) ? u : t;
}

// the key (0..31 of the tile) whose sum lane (li, h) ends up with
__device__ __forceinline__ int colsum_key(int li, int h) {
  const int reg = 8 * (li & 1) + 4 * ((li >> 1) & 1) + 2 * ((li >> 2) & 1) + ((li >> 3) & 1);
  return 8 * (reg >> 2) + 4 * h + (reg & 3);
}

// all four steps on 16 values held at once (destroys c)
__device__ __forceinline__ float colsum_all(float (&c)[16], int li) {
#pragma unroll
  for (int r = 0; r < 16; r += 2) colsum_step_bit3(c[r], c[r + 1]);
#pragma unroll
  for (int m = 0; m < 4; ++m) colsum_step_bit2(c[4 * m], c[4 * m + 2]);
  const float f0 = colsum_bit1(c[0], c[4], li);
  const float f1 = colsum_bit1(c[8], c[12], li);
  return colsum_bit0(f0, f1, li);
}

}  // namespace fs
