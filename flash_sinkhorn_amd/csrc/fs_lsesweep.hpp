// Both halves of a two-sided log-sum-exp step from ONE sweep over the logits (fp16 planes,
// d <= 64, prepared planes).
//
// A symmetric step needs, for the same matrix of base-2 logits
//     S_ij = qscale * (x_i . y_j) + r_i + c_j,   r_i = the bias of x_i as a key, c_j = that of y_j,
// the row sums R_i = sum_j 2^S_ij and the column sums C_j = sum_i 2^S_ij:
//     LSE_j(x_i . y_j + c_j) = log2 R_i - r_i,   LSE_i(x_i . y_j + r_i) = log2 C_j - c_j.
// lse2_kernel computes the logits twice, once per side, because each side wants its own running
// maximum under the exponentials.  With BOTH biases inside the exponent no maximum is needed
// once the potentials have stopped jumping: R_i is the mass the current plan gives row i, which
// is the row's weight times 2^(twice the change of its potential in this step), and likewise
// C_j; every term is at most its row's sum.  So this kernel runs lse2_kernel's pipeline on one
// side only (stationary x rows in registers, y keys through the LDS ring, key bias as the start
// of the MFMA chain, transposed 32 x 32 logits tiles), takes r_i as the addend of the exp2
// argument where lse2_kernel puts the running maximum, and has no maximum, no rescale and no
// wave-uniform branch.  Next to the lane-private row sums it adds the exponentials of a
// wavefront's two row blocks per key and reduces them over the 32 lanes that hold a key's 32
// query columns (DPP adds that halve the number of registers as they go, see below: about two
// instructions per exponential, fewer than lse2_kernel spends on its maxima).  The four wavefronts of a workgroup leave their sums per key in LDS and one of them
// adds the four, in a fixed order, and writes them out once per 64-key tile
// (LaunchArgs::col_part, one row of sums per workgroup row group): the merge kernel adds those.
//
// The merge kernel checks every sum against the range this is exact in (kSweepFailLo/Hi) and
// has the two-sided kernel redo the step otherwise; whether a step may run this kernel at all is
// decided by the merge of the step before (kSweepOkLo/Hi), so the first steps of a solve, steps
// on a plan that is moving fast and problems with empty weights stay on the two-sided kernel.
#pragma once

#include <type_traits>

#include "fs_colsum.hpp"
#include "fs_common.hpp"
#include "fs_stream.hpp"

#ifndef FS_SCHED_FENCE
#define FS_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
#endif

namespace fs {

// A unit's MFMAs are cut into this many program-order pieces, with a piece of the previous
// unit's exponentials behind each (as in lse2_kernel); from piece kSweepBiasPiece on, the
// registers of the previous logits take the next unit's bias, four at every other piece.
constexpr int kSweepPieces = 12;
constexpr int kSweepBiasPiece = 2;

template <int DP>
__global__ __launch_bounds__(256, 2) void lse_sweep_kernel(const LaunchArgs args) {
  static_assert(DP == 16 || DP == 32 || DP == 64, "two-plane rows of at most 64 columns");
  constexpr int RB = 2, NSUB = 2, JT = 64;
  constexpr int KK16 = DP / 16;
  constexpr int NMAIN = 3 * KK16;  // MFMAs of one logits tile
  constexpr int ROWW = DP;         // 32-bit words per operand row: two planes of DP/2
  constexpr int NBUF = 3;
  constexpr int PPR = ROWW / 4;    // 16-byte pieces per row
  constexpr int PER_THREAD = JT * PPR / 256;
  static_assert(JT * PPR % 256 == 0, "whole rounds of direct loads");

  __shared__ __attribute__((aligned(16))) unsigned lds_k[NBUF][JT * ROWW];
  __shared__ __attribute__((aligned(16))) float lds_b[NBUF][256];  // [buf][thread]; first JT used
  // column sums of a 64-key tile per wavefront; the tile being filled and the one before
  __shared__ __attribute__((aligned(16))) float lds_col[2][4][2][JT];  // [tile][wavefront][row of 16 lanes][key]

  // the step may not run this kernel, or the device chose another variant
  if (args.sel[kSelSweep] == 0u) return;
  if (args.sweep == 2 && args.sel[kSelWord] != 1u) return;
  if (blockIdx.x == 0 && threadIdx.x == 0) args.sel[kSelRan] = 1u;

  // Work items (key chunk, row group), key chunk slowest; workgroups are dealt round-robin to the
  // 8 XCDs, and XCD x takes the x-th eighth of the items in that order: the workgroups that run on
  // an XCD at any one time share one key chunk (two at a boundary), which stays in its L2
  // whatever the number of chunks.  (With chunk = id % chunks and 13 chunks every XCD streamed
  // the whole key matrix: 1.35 GB from beyond L2 per launch instead of 0.2.)
  // sweep_self: side 0's items, then side 1's; a chunk only has items for the row groups that
  // begin before its end.
  const bool self = args.sweep_self != 0;
  const int n_items = self ? args.sw_items : args.side[0].igroups * args.sw_splits;
  const int per_xcd = (n_items + 7) / 8;
  int item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per_xcd || item >= n_items) return;
  const bool second = self && item >= args.sw_items0;
  if (second) item -= args.sw_items0;
  const Side& sd = second ? args.side[1] : args.side[0];
  // whose key bias is the bias of this side's rows: the other side's, or (self) its own
  const Side& so = self ? sd : args.side[1];
  const int sw_chunk = second ? args.sw_chunk_b : args.sw_chunk;
  int split, ig;
  if (self) {
    split = 0;
    for (;;) {  // (item < the number of items of this side: ends within its chunks)
      const int g = self_groups_of_chunk(split, sw_chunk, sd.nk, sd.igroups);
      if (item < g) break;
      item -= g;
      ++split;
    }
    ig = item;
  } else {
    split = item / sd.igroups;
    ig = item % sd.igroups;
  }
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int h = lane >> 5;
  const int row0 = (ig * 4 + wave) * (32 * RB);
  // (self: from the first row of this row group on; chunks and row groups are multiples of the
  // 64 keys of a tile)
  const int j_begin = self ? max(split * sw_chunk, ig * 256) : split * sw_chunk;
  const int j_end = min(sd.nk, (split + 1) * sw_chunk);
  const int ntiles = (j_end - j_begin + JT - 1) / JT;
  if (ntiles <= 0) return;  // (whole workgroup: no barrier is left waiting)

  // MFMAs produce raw dot products of the scaled planes; lscale turns them into base-2 logits
  const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = 1.0f / lscale;

  // ---- stationary query operands, and the rows' own bias (base 2) ----
  u32x4 xq[RB][2][KK16];
  float cx[RB], run_s[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = min(row0 + rb * 32 + li, sd.nq - 1);
    const unsigned* qrow = sd.qplanes + (size_t)row * (size_t)ROWW;
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int kk = 0; kk < KK16; ++kk)
        xq[rb][p][kk] = *reinterpret_cast<const u32x4*>(qrow + p * (DP / 2) + 8 * kk + 4 * h);
    float r = so.kc0 * so.kb0[row];
    if (so.kb1 != nullptr) r += so.kc1 * so.kb1[row];
    if (so.kb2 != nullptr) r += so.kc2 * so.kb2[row];
    // rows past the last one (they repeat it) must not reach the column sums
    cx[rb] = (row0 + rb * 32 + li < sd.nq) ? fmaxf(r, kNegBig) : kNegBig;
    run_s[rb] = 0.f;
  }

  // ---- staging of key tiles: direct global->LDS loads, bias terms through registers ----
  float st_b0 = 0.f, st_b1 = 0.f, st_b2 = 0.f, st_pen = 0.f;
  const float* kb1p = sd.kb1 ? sd.kb1 : sd.kb0;  // always loadable; unused terms are dropped
  const float* kb2p = sd.kb2 ? sd.kb2 : sd.kb0;
  const float kc0 = sd.kc0, kc1 = sd.kc1, kc2 = sd.kc2;
  const bool has_kb1 = sd.kb1 != nullptr, has_kb2 = sd.kb2 != nullptr;
  auto swz = [&](int r) {  // slot permutation of LDS row r
    return PPR >= 16 ? (r & 15) : (PPR == 8 ? ((r >> 1) & 7) : ((r >> 2) & 3));
  };
  // lane tid fills LDS slot tid of a round of 256 slots and fetches the piece that belongs
  // there; the rounds of a tile are 4 KiB apart in the planes and the slot permutation is the
  // same in each, so one 32-bit lane offset and a wave-uniform base serve all of them
  static_assert(PER_THREAD == 1 || (256 / PPR) % (PPR >= 16 ? 16 : 16) == 0, "rounds share the slot permutation");
  const unsigned lane_off = (unsigned)(((tid / PPR) * ROWW + (((tid % PPR) ^ swz(tid / PPR)) * 4)) * 4);
  const char* ktile = reinterpret_cast<const char*>(sd.kplanes + (size_t)j_begin * (size_t)ROWW);
  auto stage_load = [&](int j0, int dbuf) {
    {
      const int j = max(0, min(j0 + tid, j_end - 1));
      st_b0 = sd.kb0[j];
      st_b1 = kb1p[j];
      st_b2 = kb2p[j];
      st_pen = (j0 + tid < j_end) ? 0.f : 2.0f * kNegBig;
    }
#pragma unroll
    for (int c = 0; c < PER_THREAD; ++c) {
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(ktile + c * (256 / PPR) * ROWW * 4 + lane_off),
          (__attribute__((address_space(3))) void*)(&lds_k[dbuf][(c * 256 + wave * 64) * 4]), 16, 0, 0);
    }
    ktile += JT * ROWW * 4;
  };
  auto stage_store = [&](int buf) {
    // masked rows get a penalty ADDED (not selected), so the loads stay unconditional
    float b = kc0 * st_b0 + (has_kb1 ? kc1 * st_b1 : 0.f);
    b += (has_kb2 ? kc2 * st_b2 : 0.f);
    lds_b[buf][tid] = (fmaxf(b, kNegBig) + st_pen) * inv_lscale;
  };

  // ---- key operands of one 32-key sub-tile, read from LDS by hand (see lse2_kernel) ----
  struct KeyRegs {
    u32x4 yq[2][KK16];
  };
  auto lds_read16 = [&](const unsigned* p) -> u32x4 {
    u32x4 v;
    const unsigned addr = (unsigned)(size_t)(const __attribute__((address_space(3))) unsigned*)p;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
  };
  auto wait_lds = [&]() { __builtin_amdgcn_s_waitcnt(0xC07F); };  // lgkmcnt(0)
  auto load_keys = [&](KeyRegs& kr, int buf, int js) {
    const unsigned* yrow = lds_k[buf] + (js * 32 + li) * ROWW;
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int kk = 0; kk < KK16; ++kk) {
        const int piece = p * (DP / 8) + 2 * kk + h;
        kr.yq[p][kk] = lds_read16(yrow + (piece ^ swz(li)) * 4);
      }
  };
  // MFMA number k of a logits tile: plane products from the lowest weight to hi*hi
  auto mfma_k = [&](int k, f32x16 acc, const KeyRegs& kr, int rb) {
    const int prod = k / KK16, kk = k % KK16;
    const int pa = (prod == 0) ? 1 : 0;  // (key plane, query plane): (lo,hi) (hi,lo) (hi,hi)
    const int pb = (prod == 1) ? 1 : 0;
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kr.yq[pa][kk]),
                                                  __builtin_bit_cast(f16x8, xq[rb][pb][kk]), acc, 0, 0, 0);
  };
  // the key bias of sub-tile js as the accumulator layout holds it (register r of lane (li, h)
  // is key 8(r/4) + 4h + r%4)
  auto load_bias4 = [&](f32x16& b, int c, int buf, int js) {
    const float4 v = *reinterpret_cast<const float4*>(&lds_b[buf][js * 32 + 8 * c + 4 * h]);
    b[4 * c + 0] = v.x;
    b[4 * c + 1] = v.y;
    b[4 * c + 2] = v.z;
    b[4 * c + 3] = v.w;
  };

  // waits on vector-memory operations by count (see lse2_kernel::wait_vm)
  auto wait_vm = [&](auto newer) {
    constexpr int n = decltype(newer)::value;
    __builtin_amdgcn_s_waitcnt(0x0F70 | (n & 15) | ((n >> 4) << 14));
  };
  constexpr int kLoadsPerTile = PER_THREAD + 3;  // direct loads + bias terms
  auto wait_older_tiles_and_lds = [&]() {
    constexpr int n = kLoadsPerTile;
    __builtin_amdgcn_s_waitcnt(0x0070 | (n & 15) | ((n >> 4) << 14));
  };

  // ---- the exponentials of one unit (32 keys x 32 rows), in pieces between the MFMAs of the
  // next one ----
  // Column sums (see fs_colsum.hpp): the steps for bits 3 and 2 of the lane number are taken on
  // every unit as its exponentials come out (16 -> 4 registers, which the second row block's
  // unit adds to); the steps for bits 1 and 0 follow once per sub-tile.  The two rows of 16
  // lanes of a half-wave are added by the wavefront that writes the sums out.
  float col[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) col[k] = 0.f;
  struct Stage {
    float t[16], e[16], ps0, ps1;
  };
  auto soft_piece = [&](int p, Stage& s, const f32x16& a, int prb) {
    // values 2p, 2p + 1: fma at piece p, exp2 at p + 1, row sums and the step for bit 3 at
    // p + 2; every other piece from 4 on, the step for bit 2 on the last two results
    if (p == 0) {
      s.ps0 = 0.f;
      s.ps1 = 0.f;
    }
    if (p < 8) {
      s.t[2 * p] = __builtin_fmaf(a[2 * p], lscale, cx[prb]);
      s.t[2 * p + 1] = __builtin_fmaf(a[2 * p + 1], lscale, cx[prb]);
    }
    if (p >= 1 && p < 9) {
      s.e[2 * p - 2] = fast_exp2(s.t[2 * p - 2]);
      s.e[2 * p - 1] = fast_exp2(s.t[2 * p - 1]);
    }
    if (p >= 2 && p < 10) {
      const int r = 2 * p - 4;
      s.ps0 += s.e[r];
      s.ps1 += s.e[r + 1];
      colsum_step_bit3(s.e[r], s.e[r + 1]);  // e[r]: registers r (+1 where bit 3 is set)
    }
    if (p >= 3 && p < 10 && p % 2 == 1) {
      const int m = (p - 3) / 2;  // results e[4m], e[4m + 2]
      colsum_step_bit2(s.e[4 * m], s.e[4 * m + 2]);
      if (prb == 0) {
        col[m] = s.e[4 * m];
      } else {
        col[m] += s.e[4 * m];
      }
    }
  };
  auto soft_tail = [&](Stage& s, int prb) { run_s[prb] += s.ps0 + s.ps1; };
  auto soft_whole = [&](const f32x16& a, int prb) {  // the last unit of the chunk
    Stage s;
#pragma unroll
    for (int p = 0; p < 10; ++p) soft_piece(p, s, a, prb);
    soft_tail(s, prb);
  };

  struct Red {
    float f[2], g;
  };
  auto red_piece = [&](int p, Red& R) {
    if (p == 0 || p == 1) R.f[p] = colsum_bit1(col[2 * p], col[2 * p + 1], li);
    if (p == 2) R.g = colsum_bit0(R.f[0], R.f[1], li);
  };
  const int my_key = colsum_key(li, h);  // of the sub-tile
  auto red_store = [&](const Red& R, int tile, int js) {
    lds_col[tile & 1][wave][li >> 4][js * 32 + my_key] = R.g;
  };
  // one wavefront adds the four wavefronts' sums of a finished tile and writes them out
  float* colp = (second ? args.col_part_b : args.col_part) + (size_t)ig * (size_t)sd.nk;
  auto flush = [&](int tile) {
    const float* c = &lds_col[tile & 1][0][0][0];  // (a fixed order of additions: the same sums on every run)
    float v = c[lane] + c[JT + lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) v += c[2 * w * JT + lane] + c[(2 * w + 1) * JT + lane];
    const int j = j_begin + tile * JT + lane;
    if (j < j_end) colp[j] = v;
  };

  KeyRegs K[2];
  int cur = 0, nxt = 1, nx2 = 2;
  auto rotate = [&]() {
    const int c = cur;
    cur = nxt;
    nxt = nx2;
    nx2 = c;
  };

  // ---- prologue: tile 0 in buffer 0, tile 1 on its way ----
  stage_load(j_begin, 0);
  stage_store(0);
  stage_load(j_begin + JT, 1);
  wait_vm(std::integral_constant<int, 0>{});
  __syncthreads();
  load_keys(K[0], 0, 0);

  // R0 and R1 swap roles from unit to unit: one holds the running MFMA chain, the other the
  // previous unit's logits, whose registers take the next unit's bias as the exponentials let
  // go of them.  Before the first unit "the previous logits" are far below everything.
  f32x16 R0, R1;
#pragma unroll
  for (int r = 0; r < 16; ++r) R1[r] = kNegBig;
#pragma unroll
  for (int c = 0; c < 4; ++c) load_bias4(R0, c, 0, 0);

  for (int t = 0; t < ntiles; ++t) {
#pragma unroll
    for (int js = 0; js < NSUB; ++js) {
      KeyRegs& kr = K[js & 1];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int prev_rb = (rb + RB - 1) % RB;
        Stage st;
        Red red;
        const bool odd = ((js * RB + rb) & 1) != 0;
        f32x16& acc = odd ? R1 : R0;
        f32x16& acc_prev = odd ? R0 : R1;
        wait_lds();  // this unit's key operands (read one unit ago) are in their registers
        FS_SCHED_FENCE();
        auto k_first = [](int p) { return (p * NMAIN) / kSweepPieces; };  // MFMAs of piece p
#pragma unroll
        for (int p = 0; p < kSweepPieces; ++p) {
#pragma unroll
          for (int k = k_first(p); k < k_first(p + 1); ++k) acc = mfma_k(k, acc, kr, rb);
          // LDS / global traffic of the pipeline, placed where it has the whole unit to land
          if (js == 0 && rb == 0 && p == 0) stage_store(nxt);  // bias of tile t+1
          if (js == 0 && rb == 0 && p == 1) stage_load(j_begin + (t + 2) * JT, nx2);
          if (rb == RB - 1 && js + 1 < NSUB && p == 1) load_keys(K[(js + 1) & 1], cur, js + 1);
          if (rb == RB - 1 && js + 1 == NSUB && p == 1) {
            // tile t+1 has landed and this wave's bias store has been performed; tile t+2 stays
            // in flight across the barrier
            wait_older_tiles_and_lds();
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
          }
          if (rb == RB - 1 && js + 1 == NSUB && p == 2) load_keys(K[0], nxt, 0);
          // pieces 2c and 2c + 1 were the last to read logits 4c .. 4c + 3 of the previous unit:
          // their registers take the next unit's bias at piece 2c + 2
          if (p >= kSweepBiasPiece && p < kSweepBiasPiece + 8 && (p - kSweepBiasPiece) % 2 == 0) {
            const bool same_js = rb + 1 < RB;
            const bool same_tile = same_js || js + 1 < NSUB;
            load_bias4(acc_prev, (p - kSweepBiasPiece) / 2, same_tile ? cur : nxt, same_js ? js : (js + 1) % NSUB);
          }
          // The column sums of the sub-tile before this one are complete once the unit before
          // this one (second row block) has passed: its wavefront-wide sums are taken here, in
          // the second row block's unit, before this unit's exponentials reuse col[].
          if (rb == RB - 1) {
            // (before piece 3, where this unit's exponentials start to replace col[])
            if (p < 3) red_piece(p, red);
            // (js == 0: the second sub-tile of tile t - 1, before this tile's barrier; js == 1:
            // the first sub-tile of tile t, behind it: the merge of tile t - 1 reads in between)
            if (p == 4) red_store(red, js == 0 ? t + 1 : t, js == 0 ? 1 : 0);
            if (js + 1 == NSUB && p == 6 && t >= 1 && wave == (t & 3)) flush(t - 1);
          }
          soft_piece(p, st, acc_prev, prev_rb);
          FS_SCHED_FENCE();
        }
        soft_tail(st, prev_rb);
        FS_SCHED_FENCE();
      }
    }
    rotate();
  }
  // ---- the last unit's exponentials, the last sub-tile's column sums, the last tile's merge ----
  soft_whole(R1, RB - 1);
  {
    Red red;
#pragma unroll
    for (int p = 0; p < 3; ++p) red_piece(p, red);
    red_store(red, ntiles - 1, 1);
  }
  __syncthreads();
  if (wave == 0) flush(ntiles - 1);

#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = row0 + rb * 32 + li;
    const float s = run_s[rb] + xor32(run_s[rb]);
    if (row < sd.nq && h == 0) {
      const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
      *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(-cx[rb], s);
    }
  }
}

// The same for rows of 65 .. 128 columns.  Two row blocks of both planes are 128 registers of
// stationary operands, which leaves no room for lse_sweep_kernel's software pipeline; this
// kernel keeps its work-item mapping, its outputs and its merge, and does the rest plainly: a
// workgroup of four wavefronts shares 64-key tiles with both planes in LDS (two buffers of
// 32 KiB, the next tile and its bias terms arriving by direct loads; two workgroups per CU), a
// wavefront takes, per 32-key sub-tile, the three plane products of both row blocks (key
// operands one 16-column step ahead, read by hand), folds the key bias and the rows' own bias
// in with one fp32 MFMA per block, and sums the exponentials along the rows (lane-private) and,
// for both blocks together, along the columns (fs_colsum.hpp).  What hides the latencies is the
// second wavefront of the SIMD.
template <int T>
__global__ __launch_bounds__(256, 2) void lse_sweep128_kernel(const LaunchArgs args) {
  constexpr int DP = 128, RB = 2, JT = 64, NSUB = JT / 32, KK16 = DP / 16;
  constexpr int ROWW = DP;        // 32-bit words per two-plane row in global memory
  constexpr int ROWH = DP / 2;    // words per plane row in LDS
  constexpr int PPRH = ROWH / 4;  // 16-byte pieces per plane row
  constexpr int PER_PLANE = JT * PPRH / 256;
  static_assert(PPRH == 16 && PER_PLANE == 4, "64 keys x 16 pieces: four direct loads per lane and plane");

  __shared__ __attribute__((aligned(16))) unsigned lds_k[2][2][JT * ROWH];  // [buffer][plane]
  __shared__ __attribute__((aligned(16))) float lds_b[2][3][JT];            // the key bias terms as given
  __shared__ __attribute__((aligned(16))) float lds_col[2][4][2][JT];       // [tile parity][wavefront][row of 16 lanes][key]

  // the step may not run this kernel, or the device chose another variant
  if (args.sel[kSelSweep] == 0u) return;
  if (args.sweep == 2 && args.sel[kSelWord] != 1u) return;
  if (blockIdx.x == 0 && threadIdx.x == 0) args.sel[kSelRan] = 1u;

  // work items as in lse_sweep_kernel
  const bool self = args.sweep_self != 0;
  const int n_items = self ? args.sw_items : args.side[0].igroups * args.sw_splits;
  const int per_xcd = (n_items + 7) / 8;
  int item = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per_xcd || item >= n_items) return;
  const bool second = self && item >= args.sw_items0;
  if (second) item -= args.sw_items0;
  const Side& sd = second ? args.side[1] : args.side[0];
  const Side& so = self ? sd : args.side[1];
  const int sw_chunk = second ? args.sw_chunk_b : args.sw_chunk;
  int split, ig;
  if (self) {
    split = 0;
    for (;;) {
      const int g = self_groups_of_chunk(split, sw_chunk, sd.nk, sd.igroups);
      if (item < g) break;
      item -= g;
      ++split;
    }
    ig = item;
  } else {
    split = item / sd.igroups;
    ig = item % sd.igroups;
  }
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int h = lane >> 5;
  const int row0 = (ig * 4 + wave) * (32 * RB);
  const int j_begin = self ? max(split * sw_chunk, ig * 256) : split * sw_chunk;
  const int j_end = min(sd.nk, (split + 1) * sw_chunk);
  const int ntiles = (j_end - j_begin + JT - 1) / JT;
  if (ntiles <= 0) return;  // (whole workgroup: no barrier is left waiting)

  const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = 1.0f / lscale;

  // ---- stationary planes of the query rows, and the rows' own bias (base 2) ----
  u32x4 xh[RB][KK16], xl[RB][KK16];
  float cx[RB], run_s[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = min(row0 + rb * 32 + li, sd.nq - 1);
    const unsigned* qrow = sd.qplanes + (size_t)row * (size_t)ROWW;
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) {
      xh[rb][kk] = *reinterpret_cast<const u32x4*>(qrow + 8 * kk + 4 * h);
      xl[rb][kk] = *reinterpret_cast<const u32x4*>(qrow + ROWH + 8 * kk + 4 * h);
    }
    float r = so.kc0 * so.kb0[row];
    if (so.kb1 != nullptr) r += so.kc1 * so.kb1[row];
    if (so.kb2 != nullptr) r += so.kc2 * so.kb2[row];
    // rows past the last one (they repeat it) must not reach the column sums
    cx[rb] = (row0 + rb * 32 + li < sd.nq) ? fmaxf(r, kNegBig) : kNegBig;
    run_s[rb] = 0.f;
  }

  // ---- LDS access by hand (the compiler cannot tell a read of one buffer from the direct loads
  // filling the other and would make every access wait for them) ----
  auto lds_addr = [](const void* p) {
    return (unsigned)(size_t)(const __attribute__((address_space(3))) void*)p;
  };
  auto ds_read16 = [&](const unsigned* p) -> u32x4 {
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(lds_addr(p)) : "memory");
    return v;
  };
  auto ds_read4 = [&](const float* p) -> float {
    float v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(lds_addr(p)) : "memory");
    return v;
  };
  auto ds_write4 = [&](float* p, float v) {
    asm volatile("ds_write_b32 %0, %1" : : "v"(lds_addr(p)), "v"(v) : "memory");
  };
  auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
  auto wait_lds = [&]() {  // lgkmcnt(0), and nothing moves across
    fence();
    __builtin_amdgcn_s_waitcnt(0xC07F);
    fence();
  };
  auto barrier = [&]() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  // ---- key tiles: lane tid of round c fills LDS slot tid of a plane's buffer and fetches the
  // piece that belongs there (slot = piece ^ (row & 15); the four rounds of a plane are 16 rows
  // apart and share the permutation); the planes end in zero rows, so tiles past the chunk are
  // fetched like any other and masked by their bias ----
  const unsigned koff = (unsigned)(((tid / PPRH) * ROWW + (((tid % PPRH) ^ ((tid / PPRH) & 15)) * 4)) * 4);
  const char* ktile = reinterpret_cast<const char*>(sd.kplanes + (size_t)j_begin * (size_t)ROWW);
  auto issue_tile = [&](int buf) {  // the next tile in sequence
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int c = 0; c < PER_PLANE; ++c)
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(ktile + (p * ROWH + c * (256 / PPRH) * ROWW) * 4 + koff),
            (__attribute__((address_space(3))) void*)(&lds_k[buf][p][(c * 256 + wave * 64) * 4]), 16, 0, 0);
    ktile += JT * ROWW * 4;
  };
  // the (up to three) bias terms of the tile's keys as they are, by direct loads of wavefront 0
  // ahead of the tile's keys; absent terms re-read the first vector and are dropped later
  const float kc0 = sd.kc0, kc1 = sd.kc1, kc2 = sd.kc2;
  const bool has_kb1 = sd.kb1 != nullptr, has_kb2 = sd.kb2 != nullptr;
  const float* kb1p = has_kb1 ? sd.kb1 : sd.kb0;
  const float* kb2p = has_kb2 ? sd.kb2 : sd.kb0;
  auto issue_bias = [&](int j0, int buf) {
    if (wave == 0) {
      const int j = max(0, min(j0 + lane, sd.nk - 1));
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(sd.kb0 + j),
                                       (__attribute__((address_space(3))) void*)(&lds_b[buf][0][0]), 4, 0, 0);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kb1p + j),
                                       (__attribute__((address_space(3))) void*)(&lds_b[buf][1][0]), 4, 0, 0);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(kb2p + j),
                                       (__attribute__((address_space(3))) void*)(&lds_b[buf][2][0]), 4, 0, 0);
    }
  };
  auto mfma16 = [](const u32x4& a, const u32x4& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  };
  // the sums of a finished tile's keys over the four wavefronts and their two rows of 16 lanes,
  // in a fixed order, by one wavefront
  const int my_key = colsum_key(li, h);
  float* colp = (second ? args.col_part_b : args.col_part) + (size_t)ig * (size_t)sd.nk;
  auto flush = [&](int tile) {
    const float* c = &lds_col[tile & 1][0][0][0];
    float v[8];
#pragma unroll
    for (int w = 0; w < 8; ++w) v[w] = ds_read4(c + w * JT + lane);
    wait_lds();
    float sum = v[0] + v[1];
#pragma unroll
    for (int w = 1; w < 4; ++w) sum += v[2 * w] + v[2 * w + 1];
    const int j = j_begin + tile * JT + lane;
    if (j < j_end) colp[j] = sum;
  };

  // ---- prologue: tile 0 and its bias terms ----
  issue_bias(j_begin, 0);
  issue_tile(0);
  fence();
  __builtin_amdgcn_s_waitcnt(0x0070);  // everything has landed
  fence();
  barrier();

  int buf = 0;
  for (int t = 0; t < ntiles; ++t) {
    const int j0 = j_begin + t * JT;
    const int nbuf = buf ^ 1;
    // the other buffer was read during tile t - 1, which every wavefront has left
    issue_bias(j0 + JT, nbuf);
    issue_tile(nbuf);
    fence();
    // (every wavefront wrote its sums of tile t - 1 before the barrier it has just passed, and
    // writes those of tile t + 1 only behind the next one)
    if (t >= 1 && wave == (t & 3)) flush(t - 1);

#pragma unroll
    for (int js = 0; js < NSUB; ++js) {
      const unsigned* yhi = lds_k[buf][0] + (js * 32 + li) * ROWH;
      const unsigned* ylo = lds_k[buf][1] + (js * 32 + li) * ROWH;
      float kb0r = ds_read4(&lds_b[buf][0][js * 32 + li]);
      float kb1r = ds_read4(&lds_b[buf][1][js * 32 + li]);
      float kb2r = ds_read4(&lds_b[buf][2][js * 32 + li]);
      // the three plane products of both row blocks, the key operands one step ahead
      u32x4 kh[2], kl[2];
      kh[0] = ds_read16(yhi + (((0 + h) ^ (li & 15)) << 2));
      kl[0] = ds_read16(ylo + (((0 + h) ^ (li & 15)) << 2));
      f32x16 acc[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rb][r] = 0.f;
#pragma unroll
      for (int kk = 0; kk < KK16; ++kk) {
        wait_lds();
        if (kk + 1 < KK16) {
          kh[(kk + 1) & 1] = ds_read16(yhi + (((2 * (kk + 1) + h) ^ (li & 15)) << 2));
          kl[(kk + 1) & 1] = ds_read16(ylo + (((2 * (kk + 1) + h) ^ (li & 15)) << 2));
        }
        // (plane products from the lowest weight to hi*hi; the two blocks alternate)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = mfma16(kl[kk & 1], xh[rb][kk], acc[rb]);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = mfma16(kh[kk & 1], xl[rb][kk], acc[rb]);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = mfma16(kh[kk & 1], xh[rb][kk], acc[rb]);
      }
      fence();
      asm volatile("" : "+v"(kb0r), "+v"(kb1r), "+v"(kb2r));  // (read before the first wait above)
      float kbias = kc0 * kb0r + (has_kb1 ? kc1 * kb1r : 0.f);
      kbias += (has_kb2 ? kc2 * kb2r : 0.f);
      kbias = (j0 + js * 32 + li < j_end) ? fmaxf(kbias, kNegBig) : kNegBig;  // keys past the chunk are masked
      kbias = fmaxf(kbias * inv_lscale, -3.0e38f);
      float c[16];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        // + key bias + the row's own bias: A = [bias_j, 1], B = [1, r_i]
        acc[rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(h ? 1.0f : kbias, h ? fmaxf(cx[rb] * inv_lscale, -3.0e38f) : 1.0f,
                                                       acc[rb], 0, 0, 0);
        float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float e0 = fast_exp2(acc[rb][r] * lscale);
          const float e1 = fast_exp2(acc[rb][r + 1] * lscale);
          ps0 += e0;
          ps1 += e1;
          if (rb == 0) {
            c[r] = e0;
            c[r + 1] = e1;
          } else {
            c[r] += e0;
            c[r + 1] += e1;
          }
        }
        run_s[rb] += ps0 + ps1;
      }
      ds_write4(&lds_col[t & 1][wave][li >> 4][js * 32 + my_key], colsum_all(c, li));
    }

    // tile t + 1 has landed (and with it its bias terms), this wavefront's column sums are
    // written; after the barrier all of it is visible and every wavefront is done reading tile t
    fence();
    __builtin_amdgcn_s_waitcnt(0x0070);
    fence();
    barrier();
    buf = nbuf;
  }
  fence();
  __builtin_amdgcn_s_waitcnt(0x0070);  // what was fetched past the chunk: let it land before the end
  fence();
  if (wave == 0) flush(ntiles - 1);

#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = row0 + rb * 32 + li;
    const float s = run_s[rb] + xor32(run_s[rb]);
    if (row < sd.nq && h == 0) {
      const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
      *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(-cx[rb], s);
    }
  }
}

// Merge after lse_sweep_kernel: rows of side 0 add their partial row sums over the key chunks
// (all taken under the same offset, the row's own bias), rows of side 1 (the keys) add the
// column sums of the workgroup row groups.  A sum outside [2^kSweepFailLo, 2^kSweepFailHi]
// raises kSelSweepFail: the two-sided kernel and its merge, enqueued behind this one, then redo
// the step and overwrite what this kernel wrote.
template <int T>
__global__ __launch_bounds__(256) void finish_sweep_kernel(const LaunchArgs args) {
  unsigned* st = args.sel;
  if (st[kSelSweep] == 0u) return;
  if (args.sweep == 2 && st[kSelWord] != 1u) return;
  const Side& s0 = args.side[0];
  const Side& s1 = args.side[1];
  const bool self = args.sweep_self != 0;
  const int rows1 = (self && args.sw_items == args.sw_items0) ? 0 : s1.nq;  // (self: side 1 may be absent)
  int it = blockIdx.x * 256 + threadIdx.x;
  const bool live = it < s0.nq + rows1;
  float l2 = 0.f;
  if (live) {
    const bool second = it >= s0.nq;
    const int row = second ? it - s0.nq : it;
    float M, s = 0.f;
    if (self) {
      // the row's partial sums over the chunks that reach its row group, and what the row
      // groups before its own added to it as one of their keys
      const Side& sd = second ? s1 : s0;
      const int chunk = second ? args.sw_chunk_b : args.sw_chunk;
      const int splits = second ? args.sw_splits_b : args.sw_splits;
      const float* colp = second ? args.col_part_b : args.col_part;
      const int g_own = row >> 8;
      float b = sd.kc0 * sd.kb0[row];
      if (sd.kb1 != nullptr) b += sd.kc1 * sd.kb1[row];
      if (sd.kb2 != nullptr) b += sd.kc2 * sd.kb2[row];
      M = -fmaxf(b, kNegBig);
#pragma unroll 4
      for (int sp = max(1, args.sw_part_mult) * ((g_own * 256) / chunk); sp < splits; ++sp)
        s += sd.part_ms[2 * ((size_t)sp * sd.nq + row) + 1];
#pragma unroll 8
      for (int g = 0; g < g_own; ++g) s += colp[(size_t)g * sd.nk + row];
    } else if (!second) {
      M = s0.part_ms[2 * (size_t)row];
#pragma unroll 8
      for (int sp = 0; sp < args.sw_splits; ++sp) s += s0.part_ms[2 * ((size_t)sp * s0.nq + row) + 1];
    } else {
      float b = s0.kc0 * s0.kb0[row];
      if (s0.kb1 != nullptr) b += s0.kc1 * s0.kb1[row];
      if (s0.kb2 != nullptr) b += s0.kc2 * s0.kb2[row];
      M = -fmaxf(b, kNegBig);
#pragma unroll 8
      for (int g = 0; g < s0.igroups; ++g) s += args.col_part[(size_t)g * s0.nk + row];
    }
    l2 = log2f(s);
    epilogue_scalar(second ? s1.ep : s0.ep, row, M, s, 0.f);
  }
  if (live && !(l2 >= kSweepFailLo && l2 <= kSweepFailHi)) st[kSelSweepFail] = 1u;
  sweep_note_sums(st, l2, live);
}

}  // namespace fs
