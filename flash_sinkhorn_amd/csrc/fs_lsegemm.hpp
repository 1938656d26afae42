// Log-sum-exp and plan-times-vector kernel for large feature dimension (d > 128) on fp16
// planes.  VEC adds the weighted sum  sum_j p_ij v_j  next to  sum_j p_ij  in the soft-max of
// each tile (plan-vector products); everything else is shared.
//
// With d in the hundreds a block of query rows no longer fits in registers, so the sweep is
// organised like a GEMM: a workgroup of 8 wavefronts owns 256 query rows, walks its key
// chunk in tiles of 256 keys and, per tile, runs a k-loop over the feature axis in chunks of
// 32 columns.  Each k-step brings the 32-column slice of the 256 query rows and of the 256
// key rows into LDS (128 bytes per row: 16 words of the hi plane, 16 of the lo plane, which
// the chunked plane layout stores contiguously) with direct global->LDS loads, double
// buffered, one barrier per k-step.  Wavefront (qg, kg) accumulates the logits of query rows
// [64 qg, 64 qg + 64) against keys [128 kg, 128 kg + 128) of the tile: 2 x 4 MFMA tiles of
// 32 keys x 32 queries = 128 accumulator registers, three fp16 products per tile and
// 16 columns.  After the k-loop the bias / running-max fold and the lane-private online
// soft-max run once per tile, which is noise next to 3*d/16 MFMAs per tile.  The two key
// groups of a workgroup write separate partial statistics, so the merge kernel sees twice
// the workgroup-level split count.
//
// LDS rows are 128 bytes with no padding (a direct load deposits 64 lanes x 16 bytes
// contiguously); 16-byte piece p of local row r sits in slot p ^ ((r >> 1) & 7), which
// makes the ds_read_b128 of 16 consecutive rows at one piece index conflict free.
#pragma once

#include <type_traits>
#include <utility>

#include "fs_colsum.hpp"
#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}) in order
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// 16 bytes from LDS at byte address addr + OFF (OFF < 65536), not visible to the compiler's
// wait-count insertion: the consumer must sit behind an explicit wait
template <int OFF>
__device__ __forceinline__ u32x4 lds_read16(unsigned addr) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
  return v;
}

constexpr int kGemmRows = 256;   // query rows per workgroup = keys per tile
constexpr int kGemmCols = 32;    // feature columns per k-step

// GM: 0 log-sum-exp, 1 plan-vector (VEC), 2 running arg-max of the logits (c-transform),
// 3 both sides of a two-sided log-sum-exp step from one sweep (SWP): side 0's grid only, the
// bias of the query rows (as keys of side 1) joins the key bias in the fold, the exponentials
// are taken without a running maximum and summed along the rows (lane-private, as for GM 0)
// and along the columns (fs_colsum.hpp over the 32 lanes of a half-wave, then over the four
// wavefronts of a key group through LDS; one row of column sums per workgroup in
// LaunchArgs::col_part).  What makes that exact, who permits it and what happens when a sum
// leaves the range is lse_sweep_kernel's story (fs_lsesweep.hpp); the merge is shared with it.
template <int GM>
__global__ __launch_bounds__(512, 1) void lse_gemm_kernel(const LaunchArgs args) {
  constexpr bool VEC = (GM == 1);
  constexpr bool AMAX = (GM == 2);
  constexpr bool SWP = (GM == 3);
  __shared__ __attribute__((aligned(16))) unsigned lds[2][2 * kGemmRows * 32];
  __shared__ __attribute__((aligned(16))) float lds_v[2][VEC ? kGemmRows : 4];  // v of a key tile
  // SWP: column sums of a tile, [wavefront][row of 16 lanes][key of the wavefront's 128]
  __shared__ __attribute__((aligned(16))) float lds_col[SWP ? 8 : 1][2][SWP ? 128 : 1];

  if constexpr (SWP) {
    if (args.sel[kSelSweep] == 0u) return;  // the step before did not permit it
  }
  if constexpr (GM == 0) {
    // a step with a one-sweep launch ahead of this one: nothing to do unless that launch did
    // not run or its sums left the range
    if (args.sweep != 0 && args.sel[kSelSweep] != 0u && args.sel[kSelSweepFail] == 0u) return;
  }

  // Work items: side 0's, then side 1's, each side in the order (block of 4 row groups, key
  // chunk, row group of the block).  Workgroups are dealt round-robin to the 8 XCDs, and XCD x
  // takes the x-th eighth of the items in that order, so the workgroups that share an L2 share
  // few row groups AND few key chunks.  (With all row groups of one key chunk on an XCD every
  // workgroup fetched its own query rows from memory once per key tile: 1.66 GB per one-sweep
  // launch at 8192 x 8192 x 1536 instead of 0.6.)
  // SWP on problems of a matrix with itself (LaunchArgs::sweep_self): side 0's items, then side
  // 1's, key chunk slowest; a chunk only has items for the row groups that begin before its end.
  const bool self = SWP && args.sweep_self != 0;
  const int n_items = SWP ? (self ? args.sw_items : args.side[0].igroups * (args.sw_splits >> 1))
                          : args.blocks_all;
  const int per_xcd = (n_items + 7) / 8;
  int item = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
  if (((int)blockIdx.x >> 3) >= per_xcd || item >= n_items) return;  // (whole workgroup, before any barrier)
  const int items0 = SWP ? args.sw_items0 : args.blocks0;
  const bool second = (SWP ? self : true) && item >= items0;
  if (second) item -= items0;
  const Side& sd = second ? args.side[1] : args.side[0];
  const int dp = args.pstride;  // words per plane row pair
  const int nch = (args.d + kGemmCols - 1) / kGemmCols;

  // workgroup-level key splits
  const int bsplits = (SWP ? (second ? args.sw_splits_b : args.sw_splits) : sd.splits) >> 1;
  const int chunk = SWP ? (second ? args.sw_chunk_b : args.sw_chunk) : sd.chunk;
  int split, ig;
  if (self) {
    split = 0;
    for (;;) {  // (item < the number of items of this side: ends within its chunks)
      const int g = self_groups_of_chunk(split, chunk, sd.nk, sd.igroups);
      if (item < g) break;
      item -= g;
      ++split;
    }
    ig = item;
  } else {
    const int blk = item / (4 * bsplits), within = item % (4 * bsplits);
    const int nb = min(4, sd.igroups - 4 * blk);
    split = within / nb;
    ig = 4 * blk + within % nb;
  }
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int h = lane >> 5;
  const int qg = wave & 3;
  const int kg = wave >> 2;
  const int row0 = ig * kGemmRows;
  // (self: from the first row of this row group on; chunks are multiples of the 256 keys of a tile)
  const int j_begin = self ? max(split * chunk, ig * kGemmRows) : split * chunk;
  const int j_end = min(sd.nk, (split + 1) * chunk);
  const int ntiles = (j_end - j_begin + kGemmRows - 1) / kGemmRows;

  const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = 1.0f / lscale;

  // ---- loader role: wavefronts 0-3 bring query rows, 4-7 key rows (64 rows each) ----
  // instruction i of a k-step covers local rows 8 i .. 8 i + 7 of this wavefront's 64
  const bool load_q = wave < 4;
  int loff[8];  // word offset of this lane's 16-byte piece inside the wavefront's row block
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int lr = i * 8 + (lane >> 3);                 // row inside the 64-row block
    const int piece = (lane & 7) ^ ((lr >> 1) & 7);     // (64 w) >> 1 has no low bits
    loff[i] = lr * dp + piece * 4;
  }
  const unsigned* qbase = sd.qplanes + (size_t)(row0 + (wave & 3) * 64) * (size_t)dp;
  auto issue_loads = [&](int buf, int j0, int c) {
    const unsigned* base =
        load_q ? qbase : sd.kplanes + (size_t)(j0 + (wave & 3) * 64) * (size_t)dp;
    unsigned* dst = &lds[buf][(wave * 64) * 32];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(base + loff[i] + c * kGemmCols),
          (__attribute__((address_space(3))) void*)(dst + i * 8 * 32), 16, 0, 0);
  };

  // ---- reader addresses: piece p of local row r at word r*32 + ((p ^ ((r>>1)&7)) * 4) ----
  // Stage reads are ds_read_b128 written out by hand: the compiler cannot tell a read of one
  // stage buffer from the global->LDS loads filling the other and would make every read wait
  // for the loads just issued (which is what it did: the prefetch of the next k-step was waited
  // for before the current one was even read).  It does not see these reads either: their
  // consumers sit behind wait_lds().  A lane reads the same four pieces (plane, 16-column half)
  // of every row block; block and stage go into the instruction's offset and a toggled bit, so
  // eight address registers serve all 24 reads of a k-step.
  unsigned qaddr[2][2], kaddr[2][2];  // [plane][half]: byte addresses in the current stage
  {
    const unsigned base = (unsigned)(size_t)(const __attribute__((address_space(3))) unsigned*)&lds[0][0];
    const int sw = (li >> 1) & 7;  // (row blocks start at multiples of 32 rows)
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const int slot = (p * 4 + kk * 2 + h) ^ sw;
        qaddr[p][kk] = base + (unsigned)(((qg * 64 + li) * 32 + slot * 4) * 4);
        kaddr[p][kk] = base + (unsigned)(((kGemmRows + kg * 128 + li) * 32 + slot * 4) * 4);
      }
  }
  static_assert(sizeof(lds[0]) == 65536, "the stages are one address bit apart");
  auto wait_lds = [&](auto newer) {  // at most `newer` of the reads issued last are still in flight
    constexpr int n = decltype(newer)::value;
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xC07F | (n << 8));  // lgkmcnt(n)
    __builtin_amdgcn_sched_barrier(0);
  };

  f32x16 acc[2][4];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb)
#pragma unroll
    for (int st = 0; st < 4; ++st)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[qb][st][r] = 0.f;
  // run_c: minus the running maximum in base-2 units as rounded once, the constant of the
  // exponentials (the logits stay in absolute raw units: a running maximum subtracted inside
  // the accumulator costs them their digits whenever it lies far below them, after a first
  // tile of keys without weight, say)
  float run_m[2] = {0.f, 0.f}, run_c[2] = {0.f, 0.f}, run_s[2] = {0.f, 0.f}, run_o[2] = {0.f, 0.f};
  int best_j[2] = {0, 0};  // AMAX: run_m holds the largest raw value so far, best_j its key
  if constexpr (AMAX) run_m[0] = run_m[1] = -3.0e38f;
  float rbias[2] = {0.f, 0.f};  // SWP: the rows' own bias (base 2), as keys of the other side
  if constexpr (SWP) {
    const Side& so = self ? sd : args.side[1];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int row = row0 + qg * 64 + qb * 32 + li;
      const int rr = min(row, sd.nq - 1);
      float r = so.kc0 * so.kb0[rr];
      if (so.kb1 != nullptr) r += so.kc1 * so.kb1[rr];
      if (so.kb2 != nullptr) r += so.kc2 * so.kb2[rr];
      // rows past the last one must not reach the column sums
      rbias[qb] = row < sd.nq ? fmaxf(r, kNegBig) : kNegBig;
    }
  }

  auto swap_halves = [&](float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  };

  issue_loads(0, j_begin, 0);
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  int buf = 0;
  for (int t = 0; t < ntiles; ++t) {
    const int j0 = j_begin + t * kGemmRows;
    if constexpr (VEC) {
      // the barriers of the k-loop publish it; tile t + 2 overwrites it after every wavefront
      // has passed a barrier of tile t + 1, hence finished the soft-max of tile t
      if (tid < kGemmRows) lds_v[t & 1][tid] = (j0 + tid < j_end) ? sd.v[j0 + tid] : 0.f;
    }
    for (int c = 0; c < nch; ++c) {
      // next k-step (or the first one of the next tile) goes into the other buffer
      const bool wrap = (c + 1 == nch);
      if (!wrap || t + 1 < ntiles) issue_loads(buf ^ 1, wrap ? j0 + kGemmRows : j0, wrap ? 0 : c + 1);

      u32x4 qreg[2][2][2];  // [query block][plane][16-column half]
      u32x4 kreg[2][2][2];  // [slot][plane][half]: sub-tile st in slot st % 2
      static_for<2>([&](auto qb_) {
        constexpr int qb = decltype(qb_)::value;
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) qreg[qb][p][kk] = lds_read16<qb * 32 * 128>(qaddr[p][kk]);
      });
      auto read_keys = [&](auto st_) {
        constexpr int st = decltype(st_)::value;
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) kreg[st % 2][p][kk] = lds_read16<st * 32 * 128>(kaddr[p][kk]);
      };
      read_keys(std::integral_constant<int, 0>{});
      read_keys(std::integral_constant<int, 1>{});
      // sub-tile st + 2 is requested into the registers of sub-tile st once its MFMAs are
      // issued (they have read their operands by then), and lands while those of st + 1 run
      static_for<4>([&](auto st_) {
        constexpr int st = decltype(st_)::value;
        if constexpr (st < 3) wait_lds(std::integral_constant<int, 4>{});
        else wait_lds(std::integral_constant<int, 0>{});
        // products lo*hi, hi*lo, hi*hi; the two query blocks alternate, so no MFMA waits for
        // the one just before it
#pragma unroll
        for (int prod = 0; prod < 3; ++prod)
#pragma unroll
          for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int qb = 0; qb < 2; ++qb) {
              const int pk = (prod == 0) ? 1 : 0, pq = (prod == 1) ? 1 : 0;
              acc[qb][st] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, kreg[st % 2][pk][kk]),
                  __builtin_bit_cast(f16x8, qreg[qb][pq][kk]), acc[qb][st], 0, 0, 0);
            }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (st < 2) read_keys(std::integral_constant<int, st + 2>{});
      });
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0);  // this wavefront's direct loads have landed
      __syncthreads();
      buf ^= 1;
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          qaddr[p][kk] ^= 65536u;
          kaddr[p][kk] ^= 65536u;
        }
    }

    // ---- tile done: fold bias - M, lane-private online soft-max over the 4 sub-tiles ----
    float ab[4];
#pragma unroll
    for (int st = 0; st < 4; ++st)
      ab[st] = h ? 1.0f : key_bias(sd, j0 + kg * 128 + st * 32 + li, j_end) * inv_lscale;
    if constexpr (SWP) {
      const float rq[2] = {h ? rbias[0] * inv_lscale : 1.0f, h ? rbias[1] * inv_lscale : 1.0f};
      const int my_key = colsum_key(li, h);
      float rs0[2] = {0.f, 0.f}, rs1[2] = {0.f, 0.f};
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        float c[16];
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
          acc[qb][st] = __builtin_amdgcn_mfma_f32_32x32x2f32(ab[st], rq[qb], acc[qb][st], 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float e00 = fast_exp2(acc[0][st][r] * lscale);
          const float e01 = fast_exp2(acc[0][st][r + 1] * lscale);
          const float e10 = fast_exp2(acc[1][st][r] * lscale);
          const float e11 = fast_exp2(acc[1][st][r + 1] * lscale);
          rs0[0] += e00;
          rs1[0] += e01;
          rs0[1] += e10;
          rs1[1] += e11;
          c[r] = e00 + e10;
          c[r + 1] = e01 + e11;
        }
        lds_col[wave][li >> 4][st * 32 + my_key] = colsum_all(c, li);
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[qb][st][r] = 0.f;
      }
      run_s[0] += rs0[0] + rs1[0];
      run_s[1] += rs0[1] + rs1[1];
      // the sums of the four wavefronts of a key group and of their two rows of 16 lanes, in a
      // fixed order; the next tile's sums reach LDS only after the barriers of its k-loop
      __syncthreads();
      if (tid < kGemmRows) {
        const int kgk = tid >> 7, kk = tid & 127;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) v += lds_col[kgk * 4 + w][0][kk] + lds_col[kgk * 4 + w][1][kk];
        float* colp = second ? args.col_part_b : args.col_part;
        if (j0 + tid < j_end) colp[(size_t)ig * (size_t)sd.nk + (size_t)(j0 + tid)] = v;
      }
      continue;
    }
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      if constexpr (AMAX) {
        // keys ascend with st and r inside a lane, tiles ascend: a strict test keeps the
        // smallest key among equal values
#pragma unroll
        for (int st = 0; st < 4; ++st) {
          acc[qb][st] =
              __builtin_amdgcn_mfma_f32_32x32x2f32(ab[st], h ? 0.0f : 1.0f, acc[qb][st], 0, 0, 0);
          const int jb = j0 + kg * 128 + st * 32 + 4 * h;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            if (acc[qb][st][r] > run_m[qb]) {
              run_m[qb] = acc[qb][st][r];
              best_j[qb] = jb + 8 * (r / 4) + (r % 4);
            }
            acc[qb][st][r] = 0.f;
          }
        }
        continue;
      }
      float m = -3.0e38f;
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        acc[qb][st] =
            __builtin_amdgcn_mfma_f32_32x32x2f32(ab[st], h ? 0.0f : 1.0f, acc[qb][st], 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 16; ++r) m = fmaxf(m, acc[qb][st][r]);
      }
      float a = m, b = m;
      swap_halves(a, b);
      m = fmaxf(a, b);
      const bool first = (t == 0);
      float cc = -m * lscale;
      asm volatile("" : "+v"(cc));  // the exponents, the rescale and the result see one number
      cc = first ? cc : fminf(cc, run_c[qb]);
      float ps0 = 0.f, ps1 = 0.f, po0 = 0.f, po1 = 0.f;
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        if constexpr (VEC) {
          // accumulator register 4 g + i of a lane holds key 8 g + 4 h + i of the sub-tile
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float4 vv = *reinterpret_cast<const float4*>(
                &lds_v[t & 1][kg * 128 + st * 32 + 8 * g + 4 * h]);
            const float e0 = fast_exp2(__builtin_fmaf(acc[qb][st][4 * g], lscale, cc));
            const float e1 = fast_exp2(__builtin_fmaf(acc[qb][st][4 * g + 1], lscale, cc));
            const float e2 = fast_exp2(__builtin_fmaf(acc[qb][st][4 * g + 2], lscale, cc));
            const float e3 = fast_exp2(__builtin_fmaf(acc[qb][st][4 * g + 3], lscale, cc));
            ps0 += e0 + e2;
            ps1 += e1 + e3;
            po0 = __builtin_fmaf(e0, vv.x, __builtin_fmaf(e2, vv.z, po0));
            po1 = __builtin_fmaf(e1, vv.y, __builtin_fmaf(e3, vv.w, po1));
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            ps0 += fast_exp2(__builtin_fmaf(acc[qb][st][r], lscale, cc));
            ps1 += fast_exp2(__builtin_fmaf(acc[qb][st][r + 1], lscale, cc));
          }
        }
      }
      const float resc = first ? 0.f : fast_exp2(cc - run_c[qb]);
      run_s[qb] = run_s[qb] * resc + (ps0 + ps1);
      if constexpr (VEC) run_o[qb] = run_o[qb] * resc + (po0 + po1);
      run_c[qb] = cc;
#pragma unroll
      for (int st = 0; st < 4; ++st)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[qb][st][r] = 0.f;
    }
  }

  // ---- partial statistics of this (query group, key group) ----
  const bool has_keys = (j_begin + kg * 128) < j_end;  // else every key this wave saw was masked
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int row = row0 + qg * 64 + qb * 32 + li;
    if constexpr (AMAX) {
      float best = run_m[qb];
      int bj = best_j[qb];
      const float ob = xor32(best);
      const int oj = __shfl_xor(bj, 32, 64);
      if (ob > best || (ob == best && oj < bj)) {
        best = ob;
        bj = oj;
      }
      if (row < sd.nq && h == 0) {
        const size_t pr = (size_t)(split * 2 + kg) * (size_t)sd.nq + (size_t)row;
        *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) =
            has_keys ? make_float2(best * lscale, __builtin_bit_cast(float, bj))
                     : make_float2(-3.0e38f, __builtin_bit_cast(float, 0x7fffffff));
      }
      continue;
    }
    const float s = run_s[qb] + xor32(run_s[qb]);
    if constexpr (SWP) {
      // every partial sum of a row is taken under the same offset, the row's own bias (a
      // wavefront whose keys were all masked adds zero)
      if (row < sd.nq && h == 0) {
        const size_t pr = (size_t)(split * 2 + kg) * (size_t)sd.nq + (size_t)row;
        *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(-rbias[qb], s);
      }
      continue;
    }
    if (row < sd.nq && h == 0) {
      const size_t pr = (size_t)(split * 2 + kg) * (size_t)sd.nq + (size_t)row;
      *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) =
          has_keys ? make_float2(-run_c[qb], s) : make_float2(kNegBig, 0.f);
    }
    if constexpr (VEC) {
      const float o = run_o[qb] + xor32(run_o[qb]);
      if (row < sd.nq && h == 0)
        sd.part_o[(size_t)(split * 2 + kg) * (size_t)sd.nq + (size_t)row] = has_keys ? o : 0.f;
    }
  }
}

}  // namespace fs
