// Plan-times-matrix and plan-times-vector products and the hard c-transform for d <= 128 on
// fp16 planes (gradient, apply_plan_mat, apply_plan_vec, c_transform in the default operand mode).
//
// Same decomposition as lse2_kernel: a workgroup of 4 wavefronts shares key tiles of 64 keys
// (32 for 128-column rows, which would not leave room for two workgroups per CU otherwise),
// brought into LDS by direct global->LDS loads of the two-plane fp16 rows (three buffers, the
// tile two ahead in flight, XOR-swizzled 16-byte slots), and every wavefront owns RB blocks
// of 32 query rows whose planes never leave its registers.  Per block and 32-key sub-tile:
//   logits   3 fp16 MFMA products per 16 columns, then one fp32 MFMA that adds the key bias
//            and subtracts the block's running maximum (both in units of the raw products);
//   soft-max lane-private and lazy: the running maximum moves only when a tile exceeds it by
//            2^4, so the exponentials stay below 2^4 (2^15 after the shift below): fp16-safe;
//   values   (kMat) the lane's own 16 probabilities are, as they stand, its B operands of the
//            two 16-key steps; they are split into hi / lo fp16 and multiplied with the V^T
//            operands that transpose_planes_f16_kernel laid out in MFMA order in global memory
//            (one coalesced 1 KiB read per instruction, shared by the four wavefronts through
//            L1): three products per column block and step.  (kVec) a weighted sum with the
//            values of v of the tile, staged in LDS.  (kMat5) as kMat with the probabilities
//            multiplied by T = <A_i, y_j>, a second contraction on planes of A held in
//            registers, scaled per row by a power of two from |A_i| max|y_j| so that p T stays
//            fp16-safe (see plan_gemm_kernel).  (kArgmax) no soft-max at all: a running
//            (largest value, key) pair per lane, ties to the smaller key.
// Row sums are exact fp32 VALU sums.  The key bias of the next tile travels in two registers
// per lane; nothing in the loop needs a second barrier.
#pragma once

#include <type_traits>

#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

constexpr float kPtLazyThresh = 4.0f;  // exponentials stay below 2^4 relative to the running maximum
// The exponentials are taken 2^11 up before they are cut into fp16 planes (values up to 2^15), and
// the maximum a row reports is lowered by the same 11: the pair (maximum, sums) means the same
// thing, while a probability keeps a nonzero fp16 image down to 2^-35 of the row's largest one
// instead of 2^-24 (a tail of many far keys would otherwise be rounded away one-sidedly).
constexpr float kPtUp = 11.0f;

template <int DP, int RB, int MODE>
__global__ __launch_bounds__(256, (MODE == kMat5 && DP == 128) ? 1 : 2) void plan_tile_kernel(const LaunchArgs args) {
  static_assert(MODE == kMat || MODE == kVec || MODE == kArgmax || MODE == kMat5,
                "plan_tile_kernel modes");
  static_assert(MODE != kMat5 || RB == 1, "mat5: the second operand needs registers");
  constexpr bool kHasO = (MODE == kMat || MODE == kMat5);
  static_assert(DP == 16 || DP == 32 || DP == 64 || DP == 128, "padded row widths");
  constexpr int kPtKeys = (DP == 128) ? 32 : 64;  // keys per tile
  constexpr int NSUB = kPtKeys / 32;
  // 128-column rows, and the matrix product with two row blocks at 64 columns (which spills
  // otherwise): key operands are read from LDS step by step instead of being held
  constexpr bool kStreamK = (DP == 128) || (DP == 64 && RB == 2 && MODE == kMat);
  constexpr int KK16 = DP / 16;                 // 16-column steps of the logits
  constexpr int NCB = (DP + 31) / 32;           // 32-column output blocks
  constexpr int ROWW = DP;                      // words per two-plane row
  constexpr int PPR = ROWW / 4;                 // 16-byte pieces per row
  constexpr int PER_THREAD = kPtKeys * PPR / 256;
  static_assert(kPtKeys * PPR % 256 == 0, "a tile is a whole number of load instructions");

  __shared__ __attribute__((aligned(16))) unsigned lds_k[3][kPtKeys * ROWW];
  __shared__ __attribute__((aligned(16))) float lds_v[3][MODE == kVec ? kPtKeys : 4];

  int bid = blockIdx.x;
  const bool second = bid >= args.blocks0;
  if (second) bid -= args.blocks0;
  const Side& sd = second ? args.side[1] : args.side[0];
  const int d = args.d;
  const bool vec_ok = args.vec_ok != 0;

  const int split = bid % sd.splits;
  const int ig = bid / sd.splits;
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int h = lane >> 5;
  const int row0 = (ig * 4 + wave) * (32 * RB);
  const int j_begin = split * sd.chunk;
  const int j_end = min(sd.nk, j_begin + sd.chunk);
  const int ntiles = (j_end > j_begin) ? (j_end - j_begin + kPtKeys - 1) / kPtKeys : 0;

  const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = 1.0f / lscale;
  // base-2 units: -40, or so far down that nothing is skipped (LaunchArgs::skip_log2)
  const float skip_below = args.skip_log2;

  // ---- stationary query planes: [block][plane][16-column step] ----
  u32x4 xq[RB][2][KK16];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = min(row0 + rb * 32 + li, sd.nq - 1);
    const unsigned* qrow = sd.qplanes + (size_t)row * (size_t)ROWW;
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int kk = 0; kk < KK16; ++kk)
        xq[rb][p][kk] = *reinterpret_cast<const u32x4*>(qrow + p * (DP / 2) + 8 * kk + 4 * h);
  }

  u32x4 aq[MODE == kMat5 ? RB : 1][2][MODE == kMat5 ? KK16 : 1];
  float t_unit = 1.0f;
  if constexpr (MODE == kMat5) {
    const int row = min(row0 + li, sd.nq - 1);
    const unsigned* arow = sd.q2planes + (size_t)row * (size_t)ROWW;
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int kk = 0; kk < KK16; ++kk)
        aq[0][p][kk] = *reinterpret_cast<const u32x4*>(arow + p * (DP / 2) + 8 * kk + 4 * h);
    // per-row power of two with |T_ij| * t_unit <= 1 from |T_ij| <= |A_i| max_j |y_j|
    float km = sd.kmax2[lane];  // 64 partial maxima of |y_j|^2
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) km = fmaxf(km, __shfl_xor(km, o, 64));
    const float bound =
        sqrtf(sd.q2norm2[row] * km) * sd.q2plane_scale[0] * sd.kplane_scale[0] * 1.0001f;
    const int e = (int)((__builtin_bit_cast(unsigned, bound) >> 23) & 255u);  // bound < 2^(e-126)
    if (e > 0 && e < 255)
      t_unit = __builtin_bit_cast(float, (unsigned)min(254, max(1, 127 - (e - 126))) << 23);
  }

  // ---- key tiles: lane idx of instruction c fills LDS slot idx and fetches the piece that
  // belongs there (slot = piece ^ swz(row)) ----
  auto swz = [&](int r) {
    return PPR >= 16 ? (r & 15) : (PPR == 8 ? ((r >> 1) & 7) : ((r >> 2) & 3));
  };
  // (one wave-uniform running base and 32-bit lane offsets: four 64-bit pointers per lane are
  // what tipped the matrix product at 64 columns into spilling inside the tile loop, and a
  // reload from scratch there waits for every load in flight)
  unsigned koff[PER_THREAD];
#pragma unroll
  for (int c = 0; c < PER_THREAD; ++c) {
    const int idx = tid + 256 * c;
    const int r = idx / PPR;
    const int piece = (idx % PPR) ^ swz(r);
    koff[c] = (unsigned)((r * ROWW + piece * 4) * 4);
  }
  const char* ktile = reinterpret_cast<const char*>(sd.kplanes + (size_t)j_begin * (size_t)ROWW);
  auto issue_tile = [&](int buf) {  // the next tile in sequence; the planes end in zero rows
#pragma unroll
    for (int c = 0; c < PER_THREAD; ++c) {
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(ktile + koff[c]),
          (__attribute__((address_space(3))) void*)(&lds_k[buf][(c * 256 + wave * 64) * 4]), 16, 0,
          0);
    }
    ktile += kPtKeys * ROWW * 4;
  };
  auto wait_newest_tile_only = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (PER_THREAD & 15));
  };
  auto lds_piece = [&](const unsigned* tile, int r, int piece) {
    return *reinterpret_cast<const u32x4*>(tile + r * ROWW + ((piece ^ swz(r)) << 2));
  };
  // the same by hand (see the streamed logits below): invisible to the compiler's wait counts,
  // the consumer sits behind wait_lds()
  auto lds_read16 = [&](const unsigned* p) -> u32x4 {
    u32x4 v;
    const unsigned addr = (unsigned)(size_t)(const __attribute__((address_space(3))) unsigned*)p;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
  };
  auto wait_lds = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
  };
  // Bias of key j (lanes with h == 0 feed it to the fp32 MFMA), in units of the raw products.
  // Its up to three terms are fetched raw, one tile ahead and without branches (absent terms
  // re-read the first vector and are dropped when the terms are combined a tile later), so
  // that no wavefront ever sits on a load it has just issued; coefficients are read once.
  const float kc0 = sd.kc0, kc1 = sd.kc1, kc2 = sd.kc2;
  const bool has_kb1 = sd.kb1 != nullptr, has_kb2 = sd.kb2 != nullptr;
  const float* kb0p = sd.kb0;
  const float* kb1p = has_kb1 ? sd.kb1 : sd.kb0;
  const float* kb2p = has_kb2 ? sd.kb2 : sd.kb0;
  struct RawBias {
    float b0, b1, b2;
  };
  auto load_raw_bias = [&](int j) {
    const int jj = max(0, min(j, j_end - 1));
    return RawBias{kb0p[jj], kb1p[jj], kb2p[jj]};
  };
  auto combine_bias = [&](const RawBias& r, int j) {
    float b = kc0 * r.b0 + (has_kb1 ? kc1 * r.b1 : 0.f);
    b += (has_kb2 ? kc2 * r.b2 : 0.f);
    b = (j < j_end) ? fmaxf(b, kNegBig) : kNegBig;
    return fmaxf(b * inv_lscale, -3.0e38f);
  };

  // ---- V^T operands (kMat): unit (32-key block, column block, step) = 128 pieces ----
  const u32x4* vt = reinterpret_cast<const u32x4*>(sd.vplanes);
  auto load_vt = [&](u32x4 (&a)[NCB][2][2], int kb) {
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const u32x4* p = vt + (((size_t)kb * NCB + cb) * 2 + s) * 128 + lane;
        a[cb][s][0] = p[0];
        a[cb][s][1] = p[64];
      }
  };

  f32x16 oacc[kHasO ? RB : 1][kHasO ? NCB : 1];
  // run_m: (kArgmax) the largest raw value so far, best_j its key; run_c: the constant of the
  // exponentials, kPtUp minus the running maximum in base-2 units
  float run_m[RB], run_c[RB], run_s[RB], run_o[RB];
  int best_j[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    best_j[rb] = 0;
    run_m[rb] = (MODE == kArgmax) ? -3.0e38f : 0.f;
    run_c[rb] = kPtUp;
    run_s[rb] = 0.f;
    run_o[rb] = 0.f;
    if constexpr (kHasO) {
#pragma unroll
      for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[rb][cb][r] = 0.f;
    }
  }

  // Where the running maxima start: 0 and the first tile's largest logit, or, when the caller
  // knew a key with a large logit for every row of this wavefront, the logits at those keys
  // (coarse_bias_kernel's seed blocks): a lower bound of the row's largest logit, from which
  // the skip below recognises tiles that cannot matter before the largest one has come by.
  bool seeded = false;
  if constexpr (MODE != kArgmax) {
    if (sd.seed != nullptr) {
      float sv[RB];
      bool ok = true;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        sv[rb] = sd.seed[min(row0 + rb * 32 + li, sd.nq - 1)];
        ok = ok && sv[rb] > -3.0e38f;
      }
      seeded = __builtin_amdgcn_ballot_w64(ok) == ~0ull;
      if (seeded) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) run_c[rb] = __builtin_fmaf(-sv[rb], lscale, kPtUp);
      }
    }
  }

  // ---- prologue: tiles 0 and 1 on their way, bias (and v) of tile 0 ----
  RawBias raw_next[NSUB];
#pragma unroll
  for (int js = 0; js < NSUB; ++js) raw_next[js] = load_raw_bias(j_begin + js * 32 + li);
  if constexpr (MODE == kVec) {
    if (tid < kPtKeys) lds_v[0][tid] = (j_begin + tid < j_end) ? sd.v[j_begin + tid] : 0.f;
  }
  if (ntiles > 0) {
    issue_tile(0);
    issue_tile(1);
    wait_newest_tile_only();
  }
  __syncthreads();

  auto swap_halves = [&](float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  };

  int buf = 0;
  for (int t = 0; t < ntiles; ++t) {
    const int j0 = j_begin + t * kPtKeys;
    const int nbuf = (buf == 2) ? 0 : buf + 1;
    const int n2buf = (nbuf == 2) ? 0 : nbuf + 1;
    float ab_cur[NSUB];
    // Key tile t + 2 first (its buffer was read during tile t - 1, which every wavefront has
    // left).  While global->LDS loads are in flight the compiler turns each of its own waits
    // for a register load into a wait for everything, so the tile load goes out as far ahead
    // of the first such wait (the V^T operands, after the first logits and soft-max) as it can.
    issue_tile(n2buf);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int js = 0; js < NSUB; ++js) {
      ab_cur[js] = combine_bias(raw_next[js], j0 + js * 32 + li);
      raw_next[js] = load_raw_bias(j0 + kPtKeys + js * 32 + li);
    }
    float v_next = 0.f;
    if constexpr (MODE == kVec) {
      if (tid < kPtKeys && j0 + kPtKeys + tid < j_end) v_next = sd.v[j0 + kPtKeys + tid];
    }
    const unsigned* tile = lds_k[buf];

#pragma unroll
    for (int js = 0; js < NSUB; ++js) {
      u32x4 va[kHasO ? NCB : 1][2][2];
      if constexpr (kHasO) load_vt(va, (j0 >> 5) + js);
      __builtin_amdgcn_sched_barrier(0);

      // A operands of the logits: key row js*32 + li, [plane][step]
      u32x4 kq[2][kStreamK ? 1 : KK16];
      if constexpr (!kStreamK) {
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int kk = 0; kk < KK16; ++kk)
            kq[p][kk] = lds_piece(tile, js * 32 + li, p * (DP / 8) + 2 * kk + h);
      }
      const float ab = h ? 1.0f : ab_cur[js];
      float vj[MODE == kVec ? 16 : 1];
      if constexpr (MODE == kVec) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const float4 v = *reinterpret_cast<const float4*>(&lds_v[buf][js * 32 + 8 * g + 4 * h]);
          vj[4 * g + 0] = v.x;
          vj[4 * g + 1] = v.y;
          vj[4 * g + 2] = v.z;
          vj[4 * g + 3] = v.w;
        }
      }

#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        f32x16 acc, tacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          acc[r] = 0.f;
          tacc[r] = 0.f;
        }
        // products lo*hi, hi*lo, hi*hi
        if constexpr (kStreamK) {
          // the key operands of step kk + 1 are requested while the MFMAs of step kk run, by
          // reads written out by hand: two steps' worth of registers instead of all of them
          // (which is what the compiler made of plain loads, spilling around the tile loop),
          // and no wait for the global->LDS loads in flight
          u32x4 ks[2][2];  // [step parity][plane]
          auto read_step = [&](int kk) {
            const unsigned* row = tile + (js * 32 + li) * ROWW;
            ks[kk & 1][0] = lds_read16(row + (((2 * kk + h) ^ swz(js * 32 + li)) << 2));
            ks[kk & 1][1] = lds_read16(row + ((((DP / 8) + 2 * kk + h) ^ swz(js * 32 + li)) << 2));
          };
          read_step(0);
#pragma unroll
          for (int kk = 0; kk < KK16; ++kk) {
            wait_lds();
            if (kk + 1 < KK16) read_step(kk + 1);
            const u32x4 k_hi = ks[kk & 1][0];
            const u32x4 k_lo = ks[kk & 1][1];
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, k_lo),
                                                         __builtin_bit_cast(f16x8, xq[rb][0][kk]),
                                                         acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, k_hi),
                                                         __builtin_bit_cast(f16x8, xq[rb][1][kk]),
                                                         acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, k_hi),
                                                         __builtin_bit_cast(f16x8, xq[rb][0][kk]),
                                                         acc, 0, 0, 0);
            if constexpr (MODE == kMat5) {  // second contraction on the same key operands
              tacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, k_lo), __builtin_bit_cast(f16x8, aq[rb][0][kk]), tacc,
                  0, 0, 0);
              tacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, k_hi), __builtin_bit_cast(f16x8, aq[rb][1][kk]), tacc,
                  0, 0, 0);
              tacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, k_hi), __builtin_bit_cast(f16x8, aq[rb][0][kk]), tacc,
                  0, 0, 0);
            }
          }
        } else {
#pragma unroll
          for (int prod = 0; prod < 3; ++prod) {
            const int pk = (prod == 0) ? 1 : 0, pq = (prod == 1) ? 1 : 0;
#pragma unroll
            for (int kk = 0; kk < KK16; ++kk)
              acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, kq[pk][kk]), __builtin_bit_cast(f16x8, xq[rb][pq][kk]),
                  acc, 0, 0, 0);
          }
        }
        if constexpr (MODE == kMat5 && !kStreamK) {
#pragma unroll
          for (int prod = 0; prod < 3; ++prod) {
            const int pk = (prod == 0) ? 1 : 0, pq = (prod == 1) ? 1 : 0;
#pragma unroll
            for (int kk = 0; kk < KK16; ++kk)
              tacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, kq[pk][kk]), __builtin_bit_cast(f16x8, aq[rb][pq][kk]),
                  tacc, 0, 0, 0);
          }
        }
        if constexpr (MODE == kArgmax) {
          // value = raw product + key bias; register r holds key 8 (r / 4) + 4 h + r % 4 of the
          // sub-tile, ascending in r, and tiles ascend: a strict test keeps the smallest key
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ab, h ? 0.0f : 1.0f, acc, 0, 0, 0);
          const int jb = j0 + js * 32 + 4 * h;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            if (acc[r] > run_m[rb]) {
              run_m[rb] = acc[r];
              best_j[rb] = jb + 8 * (r / 4) + (r % 4);
            }
          }
          continue;
        }
        // + key bias.  The logits stay in absolute raw units and the running maximum enters in
        // the exponent only (run_c): a maximum far below the unit's logits (a first
        // tile of keys without weight, a hint that names such a key) then costs no digits,
        // which its subtraction here would
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ab, h ? 0.0f : 1.0f, acc, 0, 0, 0);

        // ---- lazy lane-private soft-max (the two half-waves of a query share run_c) ----
        float tmax = fmaxf(acc[0], acc[1]);
#pragma unroll
        for (int r = 2; r < 16; ++r) tmax = fmaxf(tmax, acc[r]);
        const bool first = (t == 0 && js == 0 && !seeded);
        // the unit's largest exponent: kPtUp above its distance to the running maximum
        const float trel = __builtin_fmaf(tmax, lscale, run_c[rb]);
        // every logit of the unit 2^40 below the running maximum (itself never above the row's
        // largest logit): its exponentials could not change the fp32 sums
        if (!first && !wave_any(trel > skip_below + kPtUp)) continue;
        if (first || wave_any(trel > kPtLazyThresh + kPtUp)) {
          float a = tmax, b = tmax;
          swap_halves(a, b);
          const float tm = fmaxf(a, b);
          const bool up = first || __builtin_fmaf(tm, lscale, run_c[rb]) > kPtLazyThresh + kPtUp;
          const float c_new = up ? __builtin_fmaf(-tm, lscale, kPtUp) : run_c[rb];
          const float resc = first ? 0.f : fast_exp2(c_new - run_c[rb]);
          run_c[rb] = c_new;
          run_s[rb] *= resc;
          run_o[rb] *= resc;
          if constexpr (kHasO) {
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
              for (int r = 0; r < 16; ++r) oacc[rb][cb][r] *= resc;
          }
        }
        float p[16];
        float ps = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          p[r] = fast_exp2(__builtin_fmaf(acc[r], lscale, run_c[rb]));
          ps += p[r];
        }
        run_s[rb] += ps;
        if constexpr (MODE == kVec) {
          float po = 0.f;
#pragma unroll
          for (int r = 0; r < 16; ++r) po = __builtin_fmaf(p[r], vj[r], po);
          run_o[rb] += po;
        }
        if constexpr (MODE == kMat5) {
#pragma unroll
          for (int r = 0; r < 16; ++r) p[r] *= tacc[r] * t_unit;
        }
        if constexpr (kHasO) {
          // registers 8 s .. 8 s + 7 are this lane's B operand of 16-key step s
#pragma unroll
          for (int s = 0; s < 2; ++s) {
            unsigned hi[4], lo[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float x0 = p[8 * s + 2 * e], x1 = p[8 * s + 2 * e + 1];
              hi[e] = pack_f16(x0, x1);
              const f16x2 hh = __builtin_bit_cast(f16x2, hi[e]);
              lo[e] = pack_f16(x0 - (float)hh[0], x1 - (float)hh[1]);
            }
            const f16x8 bh = __builtin_bit_cast(f16x8, u32x4{hi[0], hi[1], hi[2], hi[3]});
            const f16x8 bl = __builtin_bit_cast(f16x8, u32x4{lo[0], lo[1], lo[2], lo[3]});
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
              oacc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, va[cb][s][1]), bh, oacc[rb][cb], 0, 0, 0);
              oacc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, va[cb][s][0]), bl, oacc[rb][cb], 0, 0, 0);
              oacc[rb][cb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                  __builtin_bit_cast(f16x8, va[cb][s][0]), bh, oacc[rb][cb], 0, 0, 0);
            }
          }
        }
      }
    }

    if constexpr (MODE == kVec) {
      if (tid < kPtKeys) lds_v[nbuf][tid] = v_next;
    }
    // tile t + 1 has landed (only the loads of tile t + 2 may still be in flight); after the
    // barrier it is visible and every wavefront is done reading tile t
    wait_newest_tile_only();
    __syncthreads();
    buf = nbuf;
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // tiles fetched past the chunk: let them land before exit

  // ---- merge the two half-waves of each query, then finish or spill ----
  float inv_vs = kHasO ? 1.0f / sd.vplane_scale[0] : 1.0f;
  if constexpr (MODE == kMat5) inv_vs /= t_unit * sd.q2plane_scale[0] * sd.kplane_scale[0];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = row0 + rb * 32 + li;
    const bool live = row < sd.nq;
    if constexpr (MODE == kArgmax) {
      float best = run_m[rb];
      int bj = best_j[rb];
      const float ob = xor32(best);
      const int oj = __shfl_xor(bj, 32, 64);
      if (ob > best || (ob == best && oj < bj)) {
        best = ob;
        bj = oj;
      }
      if (live && h == 0) {
        if (sd.splits == 1) {
          sd.ep.out[row] = -best * lscale;
          sd.ep.idx_out[row] = bj;
        } else {
          const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
          *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) =
              make_float2(ntiles > 0 ? best * lscale : -3.0e38f,
                          __builtin_bit_cast(float, ntiles > 0 ? bj : 0x7fffffff));
        }
      }
      continue;
    }
    const float M = (ntiles > 0) ? -run_c[rb] : kNegBig;
    const float s = run_s[rb] + xor32(run_s[rb]);
    const float o = run_o[rb] + xor32(run_o[rb]);
    if (sd.splits == 1) {
      if constexpr (!kHasO) {
        if (live && h == 0) epilogue_scalar(sd.ep, row, M, s, o);
      } else {
        if (live) {
#pragma unroll
          for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
              const int col = cb * 32 + 8 * q4 + 4 * h;
              const float4 O =
                  make_float4(oacc[rb][cb][4 * q4] * inv_vs, oacc[rb][cb][4 * q4 + 1] * inv_vs,
                              oacc[rb][cb][4 * q4 + 2] * inv_vs, oacc[rb][cb][4 * q4 + 3] * inv_vs);
              epilogue_vec4(sd.ep, sd.q, d, vec_ok, row, col, M, s, O);
            }
        }
      }
    } else if (live) {
      const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
      if (h == 0) {
        *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(M, s);
        if constexpr (MODE == kVec) sd.part_o[pr] = o;
      }
      if constexpr (kHasO) {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            const int col = cb * 32 + 8 * q4 + 4 * h;
            if (DP % 32 == 0 || col < DP) {
              *reinterpret_cast<float4*>(&sd.part_o[pr * DP + col]) =
                  make_float4(oacc[rb][cb][4 * q4] * inv_vs, oacc[rb][cb][4 * q4 + 1] * inv_vs,
                              oacc[rb][cb][4 * q4 + 2] * inv_vs, oacc[rb][cb][4 * q4 + 3] * inv_vs);
            }
          }
      }
    }
  }
}

}  // namespace fs
