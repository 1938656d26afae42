// Log-sum-exp kernel with the coarse tile test for rows of 65 .. 128 columns (fp16 planes).
//
// The test is the one of lse_coarse_kernel (fs_lsecoarse.hpp): the hi*hi plane product of a
// 32 x 32 logits tile, plus the exact key bias and a per-row bound on the two cross products,
// shows whether any logit of the tile lies within 2^40 of its row's running maximum; a tile
// where none does ends there, after a third of its MFMAs and without a single exponential.
// Rows start from their logit at the key that held their maximum in the launch before
// (Side::seed, computed by coarse_bias_kernel's seed blocks from Side::best_key), so on a
// peaked plan nearly every tile ends.
//
// A wavefront keeps both planes of its 64 query rows (two blocks of 32: 128 registers) and
// walks its key chunk in tiles of 64 keys whose two planes sit in LDS (32 KiB, two buffers, the
// next tile in flight; two workgroups per CU).  Per 32-key sub-tile the hi*hi products of both
// row blocks are taken first (the key operands serve both), then each block's unit is tested;
// a unit (32 keys x 32 rows) that goes on reads the keys' lo plane from LDS, adds the two cross
// products and runs the online soft-max: nothing such a block computes outlives it except the
// rows' running (maximum, sum) and the key of the maximum, and nothing in it waits for memory
// (with the lo planes fetched from global memory on demand, the tenth of the units that goes on
// at 20,000 x 30,000 x 128, eps 0.0025, cost more than all the tests).  There is no software
// pipeline across units.  Carried margins and the sparse form of the 64-column kernel do not
// exist here; the unit counters for the variant choice on the device do.
//
// Everything LDS-related is written out by hand (ds_read / ds_write / s_waitcnt / s_barrier):
// key tiles arrive by direct global->LDS loads two tiles ahead, and the compiler, which cannot
// tell a read of one ring buffer from the loads still filling another, would make every LDS
// access wait for all of them.
#pragma once

#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

template <int T>
__global__ __launch_bounds__(256, 2) void lse_coarse128_kernel(const LaunchArgs args) {
  constexpr int DP = 128, RB = 2, JT = 64, NSUB = JT / 32, KK16 = DP / 16;
  constexpr int ROWW = DP;        // 32-bit words per two-plane row in global memory
  constexpr int ROWH = DP / 2;    // words per hi-plane row in LDS
  constexpr int PPRH = ROWH / 4;  // 16-byte pieces per hi-plane row
  constexpr int PER_PLANE = JT * PPRH / 256;  // direct loads per lane and plane of a tile
  static_assert(PPRH == 16 && PER_PLANE == 4, "64 keys x 16 pieces: four direct loads per lane and plane");

  __shared__ __attribute__((aligned(16))) unsigned lds_k[2][2][JT * ROWH];  // [buffer][plane]
  __shared__ __attribute__((aligned(16))) float lds_b[2][3][JT];            // the key bias terms as given

  // variant chosen on the device: the launch of the variant that was not chosen ends here
  if (args.sel_pred && args.sel[kSelWord] != args.sel_want) return;

  int bid = blockIdx.x;
  const bool second = bid >= args.blocks0;
  if (second) bid -= args.blocks0;
  const Side& sd = second ? args.side[1] : args.side[0];
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
  const int ntiles = (j_end > j_begin) ? (j_end - j_begin + JT - 1) / JT : 0;

  // MFMAs produce raw products of the scaled planes; lscale turns them into base-2 logits
  const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = 1.0f / lscale;

  // ---- stationary planes of the query rows: [block][16-column step] ----
  u32x4 xh[RB][KK16], xl[RB][KK16];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = min(row0 + rb * 32 + li, sd.nq - 1);
    const unsigned* qrow = sd.qplanes + (size_t)row * (size_t)ROWW;
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) {
      xh[rb][kk] = *reinterpret_cast<const u32x4*>(qrow + 8 * kk + 4 * h);
      xl[rb][kk] = *reinterpret_cast<const u32x4*>(qrow + ROWH + 8 * kk + 4 * h);
    }
  }
  // Bound on the two cross products of a row, in raw units (see lse_coarse_kernel): with X, Y
  // the scaled matrices (|.| < 2^15), |Y_lo| <= 8 and |X_lo| <= 2^-11 |X_hi| (+ 2^-24), hence
  //   sum_k |Y_lo X_hi| + |Y_hi X_lo| <= 24 (1 + 2^-10) sum_k |X_hi| + DP 2^-9;
  // one base-2 unit of slack covers the fp32 roundings of the chain.
  float corr[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float l1 = 0.f;
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) {
      const f16x8 hv = __builtin_bit_cast(f16x8, xh[rb][kk]);
#pragma unroll
      for (int e = 0; e < 8; ++e) l1 += fabsf((float)hv[e]);
    }
    l1 += xor32(l1);
    corr[rb] = 24.5f * l1 + (float)DP * 0x1p-9f + inv_lscale;
  }

  // ---- LDS access by hand ----
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

  // ---- key tiles: lane idx of instruction c fills LDS slot idx of a plane's buffer and fetches
  // the piece that belongs there (slot = piece ^ (row & 15)); the plane buffers end in zero
  // rows, so tiles past the chunk are fetched like any other and masked by their bias ----
  // (the four rounds of a plane are 16 rows apart and share the slot permutation)
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
  // ---- key bias: wavefront 0 brings the (up to three) terms of the tile's 64 keys into LDS as
  // they are, by direct loads issued ahead of the tile's keys (the same wait covers both);
  // absent terms re-read the first vector and are dropped when the terms are combined ----
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
  auto swap_halves = [&](float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  };
  auto max16 = [](const f32x16& a) {
    float m = fmaxf(a[0], a[1]);
#pragma unroll
    for (int r = 2; r < 16; ++r) m = fmaxf(m, a[r]);
    return m;
  };

  // ---- running statistics.  The logits stay in absolute raw units (of the full logit with
  // its key bias); the running maximum M is kept as run_c = -M * lscale, rounded once: the
  // constant of the exponentials and what the test compares with (subtracted inside the
  // accumulator, M would cost the logits their digits whenever it lies far below them) ----
  float run_c[RB], run_s[RB], best_v[RB];
  int best_j[RB];
  const bool track = sd.best_key != nullptr;
  bool seeded = sd.seed != nullptr;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    run_c[rb] = 0.f;
    run_s[rb] = 0.f;
    best_v[rb] = -3.0e38f;
    best_j[rb] = -1;
    if (sd.seed != nullptr) {
      const float sv = sd.seed[min(row0 + rb * 32 + li, sd.nq - 1)];
      seeded = seeded && sv > -3.0e38f;
      run_c[rb] = -sv * lscale;
    }
  }
  // (wavefront-uniform: without a starting value for every row the first unit sets the maxima)
  seeded = __builtin_amdgcn_ballot_w64(seeded) == ~0ull;
  bool started[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    started[rb] = seeded;
    if (!seeded) run_c[rb] = 0.f;
  }
  unsigned n_ended = 0;

  // ---- prologue: tile 0 and its bias terms ----
  if (ntiles > 0) {
    issue_bias(j_begin, 0);
    issue_tile(0);
    fence();
    __builtin_amdgcn_s_waitcnt(0x0070);  // everything has landed
    fence();
  }
  barrier();

  int buf = 0;
  for (int t = 0; t < ntiles; ++t) {
    const int j0 = j_begin + t * JT;
    const int nbuf = buf ^ 1;
    // the other buffer was read during tile t - 1, which every wavefront has left
    issue_bias(j0 + JT, nbuf);
    issue_tile(nbuf);
    fence();

#pragma unroll
    for (int js = 0; js < NSUB; ++js) {
      const unsigned* yrow = lds_k[buf][0] + (js * 32 + li) * ROWH;
      float kb0r = ds_read4(&lds_b[buf][0][js * 32 + li]);
      float kb1r = ds_read4(&lds_b[buf][1][js * 32 + li]);
      float kb2r = ds_read4(&lds_b[buf][2][js * 32 + li]);
      // hi*hi of both row blocks, the key operands one step ahead of their MFMAs
      u32x4 ks[2];
      ks[0] = ds_read16(yrow + (((0 + h) ^ (li & 15)) << 2));
      f32x16 acc[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[rb][r] = 0.f;
#pragma unroll
      for (int kk = 0; kk < KK16; ++kk) {
        wait_lds();
        if (kk + 1 < KK16) ks[(kk + 1) & 1] = ds_read16(yrow + (((2 * (kk + 1) + h) ^ (li & 15)) << 2));
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[rb] = mfma16(ks[kk & 1], xh[rb][kk], acc[rb]);
      }
      fence();
      asm volatile("" : "+v"(kb0r), "+v"(kb1r), "+v"(kb2r));  // (read before the first wait above)
      float kbias = kc0 * kb0r + (has_kb1 ? kc1 * kb1r : 0.f);
      kbias += (has_kb2 ? kc2 * kb2r : 0.f);
      kbias = (j0 + js * 32 + li < j_end) ? fmaxf(kbias, kNegBig) : kNegBig;  // keys past the chunk are masked
      kbias = fmaxf(kbias * inv_lscale, -3.0e38f);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        // + key bias: A = [bias_j, 1], B = [1, 0]
        acc[rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(h ? 1.0f : kbias, h ? 0.0f : 1.0f,
                                                       acc[rb], 0, 0, 0);
        const float tmax = max16(acc[rb]);
        // every logit of the unit at least 2^40 below its row's running maximum, whatever the
        // cross products add: nothing of it could change the fp32 sums
        if (started[rb] && !wave_any(__builtin_fmaf(tmax + corr[rb], lscale, run_c[rb]) > args.skip_log2)) {
          ++n_ended;
          continue;
        }
        // ---- the unit goes on: cross products on the lo planes, then the online soft-max ----
        {
          // (both planes of the keys again from LDS, two steps at a time: the registers of the
          // first pass are free by now.  The cross products are summed on their own, where they
          // are small, and join the logits with one addition: added one by one to logits of a
          // few thousand base-2 units they would each be rounded to those logits' last place.)
          const unsigned* ylo = lds_k[buf][1] + (js * 32 + li) * ROWH;
          f32x16 cr;
#pragma unroll
          for (int r = 0; r < 16; ++r) cr[r] = 0.f;
#pragma unroll
          for (int part = 0; part < KK16 / 2; ++part) {
            u32x4 kh[2], kl[2];
#pragma unroll
            for (int k2 = 0; k2 < 2; ++k2) {
              const int kk = part * 2 + k2;
              kh[k2] = ds_read16(yrow + (((2 * kk + h) ^ (li & 15)) << 2));
              kl[k2] = ds_read16(ylo + (((2 * kk + h) ^ (li & 15)) << 2));
            }
            wait_lds();
#pragma unroll
            for (int k2 = 0; k2 < 2; ++k2) {
              const int kk = part * 2 + k2;
              cr = mfma16(kh[k2], xl[rb][kk], cr);
              cr = mfma16(kl[k2], xh[rb][kk], cr);
            }
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[rb][r] += cr[r];
          const float lane_max = max16(acc[rb]);
          float tm = lane_max;
          {
            float a = tm, b = tm;
            swap_halves(a, b);
            tm = fmaxf(a, b);  // the row's largest logit of the unit
          }
          // the key of the row's largest logit so far (absolute raw units; lane-private, the two
          // half-waves are merged at the end)
          // (searched only when some lane's largest value of the unit beats what it has)
          if (track && wave_any(lane_max > best_v[rb])) {
            const int jb = j0 + js * 32 + 4 * h;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float v = acc[rb][r];
              if (v > best_v[rb]) {
                best_v[rb] = v;
                best_j[rb] = jb + 8 * (r / 4) + (r % 4);
              }
            }
          }
          const bool first = !started[rb];
          float cc = -tm * lscale;
          asm volatile("" : "+v"(cc));  // the exponents, the rescale and the result see one number
          cc = first ? cc : fminf(cc, run_c[rb]);
          float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            ps0 += fast_exp2(__builtin_fmaf(acc[rb][r], lscale, cc));
            ps1 += fast_exp2(__builtin_fmaf(acc[rb][r + 1], lscale, cc));
          }
          const float resc = first ? 0.f : fast_exp2(cc - run_c[rb]);
          run_s[rb] = run_s[rb] * resc + (ps0 + ps1);
          run_c[rb] = cc;
          started[rb] = true;
        }
      }
    }

    // tile t + 1 has landed (and with it the bias terms requested ahead of it); after the barrier
    // both are visible and every wavefront is done reading tile t
    fence();
    __builtin_amdgcn_s_waitcnt(0x0070);
    fence();
    barrier();
    buf = nbuf;
  }
  fence();
  __builtin_amdgcn_s_waitcnt(0x0070);  // what was fetched past the chunk: let it land before the end

  // unit counts of this wavefront for the variant choice on the device
  if (args.sel != nullptr && lane == 0 && ntiles > 0) {
    const int slot = blockIdx.x % kSelSlots;
    atomicAdd(&args.sel[kSelEnded + slot], n_ended);
    atomicAdd(&args.sel[kSelUnits + slot], (unsigned)(ntiles * NSUB * RB));
  }

#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = row0 + rb * 32 + li;
    const float s = run_s[rb] + xor32(run_s[rb]);
    const float M2 = -run_c[rb];
    float bv = best_v[rb];
    int bj = best_j[rb];
    const float ov = xor32(bv);
    const int oj = __shfl_xor(bj, 32, 64);
    if (ov > bv || (ov == bv && oj >= 0 && (bj < 0 || oj < bj))) bj = oj;
    if (row < sd.nq && h == 0) {
      if (sd.splits == 1) {
        epilogue_scalar(sd.ep, row, M2, s, 0.f);
        if (track && bj >= 0) sd.best_key[row] = bj;
      } else {
        const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
        *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(M2, s);
        if (sd.part_best != nullptr) sd.part_best[pr] = bj;
      }
    }
  }
}

}  // namespace fs
