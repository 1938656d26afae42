// Software-pipelined log-sum-exp kernel (d <= 128).
//
// Same decomposition as stream_kernel<kLse> (stationary query blocks in VGPRs,
// key tiles through LDS, transposed logits, lane-private online soft-max), with these changes
// that matter for speed:
//   * the soft-max of logits tile u-1 is cut into pieces that sit in program order BETWEEN
//     the MFMAs of tile u, fenced with sched_barrier so the compiler keeps them there.  A
//     wavefront issues in order and a chain of dependent MFMAs blocks its issue slot, so
//     only VALU work interleaved this way runs in the MFMA shadow;
//   * the online soft-max is branch free per lane (per-lane max, rescale by exp2(-delta) every
//     tile).  With the keys split into chunks every chunk is short, new running
//     maxima are frequent, and a wave-wide "does any lane need a rescale" branch
//     would be taken on almost every tile.  Only the first tile of a block is handled apart.
//     The one wave-uniform decision is whether a tile's exponentials can matter at all
//     (LaunchArgs::skip_log2); if not, the tile runs its MFMAs only;
//   * the A operands of the next 32-key sub-tile are read from LDS while the current one is
//     multiplied, and key tiles are fetched two tiles ahead (direct global->LDS loads in the
//     two-plane modes, through registers otherwise), with one barrier per 64 keys;
//   * key bias and running max.  Two-plane modes at d <= 64: the MFMA chain of a tile starts
//     from the key bias (16 floats per lane, read from LDS into the registers the previous
//     tile's soft-max has just let go of; two accumulator tiles swap roles from tile to tile
//     and nothing is copied), and the running max enters through the addend of the exp2
//     argument's FMA.  Other modes: one extra fp32 MFMA per tile adds bias - max.
//
// Operand precision (PREC):
//   kF32   v_mfma_f32_32x32x2_f32 on fp32 operands (needs d % 4 == 0 and aligned rows).
//          (The plane mode reads operands that the split kernel has already cut into
//          packed planes and applies the logit scale in the exp2 argument's FMA, so there is no
//          per-tile conversion work.)
//   kH3    two fp16 planes (hi, lo) of the operand times a power of two that brings the
//          matrix's largest magnitude to [2^14, 2^15); hi*hi + hi*lo + lo*hi on
//          v_mfma_f32_32x32x16_f16.  The planes carry 22 significand bits and the dropped
//          lo*lo term weighs 2^-22, so a dot product is as accurate as one accumulated in
//          fp32 from exact products, at 3/16 of the fp32 MFMA time.
#pragma once

#include <type_traits>

#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

enum Prec : int { kF32 = 0, kH3 = 3 };

constexpr int kPlanePadRows = 512;  // zero rows after the last row of a plane buffer
constexpr int kAbsmaxBlocks = 256;  // partial maxima per matrix written by absmax_kernel


// Largest |value| of two matrices: blocks [0, kAbsmaxBlocks) scan a, the rest scan b; one
// partial maximum per block goes to partial[2][kAbsmaxBlocks].
__global__ __launch_bounds__(256) void absmax_kernel(const float* __restrict__ a, long long na,
                                                     const float* __restrict__ b, long long nb,
                                                     float* __restrict__ partial) {
  __shared__ float red[4];
  const bool second = blockIdx.x >= kAbsmaxBlocks;
  const float* src = second ? b : a;
  const long long cnt = second ? nb : na;
  const int blk = second ? blockIdx.x - kAbsmaxBlocks : blockIdx.x;
  float m = 0.f;
  if ((reinterpret_cast<size_t>(src) & 15) == 0) {
    // four float4 loads in flight per thread; the tail below takes what does not fill one
    const long long n4 = cnt >> 2;
    const float4* s4 = reinterpret_cast<const float4*>(src);
    const long long stride = 256LL * kAbsmaxBlocks;
    long long i = (long long)blk * 256 + threadIdx.x;
    for (; i + 3 * stride < n4; i += 4 * stride) {
      const float4 a0 = s4[i], a1 = s4[i + stride], a2 = s4[i + 2 * stride], a3 = s4[i + 3 * stride];
      m = fmaxf(m, fmaxf(fmaxf(fabsf(a0.x), fabsf(a0.y)), fmaxf(fabsf(a0.z), fabsf(a0.w))));
      m = fmaxf(m, fmaxf(fmaxf(fabsf(a1.x), fabsf(a1.y)), fmaxf(fabsf(a1.z), fabsf(a1.w))));
      m = fmaxf(m, fmaxf(fmaxf(fabsf(a2.x), fabsf(a2.y)), fmaxf(fabsf(a2.z), fabsf(a2.w))));
      m = fmaxf(m, fmaxf(fmaxf(fabsf(a3.x), fabsf(a3.y)), fmaxf(fabsf(a3.z), fabsf(a3.w))));
    }
    for (; i < n4; i += stride) {
      const float4 a0 = s4[i];
      m = fmaxf(m, fmaxf(fmaxf(fabsf(a0.x), fabsf(a0.y)), fmaxf(fabsf(a0.z), fabsf(a0.w))));
    }
    for (long long t = (n4 << 2) + (long long)blk * 256 + threadIdx.x; t < cnt; t += stride)
      m = fmaxf(m, fabsf(src[t]));
  } else {
    for (long long i = (long long)blk * 256 + threadIdx.x; i < cnt; i += 256LL * kAbsmaxBlocks)
      m = fmaxf(m, fabsf(src[i]));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0)
    partial[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// x[rows, d] (fp32) -> two packed fp16 planes [rows + kPlanePadRows][2][DP/2] of scale*x, zero
// padded to DP columns and in the trailing rows.  scale is derived from the partial maxima of
// absmax_kernel; block 0 also publishes it in *scale_out for the consuming kernel and clears
// the kSelWords words at `clear_state` (the variant-choice state that belongs to the planes);
// `best_keys` (may be null) starts three arrays of one value per row, (rows + 3) & ~3 values apart:
// the keys (reset to -1), the rows' last maxima (3e38) and the rows' last biases as keys (0).
// With `chunked` the two planes are interleaved per 32 columns (layout of lse_gemm_kernel).
// `tiled` (may be null; not with `chunked`): a second copy in MFMA operand order, see Side::ktiled.
__global__ __launch_bounds__(256) void fill_zero_kernel(unsigned* __restrict__ p, long long n) {
  const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i + 3 < n) {
    *reinterpret_cast<uint4*>(p + i) = make_uint4(0u, 0u, 0u, 0u);
  } else {
    for (long long k = i; k < n; ++k) p[k] = 0u;
  }
}

__global__ __launch_bounds__(256) void split_planes_f16_kernel(
    const float* __restrict__ src, unsigned* __restrict__ dst, int rows, int d, int dp,
    const float* __restrict__ partial_max, float* __restrict__ scale_out,
    float* __restrict__ scale_out2, int chunked, unsigned* __restrict__ clear_state,
    int* __restrict__ best_keys, unsigned* __restrict__ tiled, int start_plain) {
  __shared__ float red[4];
  float m = partial_max[threadIdx.x];  // kAbsmaxBlocks == blockDim.x
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  const float sc = f16_plane_scale(fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *scale_out = sc;
    if (scale_out2) *scale_out2 = sc;  // the same matrix plays both roles
  }
  // (start_plain: the variant choice begins with the plain kernel, see FS_FLAG_START_PLAIN)
  if (blockIdx.x == 0 && clear_state != nullptr) {
    if (threadIdx.x < kSelWords)
      clear_state[threadIdx.x] = (threadIdx.x == kSelWord && start_plain) ? 1u : 0u;
    if (threadIdx.x + 256 < kSelWords) clear_state[threadIdx.x + 256] = 0u;
  }

  const int per_row = dp / 4;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (best_keys != nullptr && idx < rows) {  // new planes: the three per-row arrays behind them
    const int stride = (rows + 3) & ~3;
    best_keys[idx] = -1;                                                  // no key known yet
    reinterpret_cast<float*>(best_keys)[stride + idx] = 3.0e38f;          // no maximum known yet
    reinterpret_cast<float*>(best_keys)[2 * stride + idx] = 0.f;          // no bias seen yet
  }
  if (idx >= (long long)(rows + kPlanePadRows) * per_row) return;
  const int r = (int)(idx / per_row);
  const int c4 = (int)(idx % per_row) * 4;
  const float* p = src + (size_t)min(r, rows - 1) * (size_t)d;
  float v[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) v[t] = (c4 + t < d && r < rows) ? p[c4 + t] * sc : 0.f;
  const unsigned h01 = pack_f16(v[0], v[1]), h23 = pack_f16(v[2], v[3]);
  const f16x2 a = __builtin_bit_cast(f16x2, h01), b = __builtin_bit_cast(f16x2, h23);
  const unsigned l01 = pack_f16(v[0] - (float)a[0], v[1] - (float)a[1]);
  const unsigned l23 = pack_f16(v[2] - (float)b[0], v[3] - (float)b[1]);
  unsigned* o = dst + (size_t)r * (size_t)dp;  // two planes of dp/2 words
  if (chunked) {
    // per 32 columns: 16 words of the hi plane, then 16 words of the lo plane (dp % 32 == 0)
    unsigned* oc = o + (c4 / 32) * 32 + (c4 % 32) / 2;
    *reinterpret_cast<uint2*>(oc) = make_uint2(h01, h23);
    *reinterpret_cast<uint2*>(oc + 16) = make_uint2(l01, l23);
  } else {
    *reinterpret_cast<uint2*>(o + c4 / 2) = make_uint2(h01, h23);
    *reinterpret_cast<uint2*>(o + dp / 2 + c4 / 2) = make_uint2(l01, l23);
    if (tiled != nullptr) {
      // the same words in MFMA operand order: per 32 rows [plane][16-column step][half h][row % 32]
      // 16 bytes; word w of a plane row belongs to step w / 8, half (w / 4) % 2
      const int w = c4 / 2, kk16 = dp / 16;
      unsigned* t = tiled + ((size_t)(r / 32) * 2 * kk16 + w / 8) * 256 + (((w >> 2) & 1) * 32 + r % 32) * 4 + (w & 3);
      *reinterpret_cast<uint2*>(t) = make_uint2(h01, h23);
      *reinterpret_cast<uint2*>(t + (size_t)kk16 * 256) = make_uint2(l01, l23);
    }
  }
}

template <int DP, int PREC>
struct Geo2 {
  static constexpr int NP = (PREC == kF32) ? 1 : 2;
  // keys per tile: 64, except 128-column fp32 rows (LDS)
  static constexpr int JT = (DP >= 128 && PREC == kF32) ? 32 : 64;
  static constexpr int NSUB = JT / 32;
  // LDS row stride in 32-bit words: fp32 row + 4, or NP 16-bit planes + 4
  static constexpr int LDW = (PREC == kF32) ? (DP + 4) : (NP * DP / 2 + 4);
  static constexpr int KK16 = DP / 16;  // 16-bit MFMAs per plane pair
  // MFMAs of one logits tile, the bias one excluded
  static constexpr int NMAIN = (PREC == kF32) ? DP / 2 : 3 * KK16;
};

#define FS_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// Soft-max of one logits tile cut into kPieces program-order pieces, so that the caller can
// place a piece after every few MFMAs of the NEXT tile: a wavefront issues in order, and only
// VALU work that sits between the MFMAs in program order runs in their shadow.
constexpr int kPieces = 12;
constexpr int kMaxPieces = 3;  // pieces 0..2 find the largest logit of the unit
constexpr int kBiasPiece = 4;  // pieces 4..7 read the next unit's bias from LDS, 16 bytes each
struct SoftmaxStage {
  float m[6], mx, aa, bb, c, cx, ps0, ps1, po;  // c: exponent of the rescale, cx: offset of the logits
  float t[16], e[16];
  float v[2][4];  // VEC: two groups of four v values in flight
};

// VEC: the plan-vector product (kVec) on the same pipeline: next to the row sums the kernel
// keeps o_i = sum_j p_ij v_j, with v staged through LDS beside the key bias.  Two-plane modes
// at d <= 64 only (the bias-as-accumulator-start variants).
template <int DP, int RB, int PREC, bool VEC = false>
__global__ __launch_bounds__(256, 2) void lse2_kernel(const LaunchArgs args) {
  using G = Geo2<DP, PREC>;
  constexpr int NP = G::NP;
  constexpr int NSUB = G::NSUB;
  constexpr int NMAIN = G::NMAIN;
  constexpr bool kPlanes = (PREC != kF32);
  constexpr int ROWW = kPlanes ? NP * DP / 2 : DP;  // 32-bit words per operand row in global memory
  // Key-register prefetch (A operands of the next 32-key sub-tile are read from LDS while the
  // current one is multiplied) and the early LDS store it needs; off where registers are short.
  constexpr bool KPF = (NSUB == 2) && DP < 128;
  // Two-plane modes with the key-register prefetch: the key bias is the initial value of the MFMA
  // chain's accumulator (16 floats per lane read from LDS while the previous unit finishes)
  // and the running max is subtracted inside the exp2 argument's FMA, which takes the fp32
  // bias MFMA (64 of 448 MFMA cycles per unit at d = 64) out of the loop.
  constexpr bool BIASC = (PREC == kH3) && KPF;
  static_assert(!VEC || BIASC, "the vector mode rides on the bias-as-accumulator-start pipeline");
  // Two-plane modes bring key tiles into LDS with direct global->LDS loads (no staging
  // registers, no ds_write): rows are unpadded and 16-byte piece p of row r sits in slot
  // p ^ swz(r), which keeps the b128 reads of 16 consecutive rows conflict free.  With the
  // key-register prefetch the tile two ahead is in flight, hence three buffers.
  constexpr bool DIRECT = kPlanes;
  constexpr int NBUF = (DIRECT && KPF) ? 3 : 2;
  constexpr int LDWK = DIRECT ? ROWW : G::LDW;  // LDS row stride in words
  constexpr int PPR = ROWW / 4;                 // 16-byte pieces per row

  __shared__ __attribute__((aligned(16))) unsigned lds_k[NBUF][G::JT * LDWK];
  __shared__ __attribute__((aligned(16))) float lds_b[NBUF][256];  // [buf][thread]; first JT used
  __shared__ __attribute__((aligned(16))) float lds_v[VEC ? NBUF : 1][VEC ? 256 : 4];  // VEC: v_j

  // variant chosen on the device: the launch of the variant that was not chosen ends here
  if (args.sel_pred && args.sel[kSelWord] != args.sel_want) return;
  // a step with a one-sweep launch: this kernel runs when that one did not, or failed
  if (args.sweep && args.sel[kSelSweep] != 0u && args.sel[kSelSweepFail] == 0u) return;
  if (args.sweep && blockIdx.x == 0 && threadIdx.x == 0) args.sel[kSelRan] = 1u;

  int bid = blockIdx.x;
  const bool second = bid >= args.blocks0;
  if (second) bid -= args.blocks0;
  const Side& sd = second ? args.side[1] : args.side[0];
  // the merge kernel reads the partial results of a launch with carried margins by the kernel
  // that wrote them: here, one per key chunk
  if (sd.margins != nullptr && bid == 0 && threadIdx.x == 0) args.sel[kSelForm + sd.ps_q] = 0u;
  const int d = args.d;

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
  const int ntiles = (j_end - j_begin + G::JT - 1) / G::JT;

  // fp32 mode: logits come out of the MFMAs already in base-2 units (queries pre-scaled).
  // 16-bit plane modes: MFMAs produce raw dot products; lscale turns them into base-2 logits
  // inside the exp2 argument, and the bias / running max are kept in dot-product units.
  // fp16 planes carry a power-of-two scale per matrix, which lscale takes out again.
  float lscale = kPlanes ? sd.qscale : 1.0f;
  if constexpr (PREC == kH3) lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = kPlanes ? 1.0f / lscale : 1.0f;
  const float skip_below = args.skip_log2 * inv_lscale;  // in accumulator units
  unsigned n_left_out = 0;  // units whose exponentials were not computed

  // ---- stationary query operands ----
  float xs[kPlanes ? 1 : RB][kPlanes ? 1 : DP / 2];
  u32x4 xq[kPlanes ? RB : 1][kPlanes ? NP : 1][kPlanes ? G::KK16 : 1];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = min(row0 + rb * 32 + li, sd.nq - 1);
    if constexpr (!kPlanes) {
      const float* qrow = sd.q + (size_t)row * (size_t)d;
#pragma unroll
      for (int q = 0; q < DP / 8; ++q) {
        const int col = 8 * q + 4 * h;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (col < d) v = *reinterpret_cast<const float4*>(qrow + col);
        xs[rb][4 * q + 0] = v.x * sd.qscale;
        xs[rb][4 * q + 1] = v.y * sd.qscale;
        xs[rb][4 * q + 2] = v.z * sd.qscale;
        xs[rb][4 * q + 3] = v.w * sd.qscale;
      }
    } else {
      const unsigned* qrow = sd.qplanes + (size_t)row * (size_t)ROWW;
#pragma unroll
      for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int kk = 0; kk < G::KK16; ++kk)
          xq[rb][p][kk] = *reinterpret_cast<const u32x4*>(qrow + p * (DP / 2) + 8 * kk + 4 * h);
    }
  }

  // The logits stay in absolute accumulator units in every configuration (a running maximum
  // subtracted inside the accumulator costs the logits their digits whenever it lies far below
  // them: after a first tile of keys without weight, say).  run_m: the running maximum in those
  // units; run_c: -run_m * lscale as rounded once, the offset every exponent of the row uses, so
  // that rescaling by differences of run_c is consistent with the exponents already summed
  float run_m[RB], run_s[RB], run_c[RB], run_o[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    run_m[rb] = 0.f;
    run_s[rb] = 0.f;
    run_c[rb] = 0.f;
    run_o[rb] = 0.f;
  }

  // ---- staging (global -> registers -> LDS), branch free: rows are clamped, masked by bias ----
  constexpr int C16_PER_ROW = ROWW / 4;  // 16-byte chunks per operand row
  constexpr int C16_TOTAL = G::JT * C16_PER_ROW;
  constexpr int PER_THREAD = (C16_TOTAL + 255) / 256;
  u32x4 st_k[DIRECT ? 1 : PER_THREAD];
  float st_b0 = 0.f, st_b1 = 0.f, st_b2 = 0.f, st_pen = 0.f, st_v = 0.f;
  const unsigned* krows = kPlanes ? sd.kplanes : reinterpret_cast<const unsigned*>(sd.k);
  const int krow_words = kPlanes ? ROWW : d;
  const float* kb1p = sd.kb1 ? sd.kb1 : sd.kb0;  // always loadable; unused terms are dropped
  const float* kb2p = sd.kb2 ? sd.kb2 : sd.kb0;
  // read once: inside the loop the launch arguments would be fetched again for every tile
  const float kc0 = sd.kc0, kc1 = sd.kc1, kc2 = sd.kc2;
  const bool has_kb1 = sd.kb1 != nullptr, has_kb2 = sd.kb2 != nullptr;
  // Plane buffers end with kPlanePadRows zero rows, so the 16-bit modes walk them with plain
  // running pointers (tiles up to two past the chunk are fetched and masked by the bias);
  // the fp32 mode reads the caller's matrix and clamps the row instead.
  auto swz = [&](int r) {  // slot permutation of LDS row r (direct mode)
    return PPR >= 16 ? (r & 15) : (PPR == 8 ? ((r >> 1) & 7) : ((r >> 2) & 3));
  };
  const unsigned* kp[PER_THREAD];
#pragma unroll
  for (int c = 0; c < PER_THREAD; ++c) {
    const int idx = tid + 256 * c;
    const int r = idx / C16_PER_ROW;
    int piece = idx % C16_PER_ROW;
    if constexpr (DIRECT) piece ^= swz(r);  // lane idx fills LDS slot idx; it fetches this piece
    kp[c] = krows + (size_t)(j_begin + r) * (size_t)krow_words + piece * 4;
  }
  // The staging code is branch free (clamped rows, additive masks): the only branches of the
  // main loop are the wave-uniform ones around soft-max pieces.
  auto stage_load = [&](int j0, int dbuf) {  // dbuf: LDS buffer of the direct loads
    {  // raw key-bias terms of row j0 + tid; combined at store time so that nothing here
       // waits for the loads (threads beyond the tile fetch a clamped, unused row).  Issued
       // before the tile itself: loads complete in order, and whoever waits for these three
       // values should not have to wait for the tile as well
      const int j = max(0, min(j0 + tid, j_end - 1));
      st_b0 = sd.kb0[j];
      st_b1 = kb1p[j];
      st_b2 = kb2p[j];
      st_pen = (j0 + tid < j_end) ? 0.f : 2.0f * kNegBig;
      if constexpr (VEC) st_v = sd.v[j];  // masked keys carry probability zero
    }
#pragma unroll
    for (int c = 0; c < PER_THREAD; ++c) {
      if constexpr (DIRECT) {
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)kp[c],
            (__attribute__((address_space(3))) void*)(&lds_k[dbuf][(c * 256 + wave * 64) * 4]),
            16, 0, 0);
        kp[c] += G::JT * ROWW;
      } else {
        const int idx = tid + 256 * c;
        const int r = idx / C16_PER_ROW;
        const int c4 = (idx % C16_PER_ROW) * 4;
        const int j = max(0, min(j0 + r, j_end - 1));
        u32x4 v = *reinterpret_cast<const u32x4*>(krows + (size_t)j * (size_t)krow_words +
                                                  min(c4, d - 4));
        if (c4 >= d) v = u32x4{0u, 0u, 0u, 0u};
        st_k[c] = v;
      }
    }
  };
  auto stage_store = [&](int buf) {
    if constexpr (!DIRECT) {
#pragma unroll
      for (int c = 0; c < PER_THREAD; ++c) {
        const int idx = tid + 256 * c;
        if (C16_TOTAL % 256 == 0 || idx < C16_TOTAL) {
          const int r = idx / C16_PER_ROW;
          const int c4 = (idx % C16_PER_ROW) * 4;
          *reinterpret_cast<u32x4*>(&lds_k[buf][r * LDWK + c4]) = st_k[c];
        }
      }
    }
    // masked rows get a penalty ADDED (not selected), so the loads stay unconditional
    float b = kc0 * st_b0 + (has_kb1 ? kc1 * st_b1 : 0.f);
    b += (has_kb2 ? kc2 * st_b2 : 0.f);
    lds_b[buf][tid] = (fmaxf(b, kNegBig) + st_pen) * inv_lscale;
    if constexpr (VEC) lds_v[buf][tid] = st_v;
  };

  // v_permlane32_swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its
  // second, so (a, b) = (t, t) becomes (low half twice, high half twice).  Issued as inline
  // asm: this compiler models the builtin's two results as one register.
  auto swap_halves = [&](float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  };
  // max over the 16 key rows this lane holds and over the other half-wave of the column
  auto column_max = [&](const f32x16& acc) {
    const float m0 = fmaxf(fmaxf(acc[0], acc[1]), acc[2]);
    const float m1 = fmaxf(fmaxf(acc[3], acc[4]), acc[5]);
    const float m2 = fmaxf(fmaxf(acc[6], acc[7]), acc[8]);
    const float m3 = fmaxf(fmaxf(acc[9], acc[10]), acc[11]);
    const float m4 = fmaxf(fmaxf(acc[12], acc[13]), acc[14]);
    const float m5 = fmaxf(fmaxf(m0, m1), acc[15]);
    const float m6 = fmaxf(fmaxf(m2, m3), m4);
    float a = fmaxf(m5, m6), b = a;
    swap_halves(a, b);
    return fmaxf(a, b);
  };
  // classic online soft-max step; acc holds logit / lscale
  auto softmax = [&](const f32x16& acc, int rb, const f32x16& v16) {
    const float m_new = fmaxf(column_max(acc), run_m[rb]);
    // rounded once, on purpose: the exponents below, the rescale and the value handed to the
    // merge must all see the same number.  The empty asm hides the product from the
    // compiler: fused into the subtraction below (fp contraction) it would rescale by
    // 2^(rounding residual) on every tile, which adds up over a long key chunk.
    float c_new = -m_new * lscale;
    asm volatile("" : "+v"(c_new));
    float ps0 = 0.f, ps1 = 0.f, po = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const float e0 = fast_exp2(__builtin_fmaf(acc[r], lscale, c_new));
      const float e1 = fast_exp2(__builtin_fmaf(acc[r + 1], lscale, c_new));
      ps0 += e0;
      ps1 += e1;
      if constexpr (VEC) po = __builtin_fmaf(e0, v16[r], __builtin_fmaf(e1, v16[r + 1], po));
    }
    const float resc = fast_exp2(c_new - run_c[rb]);
    run_s[rb] = run_s[rb] * resc + (ps0 + ps1);
    if constexpr (VEC) run_o[rb] = run_o[rb] * resc + po;
    run_m[rb] = m_new;
    run_c[rb] = c_new;
  };
  auto softmax_first = [&](const f32x16& acc, int rb, const f32x16& v16) {
    const float delta = column_max(acc);
    float c = -delta * lscale;
    asm volatile("" : "+v"(c));
    float ps = 0.f, po = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float e = fast_exp2(__builtin_fmaf(acc[r], lscale, c));
      ps += e;
      if constexpr (VEC) po = __builtin_fmaf(e, v16[r], po);
    }
    if constexpr (VEC) run_o[rb] = po;
    run_s[rb] = ps;
    run_m[rb] = delta;
    run_c[rb] = c;
  };
  // The same step as `softmax`, piece p of kPieces; fma / exp2 / add of a value sit in
  // consecutive pieces so that no piece waits on its own results.
  auto softmax_piece = [&](int p, SoftmaxStage& s, const f32x16& a, int rb, const float* vsrc) {
    if (p == 0) {
      s.m[0] = fmaxf(fmaxf(a[0], a[1]), a[2]);
      s.m[1] = fmaxf(fmaxf(a[3], a[4]), a[5]);
      s.m[2] = fmaxf(fmaxf(a[6], a[7]), a[8]);
    }
    if (p == 1) {
      s.m[3] = fmaxf(fmaxf(a[9], a[10]), a[11]);
      s.m[4] = fmaxf(fmaxf(a[12], a[13]), a[14]);
      s.m[5] = fmaxf(fmaxf(s.m[0], s.m[1]), a[15]);
    }
    if (p == 2) {
      s.mx = fmaxf(s.m[5], fmaxf(fmaxf(s.m[2], s.m[3]), s.m[4]));  // this lane's 16 keys
      s.aa = s.mx;
      s.bb = s.mx;
      swap_halves(s.aa, s.bb);
    }
    if (p == 3) {
      const float m_new = fmaxf(fmaxf(s.aa, s.bb), run_m[rb]);
      s.cx = -m_new * lscale;
      asm volatile("" : "+v"(s.cx));  // see softmax(): the rounded product, nothing fused
      s.c = s.cx - run_c[rb];
      run_m[rb] = m_new;
      run_c[rb] = s.cx;
      s.ps0 = 0.f;
      s.ps1 = 0.f;
      s.po = 0.f;
    }
    const int q = p - 3;  // two values per piece: fma at q, exp2 at q + 1, add at q + 2
    if constexpr (BIASC) {
      // four fmas per piece: the logits registers are free again after piece 6 and take the
      // next unit's bias while the exponentials go on
      if (q >= 0 && q < 4) {
#pragma unroll
        for (int r = 4 * q; r < 4 * q + 4; ++r) s.t[r] = __builtin_fmaf(a[r], lscale, s.cx);
      }
    } else if (q >= 0 && q < 8) {
      s.t[2 * q] = __builtin_fmaf(a[2 * q], lscale, s.cx);
      s.t[2 * q + 1] = __builtin_fmaf(a[2 * q + 1], lscale, s.cx);
    }
    if (q >= 1 && q < 9) {
      s.e[2 * q - 2] = fast_exp2(s.t[2 * q - 2]);
      s.e[2 * q - 1] = fast_exp2(s.t[2 * q - 1]);
    }
    if constexpr (VEC) {
      // v of values 4g .. 4g+3 (used by the adds of q = 2g+2, 2g+3) is read at q = 2g: four
      // to eight of the sixteen values are in registers at any time
      if (q >= 0 && q < 8 && q % 2 == 0) {
        const float4 t = *reinterpret_cast<const float4*>(vsrc + 8 * (q / 2));
        s.v[(q / 2) & 1][0] = t.x;
        s.v[(q / 2) & 1][1] = t.y;
        s.v[(q / 2) & 1][2] = t.z;
        s.v[(q / 2) & 1][3] = t.w;
      }
    }
    if (q >= 2 && q < 10) {
      s.ps0 += s.e[2 * q - 4];
      s.ps1 += s.e[2 * q - 3];
      if constexpr (VEC) {
        const int r = 2 * q - 4;  // values r, r + 1 of group r / 4
        s.po = __builtin_fmaf(s.e[r], s.v[(r / 4) & 1][r % 4],
                              __builtin_fmaf(s.e[r + 1], s.v[(r / 4) & 1][r % 4 + 1], s.po));
      }
    }
  };
  auto softmax_tail = [&](SoftmaxStage& s, int rb) {  // what pieces 0..11 left undone
    s.ps0 += s.e[14];
    s.ps1 += s.e[15];
    const float resc = fast_exp2(s.c);
    run_s[rb] = run_s[rb] * resc + (s.ps0 + s.ps1);
    if constexpr (VEC) {
      s.po = __builtin_fmaf(s.e[14], s.v[1][2], __builtin_fmaf(s.e[15], s.v[1][3], s.po));
      run_o[rb] = run_o[rb] * resc + s.po;
    }
  };

  // A operands (one 32-key sub-tile) from LDS
  struct KeyRegs {
    float ya[kPlanes ? 1 : DP / 2];
    u32x4 yq[kPlanes ? NP : 1][kPlanes ? G::KK16 : 1];
    float ab;
  };
  // Direct mode: the key operands are read with ds_read_b128 written out by hand.  The compiler
  // cannot tell a read of one ring buffer from the global->LDS loads still filling another, and
  // would make every key read wait for ALL of them (vmcnt(0)), which cuts the two-tile
  // prefetch down to a fraction of a tile; the waits this kernel needs are the explicit ones
  // before the barrier.  The price: the compiler does not see these reads either, so every
  // consumer sits behind wait_lds().
  auto lds_read16 = [&](const unsigned* p) -> u32x4 {
    if constexpr (DIRECT) {
      u32x4 v;
      const unsigned addr =
          (unsigned)(size_t)(const __attribute__((address_space(3))) unsigned*)p;
      asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
      return v;
    } else {
      return *reinterpret_cast<const u32x4*>(p);
    }
  };
  auto wait_lds = [&]() {  // lgkmcnt(0): every LDS read issued so far has returned
    if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0xC07F);
  };
  auto load_keys = [&](KeyRegs& kr, int buf, int js) {
    const unsigned* yrow = lds_k[buf] + (js * 32 + li) * LDWK;
    if constexpr (!kPlanes) {
#pragma unroll
      for (int q = 0; q < DP / 8; ++q) {
        const float4 v = *reinterpret_cast<const float4*>(yrow + 8 * q + 4 * h);
        kr.ya[4 * q + 0] = v.x;
        kr.ya[4 * q + 1] = v.y;
        kr.ya[4 * q + 2] = v.z;
        kr.ya[4 * q + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int p = 0; p < NP; ++p)
#pragma unroll
        for (int kk = 0; kk < G::KK16; ++kk) {
          const int piece = p * (DP / 8) + 2 * kk + h;
          const int slot = DIRECT ? (piece ^ swz(li)) : piece;  // swz(js*32 + li) == swz(li)
          kr.yq[p][kk] = lds_read16(yrow + slot * 4);
        }
    }
    const float b = lds_b[buf][js * 32 + li];
    kr.ab = h ? 1.0f : b;
  };
  // MFMA number k (0 <= k < NMAIN) of one logits tile (32 keys x 32 queries) of query block
  // rb.  Plane products run from the lowest weight to hi*hi; lo*lo (2^-22) is left out.
  auto mfma_k = [&](int k, f32x16 acc, const KeyRegs& kr, int rb) {
    if constexpr (!kPlanes) {
      return __builtin_amdgcn_mfma_f32_32x32x2f32(kr.ya[k], xs[rb][k], acc, 0, 0, 0);
    } else {
      const int prod = k / G::KK16, kk = k % G::KK16;
      // (key plane, query plane): (lo,hi) (hi,lo) (hi,hi)
      const int pa = (prod == 0) ? 1 : 0;
      const int pb = (prod == 1) ? 1 : 0;
      return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kr.yq[pa][kk]),
                                                    __builtin_bit_cast(f16x8, xq[rb][pb][kk]), acc,
                                                    0, 0, 0);
    }
  };
  // BIASC: the key bias of sub-tile js as the accumulator layout holds it (register r of lane
  // (li, h) is key 8(r/4) + 4h + r%4): four 16-byte reads, the same address in each half-wave
  auto load_bias4 = [&](f32x16& b, int c, int buf, int js) {
    const float4 v = *reinterpret_cast<const float4*>(&lds_b[buf][js * 32 + 8 * c + 4 * h]);
    b[4 * c + 0] = v.x;
    b[4 * c + 1] = v.y;
    b[4 * c + 2] = v.z;
    b[4 * c + 3] = v.w;
  };
  auto load_v16 = [&](int buf, int js) {  // VEC: v_j in the accumulator layout, like the bias
    f32x16 v;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const float4 t = *reinterpret_cast<const float4*>(&lds_v[VEC ? buf : 0][js * 32 + 8 * c + 4 * h]);
      v[4 * c + 0] = t.x;
      v[4 * c + 1] = t.y;
      v[4 * c + 2] = t.z;
      v[4 * c + 3] = t.w;
    }
    return v;
  };
  auto load_bias16 = [&](int buf, int js) {
    f32x16 b;
#pragma unroll
    for (int c = 0; c < 4; ++c) load_bias4(b, c, buf, js);
    return b;
  };
  auto chain = [&](const KeyRegs& kr, int rb, int buf, int js) {
    f32x16 acc;
    if constexpr (BIASC) {
      acc = load_bias16(buf, js);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    }
#pragma unroll
    for (int k = 0; k < NMAIN; ++k) acc = mfma_k(k, acc, kr, rb);
    return acc;
  };
  // The bias MFMA (fp32 operands in every mode): adds kbias_j.
  auto add_bias = [&](f32x16 acc, const KeyRegs& kr, int rb) -> f32x16 {
    if constexpr (BIASC) return acc;  // the chain started from the bias
    return __builtin_amdgcn_mfma_f32_32x32x2f32(kr.ab, h ? 0.0f : 1.0f, acc, 0, 0, 0);
  };

  KeyRegs K[KPF ? 2 : 1];

  // Wait until at most `newer` of this wavefront's vector-memory operations are outstanding
  // (the direct loads write LDS behind the compiler's back, so their waits are explicit).
  // Loads complete in issue order, register loads and global->LDS loads alike, which is what
  // lets a count stand for "everything older than the newest tile has landed".  gfx9 encoding
  // of s_waitcnt: vmcnt in bits 3:0 and 15:14, expcnt 6:4 (7 = no wait), lgkmcnt 11:8.
  auto wait_vm = [&](auto newer) {
    constexpr int n = decltype(newer)::value;
    __builtin_amdgcn_s_waitcnt(0x0F70 | (n & 15) | ((n >> 4) << 14));
  };
  constexpr int kLoadsPerTile = (DIRECT ? PER_THREAD : 0) + 3;  // direct loads + bias terms
  auto wait_all_vm = [&]() { wait_vm(std::integral_constant<int, 0>{}); };
  auto wait_older_tiles = [&]() { wait_vm(std::integral_constant<int, kLoadsPerTile>{}); };
  auto wait_older_tiles_and_lds = [&]() {  // the same, and lgkmcnt(0)
    constexpr int n = kLoadsPerTile;
    __builtin_amdgcn_s_waitcnt(0x0070 | (n & 15) | ((n >> 4) << 14));
  };

  // LDS buffers rotate: cur holds the tile being multiplied, nxt the next one, nx2 (direct
  // mode with three buffers) the one after that; with two buffers nx2 is cur.
  int cur = 0, nxt = 1 % NBUF, nx2 = 2 % NBUF;
  auto rotate = [&]() {
    const int c = cur;
    cur = nxt;
    nxt = nx2;
    nx2 = (NBUF == 3) ? c : cur;
    if (NBUF == 2) nxt = c;
  };

  // ---- prologue: tile 0 into buffer 0; with KPF tile 1 is already on its way ----
  stage_load(j_begin, 0);
  stage_store(0);
  if constexpr (KPF) stage_load(j_begin + G::JT, 1);
  if constexpr (DIRECT) wait_all_vm();
  __syncthreads();
  if constexpr (KPF) load_keys(K[0], 0, 0);

  // ---- tile 0: establishes the running max, no soft-max pipelining ----
  {
    if constexpr (KPF) {
      stage_store(nxt);                               // bias (and registers) of tile 1
      stage_load(j_begin + 2 * G::JT, nx2);           // tile 2
    } else {
      stage_load(j_begin + G::JT, nxt);
    }
#pragma unroll
    for (int js = 0; js < NSUB; ++js) {
      if constexpr (!KPF) load_keys(K[0], cur, js);
      KeyRegs& kr = K[KPF ? (js & 1) : 0];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (KPF && rb == RB - 1) {
          if (js + 1 < NSUB) {
            load_keys(K[(js + 1) & 1], cur, js + 1);
          } else {
            if constexpr (DIRECT) wait_older_tiles();  // tile 1 has landed
            __syncthreads();  // tile 1 is visible; every wave is done reading buffer cur
            load_keys(K[0], nxt, 0);
          }
        }
        wait_lds();
        FS_SCHED_FENCE();
        const f32x16 acc = add_bias(chain(kr, rb, cur, js), kr, rb);
        f32x16 v16;
        if constexpr (VEC) v16 = load_v16(cur, js);
        if (js == 0) softmax_first(acc, rb, v16); else softmax(acc, rb, v16);
      }
    }
    if constexpr (!KPF) {
      stage_store(nxt);
      if constexpr (DIRECT) wait_all_vm();
      __syncthreads();
    }
    rotate();
  }

  // R1: logits of the previous unit.  BIASC: R0 and R1 swap roles from unit to unit (one holds
  // the running MFMA chain, the other the previous logits, whose registers take the next
  // unit's bias as the soft-max lets go of them); a tile has an even number of units, so the
  // roles are fixed in the unrolled code and nothing is ever copied.
  f32x16 R0, R1;
#pragma unroll
  for (int r = 0; r < 16; ++r) R1[r] = kNegBig;
  if constexpr (BIASC) R0 = load_bias16(cur, 0);
  static_assert(!BIASC || (NSUB * RB) % 2 == 0, "units per tile must be even");

  // ---- steady state: the soft-max of the previous logits tile rides between the MFMAs ----
  for (int t = 1; t < ntiles; ++t) {
    if constexpr (!KPF) stage_load(j_begin + (t + 1) * G::JT, nxt);
#pragma unroll
    for (int js = 0; js < NSUB; ++js) {
      if constexpr (!KPF) load_keys(K[0], cur, js);
      KeyRegs& kr = K[KPF ? (js & 1) : 0];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int prev_rb = (rb + RB - 1) % RB;
        SoftmaxStage st;
        const bool odd = ((js * RB + rb) & 1) != 0;
        f32x16 acc_zero;
        f32x16& acc = BIASC ? (odd ? R1 : R0) : acc_zero;
        f32x16& acc_prev = BIASC ? (odd ? R0 : R1) : R1;
        if constexpr (!BIASC) {
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        }
        // VEC: v of the previous unit's keys (its soft-max runs during this unit).  The previous
        // unit sits on the same sub-tile, on the one before, or on the last one of the previous
        // tile, whose buffer is the third of the ring until the next tile's staging reuses it.
        const float* vsrc = nullptr;
        if constexpr (VEC) {
          const bool same_js = rb > 0;
          const bool same_tile = same_js || js > 0;
          vsrc = &lds_v[same_tile ? cur : nx2][(same_js ? js : (js + NSUB - 1) % NSUB) * 32 + 4 * h];
        }
        wait_lds();  // this unit's key operands (read one unit ago) are in their registers
        FS_SCHED_FENCE();
        // MFMAs of piece p of this unit, the pipeline's memory traffic, and (soft) piece p
        // of the previous unit's soft-max
        auto k_first = [](int p) { return (p * NMAIN) / kPieces; };  // MFMAs of piece p
        auto step = [&](int p, bool soft) {
#pragma unroll
          for (int k = k_first(p); k < k_first(p + 1); ++k) acc = mfma_k(k, acc, kr, rb);
          if constexpr (KPF) {
            // LDS / global traffic of the pipeline, placed where it has the whole unit to land
            if (js == 0 && rb == 0 && p == 0) stage_store(nxt);                   // tile t+1
            if (js == 0 && rb == 0 && p == 1) stage_load(j_begin + (t + 2) * G::JT, nx2);
            if (rb == RB - 1 && js + 1 < NSUB && p == 1) load_keys(K[(js + 1) & 1], cur, js + 1);
            if (rb == RB - 1 && js + 1 == NSUB && p == 1) {
              if constexpr (DIRECT) {
                // tile t+1 has landed and this wave's bias store has been performed; tile
                // t+2 stays in flight across the barrier.  A bare s_barrier: __syncthreads()
                // carries a release fence, for which the compiler waits for every
                // outstanding global->LDS load, the ones of tile t+2 included.
                wait_older_tiles_and_lds();
                // the empty asm statements keep the compiler from moving LDS accesses across
                // the barrier (the barrier builtin itself is not a memory operation to it)
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
              } else {
                __syncthreads();
              }
            }
            if (rb == RB - 1 && js + 1 == NSUB && p == 2) load_keys(K[0], nxt, 0);
          }
          if constexpr (BIASC) {
            // piece p - 1 was the last to read logits 4(p - 4) .. 4(p - 4) + 3 of the previous
            // unit: their registers take the next unit's bias
            if (p >= kBiasPiece && p < kBiasPiece + 4) {
              const bool same_js = rb + 1 < RB;
              const bool same_tile = same_js || js + 1 < NSUB;
              load_bias4(acc_prev, p - kBiasPiece, same_tile ? cur : nxt,
                         same_js ? js : (js + 1) % NSUB);
            }
          }
          // a wave-uniform branch around VALU work only: the MFMA chain itself stays one
          // straight line, accumulating in place
          if (soft) softmax_piece(p, st, acc_prev, prev_rb, vsrc);
          FS_SCHED_FENCE();
        };
#pragma unroll
        for (int p = 0; p < kMaxPieces; ++p) step(p, true);
        // Every logit of the previous unit more than 2^40 (LaunchArgs::skip_log2) below its
        // row's running maximum: its exponentials would not change the fp32 row sums, so
        // they are not computed.
        const float mx_rel = st.mx - run_m[prev_rb];
        const bool soft = wave_any(mx_rel > skip_below);
        n_left_out += soft ? 0u : 1u;
        if constexpr (BIASC) {
          // one branch per piece: a two-sided branch with the MFMAs on both sides makes the
          // compiler move the accumulator tile at the join
#pragma unroll
          for (int p = kMaxPieces; p < kPieces; ++p) step(p, soft);
          if (soft) softmax_tail(st, prev_rb);
        } else if (soft) {
#pragma unroll
          for (int p = kMaxPieces; p < kPieces; ++p) step(p, true);
          softmax_tail(st, prev_rb);
        } else {
#pragma unroll
          for (int p = kMaxPieces; p < kPieces; ++p) step(p, false);
        }
        if constexpr (!BIASC) R1 = add_bias(acc, kr, rb);
        FS_SCHED_FENCE();
      }
    }
    if constexpr (!KPF) {
      stage_store(nxt);
      if constexpr (DIRECT) wait_all_vm();
      __syncthreads();
    }
    rotate();
  }
  {  // BIASC: the last unit of a tile is an odd one, its chain ran in R1
    f32x16 v16;
    if constexpr (VEC) v16 = load_v16(nx2, NSUB - 1);  // after rotate(): the tile just finished
    softmax(R1, RB - 1, v16);
  }

  // With the variant chosen on the device, this kernel's own counts (units whose exponentials
  // it left out, of all its units) tell the merge kernel when the plan has become peaked enough
  // for the variant with the coarse tile test (a schedule of decreasing eps gets there).
  if constexpr (PREC == kH3 && !VEC) {
    if (args.sel != nullptr && args.sel_pred && lane == 0 && ntiles > 0) {
      const int slot = blockIdx.x % kSelSlots;
      atomicAdd(&args.sel[kSelEnded + slot], n_left_out);
      atomicAdd(&args.sel[kSelUnits + slot], (unsigned)(ntiles * NSUB * RB));
    }
  }

#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = row0 + rb * 32 + li;
    const float s = run_s[rb] + xor32(run_s[rb]);
    const float o = VEC ? run_o[rb] + xor32(run_o[rb]) : 0.f;
    const float M2 = -run_c[rb];
    if (row < sd.nq && h == 0) {
      if (sd.splits == 1) {
        epilogue_scalar(sd.ep, row, M2, s, o);
      } else {
        const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
        *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(M2, s);
        if constexpr (VEC) sd.part_o[pr] = o;
        // this kernel follows no keys: the merge must not take what an earlier launch (or an
        // earlier user of the workspace) left in the array for one
        if constexpr (!VEC) {
          if (sd.part_best != nullptr) sd.part_best[pr] = -1;
        }
      }
    }
  }
}

}  // namespace fs
