// Software-pipelined log-sum-exp kernel (d <= 128, d % 4 == 0, aligned rows).
//
// Same decomposition as stream_kernel<kLse> (stationary query blocks in VGPRs,
// key tiles through LDS, transposed logits, lane-private online soft-max, bias
// and running max folded into one extra MFMA), with two changes that matter for
// speed:
//   * the soft-max of logits tile u-1 is placed in program order BETWEEN the
//     MFMAs of tile u.  A chain of dependent MFMAs blocks a wavefront's issue
//     slot, so only VALU work interleaved this way runs in the MFMA shadow;
//   * the online soft-max is branch free (per-lane max, rescale by exp2(-delta) every
//     tile).  With the keys split into chunks every chunk is short, new running
//     maxima are frequent, and a wave-wide "does any lane need a rescale" branch
//     would be taken on almost every tile; ~60 VALU ops per tile hide under the
//     MFMAs instead.  Only the very first tile of a block is handled apart.
//
// Operand precision (PREC):
//   kF32   v_mfma_f32_32x32x2_f32 on fp32 operands.
//          (bf16 modes read operands that split_planes_kernel has already split into packed
//          bf16 planes, unscaled; the logit scale is applied in the exp2 argument's FMA and
//          the bias / running-max fold uses one fp32 MFMA, so no per-tile conversion work.)
//   kBf3   operands split into two bf16 planes (hi, lo); hi*hi + hi*lo + lo*hi on
//          v_mfma_f32_32x32x16_bf16, fp32 accumulate: ~2^-17 relative per product,
//          the counterpart of the reference's allow_tf32=True.
//   kBf6   three bf16 planes, the six products whose weight is >= 2^-16: same
//          accuracy class as fp32 operands (the planes sum to the fp32 value exactly)
//          at 6/16 of the fp32 MFMA time.
#pragma once

#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

enum Prec : int { kF32 = 0, kBf3 = 1, kBf6 = 2 };

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float bf16_lo_as_f32(unsigned p) {
  return __builtin_bit_cast(float, p << 16);
}
__device__ __forceinline__ float bf16_hi_as_f32(unsigned p) {
  return __builtin_bit_cast(float, p & 0xffff0000u);
}

// Split the pair (a, b) into NP packed bf16 planes with round-to-nearest pieces.
template <int NP>
__device__ __forceinline__ void split_pair(float a, float b, unsigned (&out)[NP]) {
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    out[p] = pack_bf16(a, b);
    if (p + 1 < NP) {
      a -= bf16_lo_as_f32(out[p]);
      b -= bf16_hi_as_f32(out[p]);
    }
  }
}

// x[rows, d] (fp32) -> packed bf16 planes [rows][NP][DP/2] (32-bit words), zero padded to DP
// columns; plane p holds the p-th round-to-nearest bf16 piece, so the planes sum to x.
template <int NP>
__global__ __launch_bounds__(256) void split_planes_kernel(const float* __restrict__ src,
                                                           unsigned* __restrict__ dst, int rows,
                                                           int d, int dp) {
  const int per_row = dp / 4;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long long)rows * per_row) return;
  const int r = (int)(idx / per_row);
  const int c4 = (int)(idx % per_row) * 4;
  const float* p = src + (size_t)r * (size_t)d;
  float v[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) v[t] = (c4 + t < d) ? p[c4 + t] : 0.f;
  unsigned p01[NP], p23[NP];
  split_pair<NP>(v[0], v[1], p01);
  split_pair<NP>(v[2], v[3], p23);
  unsigned* o = dst + (size_t)r * (size_t)(NP * dp / 2);
#pragma unroll
  for (int pl = 0; pl < NP; ++pl)
    *reinterpret_cast<uint2*>(o + pl * (dp / 2) + c4 / 2) = make_uint2(p01[pl], p23[pl]);
}

// Scheduling hint for one pipelined unit: N MFMAs in a row, with the 17 exp2 and ~44 plain
// VALU ops of the lagging soft-max spread evenly between them.
template <int I, int N>
struct SpreadSoftmax {
  static __device__ __forceinline__ void emit() {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                       // MFMA
    __builtin_amdgcn_sched_group_barrier(0x400, (17 * (I + 1)) / N - (17 * I) / N, 0);       // exp2
    __builtin_amdgcn_sched_group_barrier(0x002, (44 * (I + 1)) / N - (44 * I) / N, 0);       // VALU
    SpreadSoftmax<I + 1, N>::emit();
  }
};
template <int N>
struct SpreadSoftmax<N, N> {
  static __device__ __forceinline__ void emit() {}
};

template <int DP, int PREC>
struct Geo2 {
  static constexpr int NP = (PREC == kF32) ? 1 : (PREC == kBf3 ? 2 : 3);
  static constexpr int JT = (DP >= 128) ? 32 : 64;
  static constexpr int NSUB = JT / 32;
  // LDS row stride in 32-bit words: fp32 row + 4, or NP bf16 planes + 4
  static constexpr int LDW = (PREC == kF32) ? (DP + 4) : (NP * DP / 2 + 4);
  static constexpr int V4_PER_ROW = DP / 4;
  static constexpr int V4_TOTAL = JT * V4_PER_ROW;
  static constexpr int PER_THREAD = (V4_TOTAL + 255) / 256;
  static constexpr int KK16 = DP / 16;  // bf16 MFMAs per plane pair
};

template <int DP, int RB, int PREC>
__global__ __launch_bounds__(256, 2) void lse2_kernel(const LaunchArgs args) {
  using G = Geo2<DP, PREC>;
  constexpr int NP = G::NP;
  constexpr bool kBf = (PREC != kF32);
  constexpr int ROWW = kBf ? NP * DP / 2 : DP;  // 32-bit words per operand row in global memory

  __shared__ __attribute__((aligned(16))) unsigned lds_k[2][G::JT * G::LDW];
  __shared__ __attribute__((aligned(16))) float lds_b[2][G::JT];

  int bid = blockIdx.x;
  const bool second = bid >= args.blocks0;
  if (second) bid -= args.blocks0;
  const Side& sd = second ? args.side[1] : args.side[0];
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
  // bf16 modes: MFMAs produce raw dot products; lscale turns them into base-2 logits inside
  // the exp2 argument, and the bias / running max are kept in dot-product units.
  const float lscale = kBf ? sd.qscale : 1.0f;
  const float inv_lscale = kBf ? 1.0f / sd.qscale : 1.0f;

  // ---- stationary query operands ----
  float xs[kBf ? 1 : RB][kBf ? 1 : DP / 2];
  u32x4 xq[kBf ? RB : 1][kBf ? NP : 1][kBf ? G::KK16 : 1];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = min(row0 + rb * 32 + li, sd.nq - 1);
    if constexpr (!kBf) {
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

  float run_m[RB], run_s[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    run_m[rb] = 0.f;
    run_s[rb] = 0.f;
  }

  // ---- staging (global -> registers -> LDS), branch free: rows are clamped, masked by bias ----
  constexpr int C16_PER_ROW = ROWW / 4;  // 16-byte chunks per operand row
  constexpr int C16_TOTAL = G::JT * C16_PER_ROW;
  constexpr int PER_THREAD = (C16_TOTAL + 255) / 256;
  u32x4 st_k[PER_THREAD];
  float st_b = 0.f;
  const unsigned* krows = kBf ? sd.kplanes : reinterpret_cast<const unsigned*>(sd.k);
  const int krow_words = kBf ? ROWW : d;
  auto stage_load = [&](int j0) {
#pragma unroll
    for (int c = 0; c < PER_THREAD; ++c) {
      const int idx = tid + 256 * c;
      const int r = idx / C16_PER_ROW;
      const int c4 = (idx % C16_PER_ROW) * 4;
      const int j = min(j0 + r, j_end - 1);
      u32x4 v = {0u, 0u, 0u, 0u};
      if (kBf || c4 < d)
        v = *reinterpret_cast<const u32x4*>(krows + (size_t)j * (size_t)krow_words + c4);
      st_k[c] = v;
    }
    if (tid < G::JT) st_b = key_bias(sd, j0 + tid, j_end) * inv_lscale;
  };
  auto stage_store = [&](int buf) {
#pragma unroll
    for (int c = 0; c < PER_THREAD; ++c) {
      const int idx = tid + 256 * c;
      if (C16_TOTAL % 256 == 0 || idx < C16_TOTAL) {
        const int r = idx / C16_PER_ROW;
        const int c4 = (idx % C16_PER_ROW) * 4;
        *reinterpret_cast<u32x4*>(&lds_k[buf][r * G::LDW + c4]) = st_k[c];
      }
    }
    if (tid < G::JT) lds_b[buf][tid] = st_b;
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
    const float tmax = fmaxf(m5, m6);
#ifdef FS_DBG_XOR32
    return fmaxf(tmax, xor32(tmax));
#else
    // v_permlane32_swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its
    // second, so (a, b) = (tmax, tmax) becomes (low half twice, high half twice).  Issued as
    // inline asm: this compiler models the builtin's two results as one register.
    float a = tmax, b = tmax;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return fmaxf(a, b);
#endif
  };
  // classic online soft-max step; acc holds (logit - M)/lscale for the current M = run_m[rb]
  auto softmax = [&](const f32x16& acc, int rb) {
    const float delta = fmaxf(column_max(acc), 0.f);
    // the max actually applied is what fp32 can represent next to the old one
    const float m_new = run_m[rb] + delta;
    const float c = -(m_new - run_m[rb]) * lscale;
    float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      ps0 += fast_exp2(__builtin_fmaf(acc[r], lscale, c));
      ps1 += fast_exp2(__builtin_fmaf(acc[r + 1], lscale, c));
    }
    run_s[rb] = run_s[rb] * fast_exp2(c) + (ps0 + ps1);
    run_m[rb] = m_new;
  };
  auto softmax_first = [&](const f32x16& acc, int rb) {
    const float delta = column_max(acc);
    const float c = -delta * lscale;
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) ps += fast_exp2(__builtin_fmaf(acc[r], lscale, c));
    run_s[rb] = ps;
    run_m[rb] = delta;
  };

  // A operands (one 32-key sub-tile) from LDS
  struct KeyRegs {
    float ya[kBf ? 1 : DP / 2];
    u32x4 yq[kBf ? NP : 1][kBf ? G::KK16 : 1];
    float ab;
  };
  auto load_keys = [&](KeyRegs& kr, int buf, int js) {
    const unsigned* yrow = lds_k[buf] + (js * 32 + li) * G::LDW;
    if constexpr (!kBf) {
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
        for (int kk = 0; kk < G::KK16; ++kk)
          kr.yq[p][kk] = *reinterpret_cast<const u32x4*>(yrow + p * (DP / 2) + 8 * kk + 4 * h);
    }
    kr.ab = h ? 1.0f : lds_b[buf][js * 32 + li];
  };
  // One logits tile (32 keys x 32 queries) of query block rb: all MFMAs except the bias one.
  auto chain = [&](const KeyRegs& kr, int rb) {
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    if constexpr (!kBf) {
#pragma unroll
      for (int kk = 0; kk < DP / 2; ++kk)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(kr.ya[kk], xs[rb][kk], acc, 0, 0, 0);
    } else {
      // low-order products first, hi*hi last
#pragma unroll
      for (int pa = NP - 1; pa >= 0; --pa)
#pragma unroll
        for (int pb = NP - 1; pb >= 0; --pb) {
          if (pa + pb > NP - 1) continue;  // weight below 2^-16 (2^-24 for three planes)
#pragma unroll
          for (int kk = 0; kk < G::KK16; ++kk)
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, kr.yq[pa][kk]),
                __builtin_bit_cast(bf16x8, xq[rb][pb][kk]), acc, 0, 0, 0);
        }
    }
    return acc;
  };
  // The bias MFMA (fp32 operands in every mode): adds kbias_j - M_i with the freshest M.
  auto add_bias = [&](f32x16 acc, const KeyRegs& kr, int rb) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(kr.ab, h ? -run_m[rb] : 1.0f, acc, 0, 0, 0);
  };
  constexpr int kMain = kBf ? (NP == 2 ? 3 : 6) * G::KK16 : DP / 2;  // MFMAs per chain

  stage_load(j_begin);
  stage_store(0);
  __syncthreads();

  f32x16 acc_prev;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc_prev[r] = kNegBig;

  for (int t = 0; t < ntiles; ++t) {
    const int buf = t & 1;
    const bool more = (t + 1 < ntiles);
    if (more) stage_load(j_begin + (t + 1) * G::JT);

    if (t == 0) {
      // first tile of the block: establish the running max, no pipelining
#pragma unroll
      for (int js = 0; js < G::NSUB; ++js) {
        KeyRegs kr;
        load_keys(kr, buf, js);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const f32x16 acc = add_bias(chain(kr, rb), kr, rb);
          if (js == 0) softmax_first(acc, rb); else softmax(acc, rb);
        }
      }
    } else {
#pragma unroll
      for (int js = 0; js < G::NSUB; ++js) {
        KeyRegs kr;
        load_keys(kr, buf, js);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          f32x16 acc = chain(kr, rb);
          // the soft-max of the previous tile runs in the shadow of the MFMAs above
          softmax(acc_prev, (rb + RB - 1) % RB);
#ifndef FS_DBG_NOSCHED
          SpreadSoftmax<0, kMain>::emit();
#endif
          acc_prev = add_bias(acc, kr, rb);
        }
      }
    }

    if (more) stage_store(buf ^ 1);
    __syncthreads();
  }
  softmax(acc_prev, RB - 1);

#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = row0 + rb * 32 + li;
    const float s = run_s[rb] + xor32(run_s[rb]);
    const float M2 = run_m[rb] * lscale;
    if (row < sd.nq && h == 0) {
      if (sd.splits == 1) {
        epilogue_scalar(sd.ep, row, M2, s, 0.f);
      } else {
        const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
        *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(M2, s);
      }
    }
  }
}

}  // namespace fs
