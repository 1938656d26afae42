// Streaming plan kernels for feature dimension d <= 128 (fp32 MFMA).
//
// Work decomposition (one workgroup = 4 wavefronts of 64 lanes):
//   * each wavefront owns RB blocks of 32 stationary query rows, held in VGPRs
//     for the whole sweep, pre-multiplied by qscale;
//   * the workgroup streams its chunk of key rows through LDS in tiles of JT
//     rows (double buffered, one barrier per tile); all four wavefronts read the
//     same key tile;
//   * logits are produced TRANSPOSED, (keys x queries), by
//     v_mfma_f32_32x32x2_f32 with the key tile as the A operand.  In that layout
//     a lane holds ONE query column and 16 key rows, so the online soft-max over
//     keys is lane-private: no cross-lane traffic in the inner loop.  The two
//     half-waves of a column are merged once at the end;
//   * one extra MFMA per tile adds kbias_j - M_i to every logit (A = [kbias, 1],
//     B = [1, -M]), so masking, the bias and the running-max subtraction cost no
//     VALU work.  The running max M is only moved when a tile exceeds it by
//     more than 2^16 ("lazy rescale"), a wave-uniform rare branch;
//   * exp'ed logits are already laid out as the B operand of a second MFMA
//     against the value tile (keys x d), which accumulates O^T for the
//     gradient / plan-matrix / mat5 kinds.
//
// The key range can be split into `splits` chunks to fill the chip; partial
// (M, s, O) statistics are then merged by finish_kernel.
#pragma once

#include "fs_common.hpp"

namespace fs {

template <int DP>
struct Geo {
  static constexpr int JT = (DP >= 128) ? 32 : 64;  // key rows per LDS tile
  static constexpr int NSUB = JT / 32;
  static constexpr int LDW = DP + 4;                // padded LDS row stride (floats)
  static constexpr int KK = DP / 2;                 // MFMAs per 32x32 logits tile
  static constexpr int NQ8 = DP / 8;
  static constexpr int NDB = (DP + 31) / 32;        // 32-wide output column blocks
  static constexpr int V4_PER_ROW = DP / 4;
  static constexpr int V4_TOTAL = JT * V4_PER_ROW;
  static constexpr int PER_THREAD = (V4_TOTAL + 255) / 256;
  static constexpr bool VDB = false;                // separate value tile is single buffered
};

__device__ __forceinline__ float4 load_row4(const float* __restrict__ base, int row, int nrows,
                                            int col, int d, bool vec_ok) {
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (row < nrows && col < d) {
    const float* p = base + (size_t)row * (size_t)d + col;
    if (vec_ok) {
      v = *reinterpret_cast<const float4*>(p);
    } else {
      v.x = p[0];
      if (col + 1 < d) v.y = p[1];
      if (col + 2 < d) v.z = p[2];
      if (col + 3 < d) v.w = p[3];
    }
  }
  return v;
}

__device__ __forceinline__ float key_bias(const Side& sd, int j, int j_end) {
  float b = kNegBig;
  if (j < j_end) {
    b = sd.kc0 * sd.kb0[j];
    if (sd.kb1) b += sd.kc1 * sd.kb1[j];
    if (sd.kb2) b += sd.kc2 * sd.kb2[j];
    b = fmaxf(b, kNegBig);
  }
  return b;
}

// ---- epilogues -------------------------------------------------------------

__device__ __forceinline__ float apply_row_factor(const Epilogue& ep, int row, float M) {
  float t = M + ep.rc0 * ep.r0[row];
  if (ep.r1) t += ep.rc1 * ep.r1[row];
  if (ep.r2) t += ep.rc2 * ep.r2[row];
  return ep.post * exp2f(t);
}

__device__ __forceinline__ void epilogue_scalar(const Epilogue& ep, int row, float M, float s,
                                                float o) {
  if (ep.kind == kEpiLse) {
    float cand = ep.out_scale * (M + log2f(fmaxf(s, 1e-40f)));
    float r = ep.alpha * cand;
    if (ep.old) r += (1.0f - ep.alpha) * ep.old[row];
    if (ep.shift) r -= ep.shift_coef * ep.shift[row];
    ep.out[row] = r;
  } else {
    float r = apply_row_factor(ep, row, M) * o;
    if (ep.mul) r *= ep.mul[row];
    if (ep.add_a) r = ep.add_a[row] * ep.add_b[row] + ep.res_coef * r;
    ep.out[row] = r;
  }
}

__device__ __forceinline__ void epilogue_vec4(const Epilogue& ep, const float* __restrict__ q,
                                              int d, bool vec_ok, int row, int col, float M,
                                              float s, float4 O) {
  if (col >= d) return;
  float4 r;
  if (ep.kind == kEpiGrad) {
    float gs = ep.grad_scale ? ep.grad_scale[0] : 1.0f;
    float c = ep.gcoef * gs * ep.w[row];
    float inv = 1.0f / fmaxf(s, 1e-40f);
    float4 x = load_row4(q, row, row + 1, col, d, vec_ok);
    r = make_float4(c * (x.x - O.x * inv), c * (x.y - O.y * inv), c * (x.z - O.z * inv),
                    c * (x.w - O.w * inv));
  } else {
    float c = apply_row_factor(ep, row, M);
    r = make_float4(c * O.x, c * O.y, c * O.z, c * O.w);
  }
  float* p = ep.out + (size_t)row * (size_t)d + col;
  if (vec_ok) {
    *reinterpret_cast<float4*>(p) = r;
  } else {
    p[0] = r.x;
    if (col + 1 < d) p[1] = r.y;
    if (col + 2 < d) p[2] = r.z;
    if (col + 3 < d) p[3] = r.w;
  }
}

// ---- main kernel -----------------------------------------------------------

template <int MODE, int DP, int RB, bool SEPV>
__global__ __launch_bounds__(256) void stream_kernel(const LaunchArgs args) {
  using G = Geo<DP>;
  constexpr bool kHasO = (MODE == kMat || MODE == kMat5);
  constexpr int NVBUF = G::VDB ? 2 : 1;

  __shared__ __attribute__((aligned(16))) float lds_k[2][G::JT * G::LDW];
  __shared__ __attribute__((aligned(16))) float lds_v[SEPV ? NVBUF : 1][SEPV ? G::JT * G::LDW : 4];
  __shared__ __attribute__((aligned(16))) float lds_b[2][G::JT];
  __shared__ __attribute__((aligned(16))) float lds_x[2][MODE == kVec ? G::JT : 4];

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
  const int ntiles = (j_end - j_begin + G::JT - 1) / G::JT;

  // ---- stationary operands: lane (li, h) keeps q[row][8q+4h+t] for all q, t ----
  float xs[RB][G::KK];
  float x2s[MODE == kMat5 ? RB : 1][MODE == kMat5 ? G::KK : 1];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = row0 + rb * 32 + li;
#pragma unroll
    for (int q = 0; q < G::NQ8; ++q) {
      float4 v = load_row4(sd.q, row, sd.nq, 8 * q + 4 * h, d, vec_ok);
      xs[rb][4 * q + 0] = v.x * sd.qscale;
      xs[rb][4 * q + 1] = v.y * sd.qscale;
      xs[rb][4 * q + 2] = v.z * sd.qscale;
      xs[rb][4 * q + 3] = v.w * sd.qscale;
      if constexpr (MODE == kMat5) {
        float4 u = load_row4(sd.q2, row, sd.nq, 8 * q + 4 * h, d, vec_ok);
        x2s[rb][4 * q + 0] = u.x;
        x2s[rb][4 * q + 1] = u.y;
        x2s[rb][4 * q + 2] = u.z;
        x2s[rb][4 * q + 3] = u.w;
      }
    }
  }

  float run_m[RB], run_s[RB], run_o[RB];
  int best_j[RB];  // kArgmax: run_m holds the largest value so far, best_j its key
  f32x16 oacc[kHasO ? RB : 1][kHasO ? G::NDB : 1];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    best_j[rb] = 0;
    run_m[rb] = (MODE == kArgmax) ? -3.0e38f : 0.f;
    run_s[rb] = 0.f;
    run_o[rb] = 0.f;
    if constexpr (kHasO) {
#pragma unroll
      for (int db = 0; db < G::NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[rb][db][r] = 0.f;
    }
  }

  // ---- tile staging registers ----
  float4 st_k[G::PER_THREAD];
  float4 st_v[SEPV ? G::PER_THREAD : 1];
  float st_b = 0.f, st_x = 0.f;

  auto stage_load = [&](int j0) {
#pragma unroll
    for (int c = 0; c < G::PER_THREAD; ++c) {
      const int idx = tid + 256 * c;
      const int r = idx / G::V4_PER_ROW;
      const int c4 = (idx % G::V4_PER_ROW) * 4;
      const int j = j0 + r;
      st_k[c] = load_row4(sd.k, j, j_end, c4, d, vec_ok);
      if constexpr (SEPV) {
        float4 v = load_row4(sd.v, j, j_end, c4, d, vec_ok);
        if (sd.vscale && j < j_end) {
          const float sc = sd.vscale[j];
          v.x *= sc; v.y *= sc; v.z *= sc; v.w *= sc;
        }
        st_v[c] = v;
      }
    }
    if (tid < G::JT) {
      st_b = key_bias(sd, j0 + tid, j_end);
    } else if (MODE == kVec && tid < 2 * G::JT) {
      const int j = j0 + tid - G::JT;
      st_x = (j < j_end) ? sd.v[j] : 0.f;
    }
  };
  auto stage_store_k = [&](int buf) {
#pragma unroll
    for (int c = 0; c < G::PER_THREAD; ++c) {
      const int idx = tid + 256 * c;
      if (G::V4_TOTAL % 256 == 0 || idx < G::V4_TOTAL) {
        const int r = idx / G::V4_PER_ROW;
        const int c4 = (idx % G::V4_PER_ROW) * 4;
        *reinterpret_cast<float4*>(&lds_k[buf][r * G::LDW + c4]) = st_k[c];
      }
    }
    if (tid < G::JT) {
      lds_b[buf][tid] = st_b;
    } else if (MODE == kVec && tid < 2 * G::JT) {
      lds_x[buf][tid - G::JT] = st_x;
    }
  };
  auto stage_store_v = [&](int buf) {
    if constexpr (SEPV) {
#pragma unroll
      for (int c = 0; c < G::PER_THREAD; ++c) {
        const int idx = tid + 256 * c;
        if (G::V4_TOTAL % 256 == 0 || idx < G::V4_TOTAL) {
          const int r = idx / G::V4_PER_ROW;
          const int c4 = (idx % G::V4_PER_ROW) * 4;
          *reinterpret_cast<float4*>(&lds_v[buf][r * G::LDW + c4]) = st_v[c];
        }
      }
    }
  };

  stage_load(j_begin);
  stage_store_k(0);
  stage_store_v(0);
  __syncthreads();

  for (int t = 0; t < ntiles; ++t) {
    const int buf = t & 1;
    const int vbuf = G::VDB ? buf : 0;
    const bool more = (t + 1 < ntiles);
    if (more) stage_load(j_begin + (t + 1) * G::JT);

    const float* kt = lds_k[buf];
    const float* vt = SEPV ? lds_v[vbuf] : lds_k[buf];

#pragma unroll
    for (int js = 0; js < G::NSUB; ++js) {
      // A operand of the logits MFMAs: key row (js*32+li), columns 8q+4h+t
      float ya[G::KK];
      const float* yrow = kt + (js * 32 + li) * G::LDW + 4 * h;
#pragma unroll
      for (int q = 0; q < G::NQ8; ++q) {
        const float4 v = *reinterpret_cast<const float4*>(yrow + 8 * q);
        ya[4 * q + 0] = v.x;
        ya[4 * q + 1] = v.y;
        ya[4 * q + 2] = v.z;
        ya[4 * q + 3] = v.w;
      }
      const float ab = h ? 1.0f : lds_b[buf][js * 32 + li];

      float vj[MODE == kVec ? 16 : 1];
      if constexpr (MODE == kVec) {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const float4 v =
              *reinterpret_cast<const float4*>(&lds_x[buf][js * 32 + 8 * q4 + 4 * h]);
          vj[4 * q4 + 0] = v.x;
          vj[4 * q4 + 1] = v.y;
          vj[4 * q4 + 2] = v.z;
          vj[4 * q4 + 3] = v.w;
        }
      }

#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < G::KK; ++kk)
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya[kk], xs[rb][kk], acc, 0, 0, 0);
        if constexpr (MODE == kArgmax) {
          // value = scaled dot + key bias; register r of a lane holds key 8 (r / 4) + 4 h + r % 4
          // of the sub-tile, ascending in r, and tiles ascend: a strict test keeps the
          // smallest key among equal values
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ab, h ? 0.0f : 1.0f, acc, 0, 0, 0);
          const int jb = j_begin + t * G::JT + js * 32 + 4 * h;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            if (acc[r] > run_m[rb]) {
              run_m[rb] = acc[r];
              best_j[rb] = jb + 8 * (r / 4) + (r % 4);
            }
          }
          continue;
        }
        // + key bias; the logits stay absolute and the running maximum is taken off in the
        // exponent (inside the accumulator it would cost them their digits whenever it lies far
        // below them, after a first tile of keys without weight, say)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ab, h ? 0.0f : 1.0f, acc, 0, 0, 0);

        f32x16 tacc;
        if constexpr (MODE == kMat5) {
#pragma unroll
          for (int r = 0; r < 16; ++r) tacc[r] = 0.f;
#pragma unroll
          for (int kk = 0; kk < G::KK; ++kk)
            tacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya[kk], x2s[rb][kk], tacc, 0, 0, 0);
        }

        float tmax = fmaxf(acc[0], acc[1]);
#pragma unroll
        for (int r = 2; r < 16; ++r) tmax = fmaxf(tmax, acc[r]);

        const bool first = (t == 0 && js == 0);
        if (first || wave_any(tmax - run_m[rb] > kLazyThresh)) {
          const float tm = fmaxf(tmax, xor32(tmax));
          const float m_new = (first || tm - run_m[rb] > kLazyThresh) ? tm : run_m[rb];
          const float resc = first ? 0.f : fast_exp2(run_m[rb] - m_new);
          run_m[rb] = m_new;
          run_s[rb] *= resc;
          run_o[rb] *= resc;
          if constexpr (kHasO) {
#pragma unroll
            for (int db = 0; db < G::NDB; ++db)
#pragma unroll
              for (int r = 0; r < 16; ++r) oacc[rb][db][r] *= resc;
          }
        }

        float p[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) p[r] = fast_exp2(acc[r] - run_m[rb]);

        if constexpr (MODE != kMat5) {
          float ps = 0.f;
#pragma unroll
          for (int r = 0; r < 16; ++r) ps += p[r];
          run_s[rb] += ps;
        }
        if constexpr (MODE == kVec) {
          float po = 0.f;
#pragma unroll
          for (int r = 0; r < 16; ++r) po += p[r] * vj[r];
          run_o[rb] += po;
        }
        if constexpr (MODE == kMat5) {
#pragma unroll
          for (int r = 0; r < 16; ++r) p[r] *= tacc[r];
        }
        if constexpr (kHasO) {
          // O^T[dd][i] += V[j][dd] * P^T[j][i]; register r of p holds key row
          // j = js*32 + 8*(r/4) + 4*h + (r%4), which is this lane's K slot.
#pragma unroll
          for (int db = 0; db < G::NDB; ++db) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const int jr = js * 32 + 8 * (r / 4) + 4 * h + (r % 4);
              const int col = db * 32 + li;
              const float va = (DP % 32 == 0 || col < DP) ? vt[jr * G::LDW + col] : 0.f;
              oacc[rb][db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va, p[r], oacc[rb][db], 0, 0, 0);
            }
          }
        }
      }
    }

    if (more) {
      if constexpr (SEPV && !G::VDB) __syncthreads();
      stage_store_k(buf ^ 1);
      stage_store_v(G::VDB ? (buf ^ 1) : 0);
    }
    __syncthreads();
  }

  // ---- merge the two half-waves of each query column, then finish or spill ----
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
          sd.ep.out[row] = -best;
          sd.ep.idx_out[row] = bj;
        } else {
          const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
          *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) =
              make_float2(best, __builtin_bit_cast(float, bj));
        }
      }
      continue;
    }
    const float M = run_m[rb];
    const float s = run_s[rb] + xor32(run_s[rb]);
    const float o = run_o[rb] + xor32(run_o[rb]);
    if (sd.splits == 1) {
      if constexpr (!kHasO) {
        if (live && h == 0) epilogue_scalar(sd.ep, row, M, s, o);
      } else {
        if (live) {
#pragma unroll
          for (int db = 0; db < G::NDB; ++db)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
              const int col = db * 32 + 8 * q4 + 4 * h;
              const float4 O = make_float4(oacc[rb][db][4 * q4], oacc[rb][db][4 * q4 + 1],
                                           oacc[rb][db][4 * q4 + 2], oacc[rb][db][4 * q4 + 3]);
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
        for (int db = 0; db < G::NDB; ++db)
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            const int col = db * 32 + 8 * q4 + 4 * h;
            if (DP % 32 == 0 || col < DP) {
              *reinterpret_cast<float4*>(&sd.part_o[pr * DP + col]) =
                  make_float4(oacc[rb][db][4 * q4], oacc[rb][db][4 * q4 + 1],
                              oacc[rb][db][4 * q4 + 2], oacc[rb][db][4 * q4 + 3]);
            }
          }
      }
    }
  }
}

template <bool HAS_O>
__device__ __forceinline__ void finish_rows(const LaunchArgs& args, int dp, int items0, int items1,
                                            float* sweep_l2);
__device__ __forceinline__ void sweep_step_merge(const LaunchArgs& args, int items0, int items1);

// Merge `splits` partial rows and run the epilogue.  One thread per output row
// (scalar kinds) or per 4 output columns (matrix kinds); grid covers both sides.
template <bool HAS_O>
__global__ __launch_bounds__(256) void finish_kernel(const LaunchArgs args, int dp, int items0,
                                                     int items1) {
  if constexpr (!HAS_O) {  // the launch that follows both variants of a device-chosen step
    if (args.sel != nullptr && blockIdx.x == 0 && threadIdx.x < 64) {
      // the sides of this launch that carry margins (the second one only when it has rows to merge)
      int role[2] = {0, 0};
      float ls[2] = {0.f, 0.f};
      const int commit_sides = args.side[0].margins == nullptr ? 0 : (items1 > 0 ? 2 : 1);
#pragma unroll
      for (int i = 0; i < 2; ++i)
        if (i < commit_sides) {
          const Side& ms = args.side[i];
          role[i] = ms.ps_q;
          ls[i] = ms.qscale / (ms.plane_scale[ms.ps_q] * ms.plane_scale[ms.ps_k]);
        }
      state_after_launch(args.sel, threadIdx.x, commit_sides, role, ls);
    }
  }
  if constexpr (!HAS_O) {
    // a step with a one-sweep launch (see lse_sweep_kernel); with the variant chosen on the
    // device that form belongs to the plain variant, and a step of the other one has nothing to
    // do with it
    if (args.sweep == 1 || (args.sweep == 2 && args.sel[kSelRan] == 1u)) {
      sweep_step_merge(args, items0, items1);
      return;
    }
  }
  finish_rows<HAS_O>(args, dp, items0, items1, nullptr);
}

// The merge itself.  sweep_l2 (may be null): receives log2 of what the row's sum would be with
// the row's own bias (as a key of the other side) inside the exponent, see lse_sweep_kernel.
template <bool HAS_O>
__device__ __forceinline__ void finish_rows(const LaunchArgs& args, int dp, int items0, int items1,
                                            float* sweep_l2) {
  int it = blockIdx.x * 256 + threadIdx.x;
  if (it >= items0 + items1) return;  // the other side may have nothing to merge
  const bool second = it >= items0;
  if (second) it -= items0;
  const Side& sd = second ? args.side[1] : args.side[0];
  const int per_row = HAS_O ? dp / 4 : 1;
  const int row = it / per_row;
  const int col = (it % per_row) * 4;
  if (row >= sd.nq) return;
  // lse_sparse_kernel wrote this side's partial results: per key range only as many as its
  // list had pieces (Side::npieces), in the range's first chunks
  bool by_range = false;
  if constexpr (!HAS_O)
    by_range = sd.npieces != nullptr && args.sel != nullptr && args.sel[kSelForm + sd.ps_q] == 2u;
  const int rgroup = by_range ? sd.sparse_group : 1;
  const int nranges = by_range ? (sd.splits + rgroup - 1) / rgroup : sd.splits;
  const unsigned char* np = by_range ? sd.npieces + (size_t)(row / 64) * nranges : nullptr;
  // (loops unrolled so that the loads of several key splits are in flight together: the merge
  // is a chain of memory round trips and nothing else)
  float M = -3.0e38f;
  if (!by_range) {
#pragma unroll 8
    for (int sp = 0; sp < sd.splits; ++sp)
      M = fmaxf(M, sd.part_ms[2 * ((size_t)sp * sd.nq + row)]);
  }
  float s = 0.f, o = 0.f;
  float4 O = make_float4(0.f, 0.f, 0.f, 0.f);
  if constexpr (HAS_O) {
    for (int sp = 0; sp < sd.splits; ++sp) {
      const size_t pr = (size_t)sp * sd.nq + row;
      const float w = exp2f(sd.part_ms[2 * pr] - M);
      s += w * sd.part_ms[2 * pr + 1];
      const float4 v = *reinterpret_cast<const float4*>(&sd.part_o[pr * dp + col]);
      O.x += w * v.x; O.y += w * v.y; O.z += w * v.z; O.w += w * v.w;
    }
    epilogue_vec4(sd.ep, sd.q, args.d, args.vec_ok != 0, row, col, M, s, O);
  } else {
    // the sums, and the key behind the largest partial maximum that a key of its chunk attained
    const bool keys = sd.best_key != nullptr && sd.part_best != nullptr;
    const bool has_o = sd.part_o != nullptr;
    float bm = -3.0e38f;
    int bj = -1;
    auto merge = [&](int sp) {
      const size_t pr = (size_t)sp * sd.nq + row;
      const float2 ms = *reinterpret_cast<const float2*>(&sd.part_ms[2 * pr]);
      const float w = exp2f(ms.x - M);
      s += w * ms.y;
      if (has_o) o += w * sd.part_o[pr];
      if (keys) {
        const int j = sd.part_best[pr];
        if (j >= 0 && ms.x > bm) {
          bm = ms.x;
          bj = j;
        }
      }
    };
    if (by_range) {
      // one pass, eight ranges at a time: the counts, and the first piece of every range (there
      // always is one), are loads that wait for nothing; further pieces are rare
      auto merge_online = [&](float2 ms, int j) {
        if (ms.x > M) {
          s = s * exp2f(M - ms.x) + ms.y;
          M = ms.x;
        } else {
          s += ms.y * exp2f(ms.x - M);
        }
        if (keys && j >= 0 && ms.x > bm) {
          bm = ms.x;
          bj = j;
        }
      };
      for (int r0 = 0; r0 < nranges; r0 += 8) {
        int cnt[8], pj[8];
        float2 first[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int r = min(r0 + i, nranges - 1);
          const size_t pr = (size_t)(r * rgroup) * sd.nq + row;
          cnt[i] = (r0 + i < nranges) ? (int)np[r] : 0;
          first[i] = *reinterpret_cast<const float2*>(&sd.part_ms[2 * pr]);
          pj[i] = keys ? sd.part_best[pr] : -1;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (r0 + i < nranges) merge_online(first[i], pj[i]);
#pragma unroll
        for (int i = 0; i < 8; ++i)
          for (int p = 1; p < cnt[i]; ++p) {
            const size_t pr = (size_t)((r0 + i) * rgroup + p) * sd.nq + row;
            merge_online(*reinterpret_cast<const float2*>(&sd.part_ms[2 * pr]), keys ? sd.part_best[pr] : -1);
          }
      }
    } else {
#pragma unroll 8
      for (int sp = 0; sp < sd.splits; ++sp) merge(sp);
    }
    if (keys && bj >= 0) sd.best_key[row] = bj;  // no chunk exceeded the starting value: the old key stays
    if (sd.m_prev != nullptr) sd.m_prev[row] = M;
    epilogue_scalar(sd.ep, row, M, s, o);
    if (sweep_l2 != nullptr) {
      // (the row's own bias as a key: of the other side, or of its own in a problem of a
      // matrix with itself)
      const Side& so = args.sweep_self ? sd : (second ? args.side[0] : args.side[1]);
      float b = so.kc0 * so.kb0[row];
      if (so.kb1 != nullptr) b += so.kc1 * so.kb1[row];
      if (so.kb2 != nullptr) b += so.kc2 * so.kb2[row];
      *sweep_l2 = (M + log2f(s)) + fmaxf(b, kNegBig);
    }
  }
}

// log2 of a row or column sum joins the step's extremes (kSelSweepHi / kSelSweepLo: float bits of
// non-negative numbers order like unsigned integers; anything that is not a number counts as
// out of every range).  One atomic per wavefront and slot.
__device__ __forceinline__ void sweep_note_sums(unsigned* st, float l2, bool live) {
  float hi = live ? fmaxf(l2, 0.f) : 0.f, lo = live ? fmaxf(-l2, 0.f) : 0.f;
  if (live && !(l2 == l2)) hi = lo = 3.0e38f;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    hi = fmaxf(hi, __shfl_xor(hi, o, 64));
    lo = fmaxf(lo, __shfl_xor(lo, o, 64));
  }
  if ((threadIdx.x & 63) == 0) {
    const int slot = (blockIdx.x * 4 + (threadIdx.x >> 6)) % kSweepSlots;
    if (hi > 0.f) atomicMax(&st[kSelSweepHi + slot], __builtin_bit_cast(unsigned, hi));
    if (lo > 0.f) atomicMax(&st[kSelSweepLo + slot], __builtin_bit_cast(unsigned, lo));
  }
}

// Did lse_sweep_kernel and its merge produce this step's results?  (Asked in a step of the
// plain variant only.)
__device__ __forceinline__ bool sweep_done(const LaunchArgs& args) {
  const unsigned* st = args.sel;
  return st[kSelSweep] != 0u && st[kSelSweepFail] == 0u;
}

// The last merge launch of a step that had a one-sweep launch.  If that launch produced the
// step's results there is nothing left to merge; else the two-sided kernel ran and its rows are
// merged here, each noting what its sum would have been in the one-sweep form.  The workgroup
// that finishes last turns the step's extremes into the permission for the next step.
__device__ __forceinline__ void sweep_step_merge(const LaunchArgs& args, int items0, int items1) {
  unsigned* st = args.sel;
  __shared__ int last;
  if (!sweep_done(args)) {
    float l2 = 0.f;
    bool live = false;
    {
      float v = __builtin_bit_cast(float, 0x7fc00000u);  // stays so for rows that wrote nothing
      const int it = blockIdx.x * 256 + threadIdx.x;
      live = it < items0 + items1;
      finish_rows<false>(args, 0, items0, items1, &v);
      l2 = v;
    }
    sweep_note_sums(st, l2, live);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    __threadfence();
    last = atomicAdd(&st[kSelSweepDone], 1u) == gridDim.x - 1 ? 1 : 0;
  }
  __syncthreads();
  if (last && threadIdx.x < 64) {
    __threadfence();
    const int lane = threadIdx.x;
    unsigned hi = 0u, lo = 0u;
    if (lane < kSweepSlots) {
      hi = __hip_atomic_load(&st[kSelSweepHi + lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      lo = __hip_atomic_load(&st[kSelSweepLo + lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      st[kSelSweepHi + lane] = 0u;
      st[kSelSweepLo + lane] = 0u;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      hi = max(hi, (unsigned)__shfl_xor((int)hi, o, 64));
      lo = max(lo, (unsigned)__shfl_xor((int)lo, o, 64));
    }
    if (lane == 0) {
      const bool ok = __builtin_bit_cast(float, hi) <= kSweepOkHi && __builtin_bit_cast(float, lo) <= -kSweepOkLo;
      st[kSelSweep] = ok ? 1u : 0u;
      st[kSelSweepLast] = hi;
      st[kSelSweepLast + 1] = lo;
      if (st[kSelSweepFail] != 0u) st[kSelSweepRedone] += 1u;
      st[kSelSweepFail] = 0u;
      st[kSelSweepDone] = 0u;
    }
  }
}

// The decision alone, for a step whose launch split no keys (no merge follows).
template <int T>
__global__ __launch_bounds__(64) void coarse_decide_kernel(unsigned* state) {
  const int role[2] = {0, 0};
  const float ls[2] = {0.f, 0.f};
  state_after_launch(state, threadIdx.x, 0, role, ls);
}

// kArgmax: merge the partial (largest value, key) pairs of the key splits; equal values keep
// the smaller key.  One thread per row; T only makes this a template (header-defined kernel).
template <int T>
__global__ __launch_bounds__(256) void finish_argmax_kernel(const LaunchArgs args) {
  const int row = blockIdx.x * 256 + threadIdx.x;
  const Side& sd = args.side[0];
  if (row >= sd.nq) return;
  float best = -3.0e38f;
  int bj = 0x7fffffff;
  for (int sp = 0; sp < sd.splits; ++sp) {
    const float2 v = *reinterpret_cast<const float2*>(&sd.part_ms[2 * ((size_t)sp * sd.nq + row)]);
    const int j = __builtin_bit_cast(int, v.y);
    if (v.x > best || (v.x == best && j < bj)) {
      best = v.x;
      bj = j;
    }
  }
  sd.ep.out[row] = -best * args.out_scale;
  sd.ep.idx_out[row] = bj;
}

}  // namespace fs
