// Plan kernels for large feature dimension (d > 128, fp32 MFMA).
//
// A workgroup of NW wavefronts owns ONE block of 32 query rows and splits the
// feature axis into NW column slices of NSL*32 columns.  Wavefront w keeps its
// slice of the query rows in VGPRs and, for the matrix kinds, its slice of the
// output accumulator O^T (NSL blocks of 32x32).  Per tile of 32 keys:
//   1. every wavefront contracts its column slice: partial S^T (keys x queries);
//   2. the NW partial tiles are summed through LDS (double buffered, one
//      barrier per tile); every wavefront then holds the full logits tile and
//      runs the same lane-private online soft-max, so they all agree on M;
//   3. the exp'ed tile is the B operand of the second contraction against this
//      wavefront's column slice of the value rows.
// Nothing of size n x m, and no accumulator, ever goes to global memory; the
// soft-max work is replicated NW times, which is noise next to d/2 MFMAs.
// Key and value rows are read straight from global memory (L2-resident across
// the workgroups of an XCD, which sweep the keys in the same order).
// A workgroup spans NW*NSL*32 columns (1536 at most).  Wider rows are cut into `nss`
// super-slices of that width: every workgroup contracts ALL super-slices for the logits
// (its own one from registers, the others with the query rows re-read per tile), and for the
// matrix kinds the grid is multiplied by nss, workgroup ss accumulating and writing the
// output columns of super-slice ss only.
#pragma once

#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

template <int MODE, int NW, int NSL, bool STAT, bool MULTI>
__global__ __launch_bounds__(NW * 64) void sliced_kernel(const LaunchArgs args) {
  constexpr bool kHasO = (MODE == kMat || MODE == kMat5);
  constexpr int SW = NSL * 32;  // slice width in columns
  constexpr int NQ8 = SW / 8;
  constexpr int KK = SW / 2;

  __shared__ __attribute__((aligned(16))) float lds_p[2][NW * 16 * 64];
  __shared__ __attribute__((aligned(16))) float lds_t[MODE == kMat5 ? 2 : 1]
                                                     [MODE == kMat5 ? NW * 16 * 64 : 4];

  int bid = blockIdx.x;
  const bool second = bid >= args.blocks0;
  if (second) bid -= args.blocks0;
  const Side& sd = second ? args.side[1] : args.side[0];
  const int d = args.d;
  const bool vec_ok = args.vec_ok != 0;

  const int nss = MULTI ? args.nss : 1;      // column super-slices of the logits contraction
  const int ss_own = kHasO ? bid % nss : 0;  // the one whose output columns this workgroup owns
  if (kHasO) bid /= nss;
  const int split = bid % sd.splits;
  const int ig = bid / sd.splits;
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int h = lane >> 5;
  const int row = ig * 32 + li;
  const int c0 = ss_own * (NW * SW) + wave * SW;
  const int j_begin = split * sd.chunk;
  const int j_end = min(sd.nk, j_begin + sd.chunk);
  const int ntiles = (j_end - j_begin + 31) / 32;
  const float* vrows = (MODE == kMat && sd.v) ? sd.v : sd.k;

  float qs[STAT ? KK : 1];
  if constexpr (STAT) {
#pragma unroll
    for (int q = 0; q < NQ8; ++q) {
      const float4 v = load_row4(sd.q, row, sd.nq, c0 + 8 * q + 4 * h, d, vec_ok);
      qs[4 * q + 0] = v.x * sd.qscale;
      qs[4 * q + 1] = v.y * sd.qscale;
      qs[4 * q + 2] = v.z * sd.qscale;
      qs[4 * q + 3] = v.w * sd.qscale;
    }
  }

  float run_m = 0.f, run_s = 0.f, run_o = 0.f;
  f32x16 oacc[kHasO ? NSL : 1];
  if constexpr (kHasO) {
#pragma unroll
    for (int db = 0; db < NSL; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  }

  for (int t = 0; t < ntiles; ++t) {
    const int j0 = j_begin + t * 32;
    const int buf = t & 1;

    // ---- partial logits over this wavefront's column slice ----
    f32x16 acc, tacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[r] = 0.f;
      tacc[r] = 0.f;
    }
    for (int ss = 0; ss < nss; ++ss) {
      const int cs0 = ss * (NW * SW) + wave * SW;
      const bool own = (ss == ss_own);
#pragma unroll
      for (int q = 0; q < NQ8; ++q) {
        const int col = cs0 + 8 * q + 4 * h;
        const float4 ya = load_row4(sd.k, j0 + li, j_end, col, d, vec_ok);
        float4 xb;
        if (STAT && own) {
          xb = make_float4(qs[4 * q], qs[4 * q + 1], qs[4 * q + 2], qs[4 * q + 3]);
        } else {
          const float4 v = load_row4(sd.q, row, sd.nq, col, d, vec_ok);
          xb = make_float4(v.x * sd.qscale, v.y * sd.qscale, v.z * sd.qscale, v.w * sd.qscale);
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya.x, xb.x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya.y, xb.y, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya.z, xb.z, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya.w, xb.w, acc, 0, 0, 0);
        if constexpr (MODE == kMat5) {
          const float4 u = load_row4(sd.q2, row, sd.nq, col, d, vec_ok);
          tacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya.x, u.x, tacc, 0, 0, 0);
          tacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya.y, u.y, tacc, 0, 0, 0);
          tacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya.z, u.z, tacc, 0, 0, 0);
          tacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ya.w, u.w, tacc, 0, 0, 0);
        }
        // keep at most a few row loads in flight: the slice is register-heavy already
        if (q % 4 == 3) __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (wave == 0) {
      const float ab = h ? 1.0f : key_bias(sd, j0 + li, j_end);
      // (+ key bias; the running maximum is taken off in the exponent: see stream_kernel)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ab, h ? 0.0f : 1.0f, acc, 0, 0, 0);
    }

    // ---- sum the NW partial tiles through LDS ----
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      *reinterpret_cast<float4*>(&lds_p[buf][((wave * 4 + q4) * 64 + lane) * 4]) =
          make_float4(acc[4 * q4], acc[4 * q4 + 1], acc[4 * q4 + 2], acc[4 * q4 + 3]);
      if constexpr (MODE == kMat5)
        *reinterpret_cast<float4*>(&lds_t[buf][((wave * 4 + q4) * 64 + lane) * 4]) =
            make_float4(tacc[4 * q4], tacc[4 * q4 + 1], tacc[4 * q4 + 2], tacc[4 * q4 + 3]);
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[r] = 0.f;
      tacc[r] = 0.f;
    }
#pragma unroll
    for (int w = 0; w < NW; ++w) {
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const float4 v =
            *reinterpret_cast<const float4*>(&lds_p[buf][((w * 4 + q4) * 64 + lane) * 4]);
        acc[4 * q4] += v.x;
        acc[4 * q4 + 1] += v.y;
        acc[4 * q4 + 2] += v.z;
        acc[4 * q4 + 3] += v.w;
        if constexpr (MODE == kMat5) {
          const float4 u =
              *reinterpret_cast<const float4*>(&lds_t[buf][((w * 4 + q4) * 64 + lane) * 4]);
          tacc[4 * q4] += u.x;
          tacc[4 * q4 + 1] += u.y;
          tacc[4 * q4 + 2] += u.z;
          tacc[4 * q4 + 3] += u.w;
        }
      }
    }

    // ---- lane-private online soft-max (identical in every wavefront) ----
    float tmax = fmaxf(acc[0], acc[1]);
#pragma unroll
    for (int r = 2; r < 16; ++r) tmax = fmaxf(tmax, acc[r]);
    const bool first = (t == 0);
    if (first || wave_any(tmax - run_m > kLazyThresh)) {
      const float tm = fmaxf(tmax, xor32(tmax));
      const float m_new = (first || tm - run_m > kLazyThresh) ? tm : run_m;
      const float resc = first ? 0.f : fast_exp2(run_m - m_new);
      run_m = m_new;
      run_s *= resc;
      run_o *= resc;
      if constexpr (kHasO) {
#pragma unroll
        for (int db = 0; db < NSL; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[db][r] *= resc;
      }
    }
    float p[16];
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      p[r] = fast_exp2(acc[r] - run_m);
      ps += p[r];
    }
    run_s += ps;
    if constexpr (MODE == kVec) {
      float po = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = j0 + 8 * (r / 4) + 4 * h + (r % 4);
        po += p[r] * ((j < j_end) ? sd.v[j] : 0.f);
      }
      run_o += po;
    }
    if constexpr (MODE == kMat5) {
#pragma unroll
      for (int r = 0; r < 16; ++r) p[r] *= tacc[r];
    }
    if constexpr (MODE == kMat) {
      if (sd.vscale) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = j0 + 8 * (r / 4) + 4 * h + (r % 4);
          p[r] *= (j < j_end) ? sd.vscale[j] : 0.f;
        }
      }
    }

    // ---- O^T slice += V^T slice * P^T ----
    if constexpr (kHasO) {
#pragma unroll
      for (int db = 0; db < NSL; ++db) {
        const int col = c0 + db * 32 + li;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = j0 + 8 * (r / 4) + 4 * h + (r % 4);
          const float va = (j < j_end && col < d) ? vrows[(size_t)j * (size_t)d + col] : 0.f;
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(va, p[r], oacc[db], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // ---- finish or spill (statistics are identical in all wavefronts) ----
  const float M = run_m;
  const float s = run_s + xor32(run_s);
  const float o = run_o + xor32(run_o);
  const bool live = row < sd.nq;
  const int DPF = nss * NW * SW;  // padded feature width of the partial buffers
  if (sd.splits == 1) {
    if constexpr (!kHasO) {
      if (live && wave == 0 && h == 0) epilogue_scalar(sd.ep, row, M, s, o);
    } else if (live) {
#pragma unroll
      for (int db = 0; db < NSL; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int col = c0 + db * 32 + 8 * q4 + 4 * h;
          const float4 O = make_float4(oacc[db][4 * q4], oacc[db][4 * q4 + 1],
                                       oacc[db][4 * q4 + 2], oacc[db][4 * q4 + 3]);
          epilogue_vec4(sd.ep, sd.q, d, vec_ok, row, col, M, s, O);
        }
    }
  } else if (live) {
    const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
    if (wave == 0 && h == 0 && ss_own == 0) {
      *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(M, s);
      if constexpr (MODE == kVec) sd.part_o[pr] = o;
    }
    if constexpr (kHasO) {
#pragma unroll
      for (int db = 0; db < NSL; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int col = c0 + db * 32 + 8 * q4 + 4 * h;
          *reinterpret_cast<float4*>(&sd.part_o[pr * (size_t)DPF + col]) =
              make_float4(oacc[db][4 * q4], oacc[db][4 * q4 + 1], oacc[db][4 * q4 + 2],
                          oacc[db][4 * q4 + 3]);
        }
    }
  }
}

}  // namespace fs
