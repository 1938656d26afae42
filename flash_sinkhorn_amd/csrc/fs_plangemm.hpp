// Plan-times-matrix products (gradient, apply_plan_mat, mat5) for large feature dimension
// (d > 128) on fp16 planes: out_i = epilogue( sum_j exp2(logit_ij - M_i) V_j ).
//
// A workgroup of 8 wavefronts owns 32 query rows and the output columns of one column group
// (8 * CB blocks of 32 columns, the whole row for d <= 256 * CB) and walks its key chunk in
// tiles of 256 keys.  Per tile:
//   1. logits: a k-loop over the feature axis in chunks of 32 columns, exactly the staging
//      scheme of lse_gemm_kernel (direct global->LDS loads of the chunked hi/lo planes, one
//      barrier per k-step) with 32 query rows + 256 key rows per stage and three stages, two
//      k-steps ahead: a k-step has only six MFMAs per wavefront to hide the loads behind;
//      wavefront w multiplies keys [32 w, 32 w + 32) of the tile against the 32 queries;
//   2. soft-max: the eight per-wavefront row maxima meet in LDS, every wavefront takes the
//      same (lazy) decision on the running maximum, exponentiates its 32 x 32 tile once and
//      leaves it in LDS as two fp16 planes, already in MFMA operand order;
//   3. values: O^T[cols, queries] += V^T[cols, keys] * P^T[keys, queries] with three fp16
//      products (hi*hi, hi*lo, lo*hi) per 16 keys; wavefront w owns CB column blocks and reads
//      its V^T operands straight from global memory, where transpose_planes_f16_kernel stored
//      them in operand order (one fully coalesced 1 KiB read per instruction).
// The fp32 sums of the probabilities stay exact (VALU); only the products run on fp16 planes,
// whose two-plane split carries 22 bits per value.
//
// MAT5 (sum_j P_ij <A_i, y_j> y_j): the k-loop also accumulates T = A K^T from planes of A
// staged next to the query rows, and the probabilities are multiplied by T before they go to
// LDS.  |T_ij| <= |A_i| max_j |y_j| (Cauchy-Schwarz), so a per-row power of two taken from
// that bound keeps |p T| within 2^15 whatever the data and as high in the fp16 range as a
// safe bound allows; it is divided out with the plane scales at the end.
//
// Operand order of the key axis: accumulator register 8 s + e (s = 0, 1; e = 0..7) of lane
// (li, h) of a 32 x 32 logits tile holds key 8 (2 s + e / 4) + 4 h + e % 4 of the block, so
// the lane's own registers 8 s .. 8 s + 7 are its B operand of 16-key step s, and the V^T
// planes store, for lane (li, h) of step s, exactly those eight keys of column li.
#pragma once

#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

constexpr int kPgKeys = 256;          // keys per tile
constexpr int kPgRows = 32;           // query rows per workgroup
constexpr float kPgLazyThresh = 4.0f; // exponentials stay below 2^4 relative to the running maximum
// exponentials are taken 2^11 up before the fp16 split and the reported maximum 11 down, as in
// plan_tile_kernel: a probability keeps a nonzero fp16 image down to 2^-35 of the row's largest
constexpr float kPgUp = 11.0f;

// Largest |rowscale[r] * src[r, c]| (rowscale may be null): one partial maximum per block.
__global__ __launch_bounds__(256) void absmax_rows_kernel(const float* __restrict__ src,
                                                          long long rows, int d,
                                                          const float* __restrict__ rowscale,
                                                          float* __restrict__ partial) {
  __shared__ float red[4];
  float m = 0.f;
  const long long cnt = rows * (long long)d;
  if ((d & 3) == 0 && (reinterpret_cast<size_t>(src) & 15) == 0) {
    // rows are whole float4 runs: one row lookup per four values
    const float4* s4 = reinterpret_cast<const float4*>(src);
    const int d4 = d >> 2;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < (cnt >> 2);
         i += 256LL * gridDim.x) {
      const float4 a = s4[i];
      float v = fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w)));
      if (rowscale) v *= fabsf(rowscale[i / d4]);
      m = fmaxf(m, v);
    }
  } else {
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < cnt; i += 256LL * gridDim.x) {
      float v = src[i];
      if (rowscale) v *= rowscale[i / d];
      m = fmaxf(m, fabsf(v));
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// v[rows, d] (fp32, optionally times rowscale[r]) -> two fp16 planes of scale * v, transposed
// into MFMA operand order: [key block of 32][column block of 32][step s][plane][lane] x 16 B,
// lane (li, h) holding keys 8 (2 s + e / 4) + 4 h + e % 4, e = 0..7, of column li.  nkb key
// blocks and ncb column blocks are written; rows >= `rows` and columns >= d are zero.
// gridDim.x * 4 wavefront units cover nkb * ncb * 2.  The scale comes from 256 partial maxima.
__global__ __launch_bounds__(256) void transpose_planes_f16_kernel(
    const float* __restrict__ src, const float* __restrict__ rowscale, unsigned* __restrict__ dst,
    int rows, int d, int nkb, int ncb, const float* __restrict__ partial_max,
    float* __restrict__ scale_out) {
  __shared__ float red[4];
  float m = partial_max[threadIdx.x];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  const float sc = f16_plane_scale(fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
  if (blockIdx.x == 0 && threadIdx.x == 0) *scale_out = sc;

  const long long unit = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= (long long)nkb * ncb * 2) return;
  const int lane = threadIdx.x & 63, li = lane & 31, h = lane >> 5;
  const int s = (int)(unit & 1);
  const int cb = (int)((unit >> 1) % ncb);
  const int kb = (int)((unit >> 1) / ncb);
  const int col = cb * 32 + li;
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int r = kb * 32 + 8 * (2 * s + e / 4) + 4 * h + (e % 4);
    float x = 0.f;
    if (r < rows && col < d) {
      x = src[(size_t)r * (size_t)d + col] * sc;
      if (rowscale) x *= rowscale[r];
    }
    v[e] = x;
  }
  unsigned hi[4], lo[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    hi[e] = pack_f16(v[2 * e], v[2 * e + 1]);
    const f16x2 a = __builtin_bit_cast(f16x2, hi[e]);
    lo[e] = pack_f16(v[2 * e] - (float)a[0], v[2 * e + 1] - (float)a[1]);
  }
  u32x4* o = reinterpret_cast<u32x4*>(dst) + (size_t)unit * 128 + lane;
  o[0] = u32x4{hi[0], hi[1], hi[2], hi[3]};
  o[64] = u32x4{lo[0], lo[1], lo[2], lo[3]};
}

// MAT5 helpers: out[r] = |src[r, :]|^2 (one wavefront per row), and 64 partial maxima of v.
__global__ __launch_bounds__(256) void rownorm2_kernel(const float* __restrict__ src, int rows,
                                                       int d, float* __restrict__ out) {
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const float* p = src + (size_t)r * (size_t)d;
  float s = 0.f;
  for (int c = threadIdx.x & 63; c < d; c += 64) s = __builtin_fmaf(p[c], p[c], s);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
  if ((threadIdx.x & 63) == 0) out[r] = s;
}

__global__ __launch_bounds__(256) void vecmax_kernel(const float* __restrict__ v, long long cnt,
                                                     float* __restrict__ out) {  // out[gridDim.x]
  __shared__ float red[4];
  float m = 0.f;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < cnt; i += 256LL * gridDim.x)
    m = fmaxf(m, v[i]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) out[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

template <int CB, bool MAT5>
__global__ __launch_bounds__(512, 1) void plan_gemm_kernel(const LaunchArgs args) {
  // stage rows: 32 query rows, (MAT5) 32 rows of the second stationary operand, 256 key rows
  constexpr int kKeyRow0 = MAT5 ? 2 * kPgRows : kPgRows;
  constexpr int kPgStageRows = kKeyRow0 + kPgKeys;
  __shared__ __attribute__((aligned(16))) unsigned lds[3][kPgStageRows * 32];
  __shared__ __attribute__((aligned(16))) u32x4 lds_p[8 * 2 * 2 * 64];  // [key block][s][plane][lane]
  __shared__ float lds_x[8][32];                                        // per-wavefront row statistics

  int bid = blockIdx.x;
  const bool second = bid >= args.blocks0;
  if (second) bid -= args.blocks0;
  const Side& sd = second ? args.side[1] : args.side[0];
  const int d = args.d;
  const int dp = args.pstride;  // words per row of the chunked planes
  const int nch = (d + 31) / 32;
  const int ncb = nch;                // column blocks of the V^T planes
  const int ncg = args.nss;           // column groups

  const int cg = bid % ncg;
  const int rest = bid / ncg;
  const int split = rest % sd.splits;
  const int ig = rest / sd.splits;
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int h = lane >> 5;
  const int row0 = ig * kPgRows;
  const int row = row0 + li;
  const int j_begin = split * sd.chunk;
  const int j_end = min(sd.nk, j_begin + sd.chunk);
  const int ntiles = (j_end > j_begin) ? (j_end - j_begin + kPgKeys - 1) / kPgKeys : 0;
  const int cb0 = (cg * 8 + wave) * CB;  // first column block of this wavefront

  const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = 1.0f / lscale;
  // MAT5: per-row power of two with |T_ij| * t_unit <= 1 from |T_ij| <= |A_i| max_j |y_j|
  // (in plane units; sd.q2norm2 = |A_i|^2, sd.kmax2 = 64 partial maxima of |y_j|^2, fp32 rows)
  float t_unit = 1.0f;
  if constexpr (MAT5) {
    const float a2 = (row < sd.nq) ? sd.q2norm2[row] : 0.f;
    float km = sd.kmax2[lane];  // 64 partial maxima
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) km = fmaxf(km, __shfl_xor(km, o, 64));
    const float bound = sqrtf(a2 * km) * sd.q2plane_scale[0] * sd.kplane_scale[0] * 1.0001f;
    const int e = (int)((__builtin_bit_cast(unsigned, bound) >> 23) & 255u);  // bound < 2^(e-126)
    if (e > 0 && e < 255) t_unit = __builtin_bit_cast(float, (unsigned)min(254, max(1, 127 - (e - 126))) << 23);
  }

  // ---- loaders: wavefront w brings key rows [32 w, 32 w + 32) of the tile (4 instructions of
  // 8 rows), wavefronts 0-3 also 8 query rows each, wavefronts 4-7 (MAT5) 8 rows of A ----
  int koff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int lr = wave * 32 + i * 8 + (lane >> 3);
    koff[i] = lr * dp + (((lane & 7) ^ ((lr >> 1) & 7)) << 2);
  }
  const int qlr = (wave & 3) * 8 + (lane >> 3);
  const unsigned* qsrc = ((MAT5 && wave >= 4) ? sd.q2planes : sd.qplanes) +
                         (size_t)(row0 + qlr) * (size_t)dp + (((lane & 7) ^ ((qlr >> 1) & 7)) << 2);
  auto issue_loads = [&](int buf, int j0, int c) {
    const unsigned* kbase = sd.kplanes + (size_t)j0 * (size_t)dp + c * 32;
    unsigned* kdst = &lds[buf][(kKeyRow0 + wave * 32) * 32];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(kbase + koff[i]),
          (__attribute__((address_space(3))) void*)(kdst + i * 8 * 32), 16, 0, 0);
    if (MAT5 || wave < 4)  // rows 0-31 queries, 32-63 second operand: wavefront w fills 8 w ..
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(qsrc + c * 32),
          (__attribute__((address_space(3))) void*)(&lds[buf][(wave * 8) * 32]), 16, 0, 0);
  };
  // Stage reads are ds_read_b128 written out by hand: the compiler cannot tell a read of one
  // stage buffer from the global->LDS loads filling the others and would make every read wait
  // for all of them, which leaves the three-stage ring no load in flight across a k-step.  It
  // does not see these reads either: their consumers sit behind wait_lds().
  auto lds_piece = [&](const unsigned* stage, int r, int p) {
    u32x4 v;
    const unsigned addr = (unsigned)(size_t)(const __attribute__((address_space(3))) unsigned*)(
        stage + r * 32 + ((p ^ ((r >> 1) & 7)) << 2));
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
  };
  auto wait_lds = [&]() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- V^T operands: unit (key block, column block, s) = 128 pieces of 16 bytes ----
  const u32x4* vt = reinterpret_cast<const u32x4*>(sd.vplanes);
  int cbc[CB];  // column blocks past the last one re-read it; their output is never stored
#pragma unroll
  for (int i = 0; i < CB; ++i) cbc[i] = min(cb0 + i, ncb - 1);
  auto load_vt = [&](u32x4 (&a)[CB][2], int kb, int s) {
#pragma unroll
    for (int i = 0; i < CB; ++i) {
      const u32x4* p = vt + (((size_t)kb * (size_t)ncb + (size_t)cbc[i]) * 2 + s) * 128 + lane;
      a[i][0] = p[0];
      a[i][1] = p[64];
    }
  };

  f32x16 oacc[CB];
#pragma unroll
  for (int i = 0; i < CB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[i][r] = 0.f;
  // run_c: the constant of the exponentials, kPgUp minus the running maximum in base-2 units
  // (the logits stay in absolute raw units: see plan_tile_kernel)
  float run_c = kPgUp, run_s = 0.f;

  auto swap_halves = [&](float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  };

  // Three stage buffers: the loads of k-step g + 2 are issued at k-step g (their buffer was
  // read at step g - 1, which every wavefront has left), so a stage has two steps to arrive.
  // The sequence of steps runs across tiles; (lt, lc) is the next (tile, chunk) to load.
  const int nsteps = ntiles * nch;
  int lt = 0, lc = 0, lbuf = 0, issued = 0;
  auto issue_next = [&]() {
    if (issued < nsteps) {
      issue_loads(lbuf, j_begin + lt * kPgKeys, lc);
      lbuf = (lbuf == 2) ? 0 : lbuf + 1;
      if (++lc == nch) {
        lc = 0;
        ++lt;
      }
    }
    ++issued;
  };
  // at most the loads of the newest stage stay in flight (5 per wavefront, 4 for wavefronts
  // 4-7 when there is no second stationary operand)
  auto wait_stage = [&]() {
    if (issued > nsteps) {
      __builtin_amdgcn_s_waitcnt(0x0F70);
    } else if (MAT5 || wave < 4) {
      __builtin_amdgcn_s_waitcnt(0x0F70 | 5);
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
    }
  };
  issue_next();
  issue_next();
  wait_stage();
  __syncthreads();

  int buf = 0;
  for (int t = 0; t < ntiles; ++t) {
    const int j0 = j_begin + t * kPgKeys;
    f32x16 acc, acc2, tacc;  // one T accumulator: registers are short with CB = 6
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[r] = 0.f;
      acc2[r] = 0.f;
      tacc[r] = 0.f;
    }
    // ---- 1. logits of keys [32 wave, 32 wave + 32) x 32 queries ----
    for (int c = 0; c < nch; ++c) {
      issue_next();
      const unsigned* stage = lds[buf];
      u32x4 qr[2][2], kr[2][2];  // [plane][16-column half]
#pragma unroll
      for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          qr[p][kk] = lds_piece(stage, li, p * 4 + kk * 2 + h);
          kr[p][kk] = lds_piece(stage, kKeyRow0 + wave * 32 + li, p * 4 + kk * 2 + h);
        }
      u32x4 ar[MAT5 ? 2 : 1][2];
      if constexpr (MAT5) {
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) ar[p][kk] = lds_piece(stage, kPgRows + li, p * 4 + kk * 2 + h);
      }
      wait_lds();
#pragma unroll
      for (int prod = 0; prod < 3; ++prod) {
        const int pk = (prod == 0) ? 1 : 0, pq = (prod == 1) ? 1 : 0;
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kr[pk][0]),
                                                     __builtin_bit_cast(f16x8, qr[pq][0]), acc, 0, 0, 0);
        acc2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kr[pk][1]),
                                                      __builtin_bit_cast(f16x8, qr[pq][1]), acc2, 0, 0, 0);
      }
      if constexpr (MAT5) {
#pragma unroll
        for (int prod = 0; prod < 3; ++prod) {
          const int pk = (prod == 0) ? 1 : 0, pq = (prod == 1) ? 1 : 0;
          tacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kr[pk][0]),
                                                        __builtin_bit_cast(f16x8, ar[pq][0]), tacc, 0, 0, 0);
          tacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, kr[pk][1]),
                                                        __builtin_bit_cast(f16x8, ar[pq][1]), tacc, 0, 0, 0);
        }
      }
      // this wavefront's direct loads of the next stage have landed; the stage after it stays
      // in flight across the barrier (a bare s_barrier: __syncthreads() carries a release
      // fence, for which the compiler waits for every outstanding global->LDS load)
      wait_stage();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      buf = (buf == 2) ? 0 : buf + 1;
    }

    // first V^T operands of the tile travel while the soft-max runs
    const int kb0 = j0 >> 5;
    u32x4 va[CB][2];
    load_vt(va, kb0, 0);
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. bias - M fold, shared running maximum, probabilities into LDS ----
    {
      const float ab =
          h ? 1.0f : fmaxf(key_bias(sd, j0 + wave * 32 + li, j_end) * inv_lscale, -3.0e38f);
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] += acc2[r];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ab, h ? 0.0f : 1.0f, acc, 0, 0, 0);
    }
    float m = acc[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) m = fmaxf(m, acc[r]);
    {
      float a = m, b = m;
      swap_halves(a, b);
      m = fmaxf(a, b);
    }
    if (h == 0) lds_x[wave][li] = m;
    __syncthreads();
    float tm = lds_x[0][li];
#pragma unroll
    for (int w = 1; w < 8; ++w) tm = fmaxf(tm, lds_x[w][li]);
    const bool first = (t == 0);
    const bool up = first || (__builtin_fmaf(tm, lscale, run_c) > kPgLazyThresh + kPgUp);
    if (first || wave_any(up)) {  // the same lanes vote in every wavefront
      const float c_new = up ? __builtin_fmaf(-tm, lscale, kPgUp) : run_c;
      const float resc = first ? 0.f : fast_exp2(c_new - run_c);
      run_c = c_new;
      run_s *= resc;
#pragma unroll
      for (int i = 0; i < CB; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[i][r] *= resc;
    }
    float p[16];
    float ps = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      p[r] = fast_exp2(__builtin_fmaf(acc[r], lscale, run_c));
      ps += p[r];
    }
    run_s += ps;
    if constexpr (MAT5) {
#pragma unroll
      for (int r = 0; r < 16; ++r) p[r] *= tacc[r] * t_unit;
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      unsigned hi[4], lo[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float x0 = p[8 * s + 2 * e], x1 = p[8 * s + 2 * e + 1];
        hi[e] = pack_f16(x0, x1);
        const f16x2 a = __builtin_bit_cast(f16x2, hi[e]);
        lo[e] = pack_f16(x0 - (float)a[0], x1 - (float)a[1]);
      }
      lds_p[((wave * 2 + s) * 2 + 0) * 64 + lane] = u32x4{hi[0], hi[1], hi[2], hi[3]};
      lds_p[((wave * 2 + s) * 2 + 1) * 64 + lane] = u32x4{lo[0], lo[1], lo[2], lo[3]};
    }
    __syncthreads();

    // ---- 3. O^T += V^T P^T over the 16 steps of 16 keys, operands one step ahead ----
#pragma unroll
    for (int st = 0; st < 16; ++st) {
      u32x4 vn[CB][2];
      if (st + 1 < 16) load_vt(vn, kb0 + ((st + 1) >> 1), (st + 1) & 1);
      // the loads of the next step stay ahead of this step's MFMAs (the compiler would sink
      // them to their first use to save registers, and every MFMA would wait for memory)
      __builtin_amdgcn_sched_barrier(0);
      const u32x4 bh = lds_p[(st * 2 + 0) * 64 + lane];
      const u32x4 bl = lds_p[(st * 2 + 1) * 64 + lane];
#pragma unroll
      for (int i = 0; i < CB; ++i) {
        oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, va[i][1]),
                                                         __builtin_bit_cast(f16x8, bh), oacc[i], 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < CB; ++i) {
        oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, va[i][0]),
                                                         __builtin_bit_cast(f16x8, bl), oacc[i], 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < CB; ++i) {
        oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, va[i][0]),
                                                         __builtin_bit_cast(f16x8, bh), oacc[i], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (st + 1 < 16) {
#pragma unroll
        for (int i = 0; i < CB; ++i) {
          va[i][0] = vn[i][0];
          va[i][1] = vn[i][1];
        }
      }
    }
  }

  // ---- row sums of all wavefronts, then finish or spill ----
  __syncthreads();
  {
    const float sw = run_s + xor32(run_s);
    if (h == 0) lds_x[wave][li] = sw;
  }
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < 8; ++w) s += lds_x[w][li];
  const float M = (ntiles > 0) ? -run_c : kNegBig;
  float inv_vs = 1.0f / sd.vplane_scale[0];
  if constexpr (MAT5) inv_vs /= t_unit * sd.q2plane_scale[0] * sd.kplane_scale[0];
  const bool live = row < sd.nq;
  const bool vec_ok = args.vec_ok != 0;
  if (sd.splits == 1) {
    if (live) {
#pragma unroll
      for (int i = 0; i < CB; ++i)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int col = (cb0 + i) * 32 + 8 * q4 + 4 * h;
          const float4 O = make_float4(oacc[i][4 * q4] * inv_vs, oacc[i][4 * q4 + 1] * inv_vs,
                                       oacc[i][4 * q4 + 2] * inv_vs, oacc[i][4 * q4 + 3] * inv_vs);
          epilogue_vec4(sd.ep, sd.q, d, vec_ok, row, col, M, s, O);
        }
    }
  } else if (live) {
    const size_t pr = (size_t)split * (size_t)sd.nq + (size_t)row;
    const size_t dpo = (size_t)ncg * 8 * CB * 32;  // row stride of the partial outputs
    if (wave == 0 && h == 0 && cg == 0)
      *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(M, s);
#pragma unroll
    for (int i = 0; i < CB; ++i)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int col = (cb0 + i) * 32 + 8 * q4 + 4 * h;
        *reinterpret_cast<float4*>(&sd.part_o[pr * dpo + col]) =
            make_float4(oacc[i][4 * q4] * inv_vs, oacc[i][4 * q4 + 1] * inv_vs,
                        oacc[i][4 * q4 + 2] * inv_vs, oacc[i][4 * q4 + 3] * inv_vs);
      }
  }
}

}  // namespace fs
