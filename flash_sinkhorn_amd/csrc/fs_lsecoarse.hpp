// Log-sum-exp kernel with the coarse tile test as a software pipeline (fp16 planes, d <= 64).
//
// Operands are two fp16 planes (hi, lo) per matrix; a logit needs the three plane products
// hi*hi + hi*lo + lo*hi.  The hi*hi product alone (a third of the MFMAs) already tells whether
// a 32 x 32 logits tile can matter: with B_i a bound on the two cross products of query row i
// (it needs no look at the keys, see `corr` below) and b~_j an upper bound of the key bias,
//     hi*hi_ij + b~_j + B_i  <  M_i - 2^40 distance   for every i, j of the tile
// means no logit of the tile could change the fp32 row sums, and the tile ends there.
// The bias bound rides in the same MFMA chain: b~_j = bmax + 2^18 a_j with bmax the largest
// bias of the 32-key sub-tile and a_j <= 0 one fp16 number per key, (b_j - bmax) / 2^18 rounded
// towards zero, multiplied in by one more 16-column MFMA step (keys: eight copies of a_j,
// queries: eight times 2^15); bmax itself moves to the other side of the comparison.  A unit
// that goes on gets b_j - 2^18 a_j added in fp32, which restores the exact bias.
//
// A wavefront owns 64 query rows (two blocks of 32) whose planes stay in registers, and walks
// its key chunk in 32-key sub-tiles ("unit": 32 keys x 32 queries).  One step per sub-tile s:
//   1. the hi*hi products of the two units of sub-tile s+1 go to the matrix pipe (the a_j step,
//      then two independent chains of four MFMAs), and between them in program order sit
//   2. the tests of the two units of sub-tile s, whose products finished during the last step:
//      a wavefront issues in order, so only work placed between MFMAs runs in their shadow;
//   3. for a unit of s that goes on, in a block of its own: the cross products khi*qlo and
//      klo*qhi and the exact key bias (one fp32 MFMA) on top of its hi*hi product, then the
//      soft-max.
// Nothing a conditional block computes outlives it except the running (maximum, sum) of the
// rows and the key of the maximum: no accumulator tile is carried across a branch, so the
// register allocator never has to reconcile two versions of one (four tiles hold the hi*hi
// products of two sub-tiles, and they are only ever written unconditionally).  Key tiles hold
// hi planes only (128 keys, 16 KiB at 64 columns, ring of four, three tiles ahead, one barrier
// per tile): the few units that go on read the hi plane and the per-key biases of their
// sub-tile again from LDS and fetch the lo plane from global memory.  A unit that ends costs
// four and a half MFMAs (the a_j step serves both row blocks), a 16-value maximum and a ballot.
//
// What the test can end depends on where a row's running maximum starts.  The launch keeps,
// per row, the key that held the row's largest logit (Side::best_key, merged over the key
// chunks by finish_kernel), and the next launch over the same planes starts the row from its
// current logit at that key: a lower bound of the new maximum by construction, and the maximum
// itself once the potentials settle.  Rows without a key (the first launch on new planes)
// start from the largest logit of 64 keys sampled evenly over the whole key set, so that a key
// chunk without any of the row's near keys is measured against a meaningful maximum from its
// first tile on.  The key-side quantities of the test (a_j, b_j - 2^18 a_j, bmax per sub-tile)
// are the same for every workgroup: coarse_bias_kernel writes them once per launch, one record
// per 64 keys, in the layout the records take in LDS.
//
// Everything LDS-related is written out by hand (ds_read / ds_write / s_waitcnt / s_barrier):
// key tiles arrive by direct global->LDS loads three tiles ahead, and the compiler, which
// cannot tell a read of one ring buffer from the loads still filling another, would make
// every LDS access wait for all of them.
#pragma once

#include <type_traits>

#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

#define FS_LC_FENCE() __builtin_amdgcn_sched_barrier(0)

// What lse_coarse_kernel needs of the key bias, once per launch instead of once per workgroup:
// one wavefront per 64-key tile writes the tile's record (layout: kAux* in fs_common.hpp) in raw
// units: a_j as eight fp16 copies, b_j - 2^18 a_j, and the largest bias of each 32-key
// sub-tile.  Keys past the end of the key set get a bias that masks them.  T only makes this a
// template (header-defined kernel).
//
// The blocks behind the tiles (8 query rows each, side 0 first: seed_blocks0 of them) compute
// where the rows' running maxima start.  A row whose largest logit of the last launch sat at key
// j starts from its current logit at j, computed on the vector pipe from the same planes:
// whatever the potentials did since, this is a logit of the row, hence a lower bound of its new
// maximum, and close to it once the potentials settle.  (Any index inside the key set keeps the
// result exact; a stale one only costs tests that pass.)  The sum of the fp32 roundings of the
// two routes to a logit is far below 1/64 of the row's bound on its cross products, which is taken
// off together with one base-2 unit.  A row without a key gets -3e38.
template <int T>
__global__ __launch_bounds__(64) void coarse_bias_kernel(const LaunchArgs args, int tiles0, int tiles_all,
                                                         int seed_blocks0, int dp) {
  // variant chosen on the device: nothing reads the records when the plain kernel runs
  if (args.sel_pred && args.sel[kSelWord] != 0u) return;
  if (args.sweep && blockIdx.x == 0 && threadIdx.x == 0) args.sel[kSelRan] = 0u;
  if (args.queue != nullptr)  // lse_sparse_kernel's work queues start empty
    for (int i = blockIdx.x * 64 + threadIdx.x; i < 2 * 8 * kQueueWords; i += gridDim.x * 64)
      args.queue[i] = 0u;
  if ((int)blockIdx.x >= tiles_all) {
    int blk = blockIdx.x - tiles_all;
    const bool second_s = blk >= seed_blocks0;
    if (second_s) blk -= seed_blocks0;
    const Side& ss = second_s ? args.side[1] : args.side[0];
    if (ss.seed == nullptr) return;
    // eight lanes per row, 16 bytes of each plane per lane and 64-column piece of the row (whole
    // cache lines per row); one short wavefront per eight rows, so that the launch is as long as
    // one chain of loads
    const int lane = threadIdx.x, piece = lane & 7, sub = lane >> 3;
    const float inv_ls = ss.plane_scale[ss.ps_q] * ss.plane_scale[ss.ps_k] / ss.qscale;
    {
      const int row = blk * 8 + sub;
      const int rc = min(row, ss.nq - 1);
      const int j = ss.best_key[rc];
      const int jc = min(max(j, 0), ss.nk - 1);
      float b = ss.kc0 * ss.kb0[jc];  // (every lane of the row: the loads go out with the planes')
      if (ss.kb1) b += ss.kc1 * ss.kb1[jc];
      if (ss.kb2) b += ss.kc2 * ss.kb2[jc];
      float dot = 0.f, l1 = 0.f;
      // words [w0, w0 + 4) of each plane: rows wider than 64 columns take more than one round
      for (int w0 = piece * 4; w0 < dp / 2; w0 += 32) {
        const unsigned* q = ss.qplanes + (size_t)rc * (size_t)dp + w0;
        const unsigned* k = ss.kplanes + (size_t)jc * (size_t)dp + w0;
        const u32x4 qh4 = *reinterpret_cast<const u32x4*>(q);
        const u32x4 ql4 = *reinterpret_cast<const u32x4*>(q + dp / 2);
        const u32x4 kh4 = *reinterpret_cast<const u32x4*>(k);
        const u32x4 kl4 = *reinterpret_cast<const u32x4*>(k + dp / 2);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // (words copied out first: a bit cast applied to a vector element reads element 0)
          const unsigned qhw = qh4[e], qlw = ql4[e], khw = kh4[e], klw = kl4[e];
          const f16x2 qh = __builtin_bit_cast(f16x2, qhw), ql = __builtin_bit_cast(f16x2, qlw);
          const f16x2 kh = __builtin_bit_cast(f16x2, khw), kl = __builtin_bit_cast(f16x2, klw);
          dot = __builtin_amdgcn_fdot2(kh, qh, dot, false);
          dot = __builtin_amdgcn_fdot2(kh, ql, dot, false);
          dot = __builtin_amdgcn_fdot2(kl, qh, dot, false);
          l1 += fabsf((float)qh[0]) + fabsf((float)qh[1]);
        }
      }
#pragma unroll
      for (int o = 4; o > 0; o >>= 1) {
        dot += __shfl_xor(dot, o, 64);
        l1 += __shfl_xor(l1, o, 64);
      }
      if (piece == 0 && row < ss.nq) {
        float w = -3.0e38f;
        // a key that is masked out (bias at the stand-in for -inf) says nothing about the row
        if (j >= 0 && b > 0.5f * kNegBig) {
          const float corr = 24.5f * l1 + (float)dp * 0x1p-9f + inv_ls;  // as in lse_coarse_kernel
          b = fmaxf(fmaxf(b, kNegBig) * inv_ls, -3.0e38f);
          w = fmaxf(dot + b - (corr * 0x1p-6f + inv_ls), -3.0e38f);
        }
        ss.seed[row] = w;
      }
    }
    return;
  }
  int tile = blockIdx.x;
  const bool second = tile >= tiles0;
  if (second) tile -= tiles0;
  const Side& sd = second ? args.side[1] : args.side[0];
  const int lane = threadIdx.x, li = lane & 31, h = lane >> 5;
  const int j = tile * 64 + lane;
  const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = 1.0f / lscale;
  float b = 2.0f * kNegBig;
  if (j < sd.nk) {
    b = sd.kc0 * sd.kb0[j];
    if (sd.kb1) b += sd.kc1 * sd.kb1[j];
    if (sd.kb2) b += sd.kc2 * sd.kb2[j];
    b = fmaxf(b, kNegBig);
  }
  b = fmaxf(b * inv_lscale, -3.0e38f);
  float mx = b;
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  // a_j: (b - bmax) / 2^18 as fp16, rounded towards zero (never below the true value)
  const float rel = fmaxf((b - mx) * 0x1p-18f, -65504.0f);
  _Float16 ah = (_Float16)rel;
  if ((float)ah < rel)  // negative and one step too low: the next fp16 towards zero
    ah = __builtin_bit_cast(_Float16, (unsigned short)(__builtin_bit_cast(unsigned short, ah) - 1));
  const unsigned aw = (unsigned)__builtin_bit_cast(unsigned short, ah) * 0x00010001u;
  unsigned* rec = sd.key_aux + (size_t)tile * kAuxWords;
  *reinterpret_cast<u32x4*>(rec + kAuxA + lane * 4) = u32x4{aw, aw, aw, aw};
  rec[kAuxB + lane] = __builtin_bit_cast(unsigned, b - (float)ah * 0x1p18f);
  const float mx_sub = __shfl(mx, (lane & 1) * 32, 64);  // lanes 0 and 1: the two sub-tiles' maxima
  rec[kAuxMax + lane] = lane < 2 ? __builtin_bit_cast(unsigned, mx_sub) : 0u;

  // Carried margins: the largest change of a key's bias since the last launch with this side
  // (raw units), and the generation of the margins: a launch whose tag differs from the one the
  // margins were taken under (other operands, eps, coefficients) starts a new one.
  if (sd.bias_prev != nullptr && args.sel != nullptr) {
    const int side = sd.ps_q;  // the margins' state goes with the matrix that holds the query rows
    float dch = 0.f;
    if (j < sd.nk) {
      dch = fabsf(b - sd.bias_prev[j]);
      if (!(dch <= 3.0e38f)) dch = __builtin_bit_cast(float, 0x7f800000u);  // NaN or inf: everything expires
      sd.bias_prev[j] = b;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) dch = fmaxf(dch, __shfl_xor(dch, o, 64));
    if (lane == 0) {
      // (most wavefronts find a larger value already there; a stale read only costs an atomic)
      const unsigned dbits = __builtin_bit_cast(unsigned, dch);
      unsigned* dslot = &args.sel[kSelDmax + side * kDmaxSlots + (tile & (kDmaxSlots - 1))];
      if (dbits > *dslot) atomicMax(dslot, dbits);
      if (tile == 0 && args.sel[kSelTag + side] != args.tag[second ? 1 : 0]) {
        args.sel[kSelTag + side] = args.tag[second ? 1 : 0];
        // entries carry the generation in 8 bits and are cleared only with the planes: after 255
        // generations the margins of this side stay off (256 matches no entry)
        args.sel[kSelGen + side] = min(args.sel[kSelGen + side] + 1u, 256u);
        args.sel[kSelBump + side] = 1u;
      }
    }
  }
}

// With carried margins (Side::margins) this kernel is the form for potentials that still move:
// lse_sparse_kernel, enqueued behind it, runs instead once they have settled (the state words
// say which of the two runs for a side; the other's workgroups return at once).  In its last
// launches before that switch (largest bias change below 1024 base-2 units) this form also
// leaves margin entries behind for the units that end by at least kEntryMargin, so that the first
// sparse launch finds a list to work from instead of visiting every unit.
template <int DP>
__global__ __launch_bounds__(256, 2) void lse_coarse_kernel(const LaunchArgs args) {
  static_assert(DP == 16 || DP == 32 || DP == 64, "two-plane rows of at most 64 columns");
  constexpr int RB = 2;                // blocks of 32 query rows per wavefront
  constexpr int JT = 128;              // keys per tile: hi planes only, four 32-key sub-tiles
  constexpr int NSUB = JT / 32;
  constexpr int NREC = JT / 64;        // bias records (64 keys each) per tile
  constexpr int KK16 = DP / 16;        // MFMAs of one plane product
  constexpr int ROWW = DP;             // 32-bit words per two-plane row in global memory
  constexpr int PPR = ROWW / 4;        // 16-byte pieces per two-plane row
  constexpr int ROWH = DP / 2;         // words per hi-plane row in LDS
  constexpr int PPRH = ROWH / 4;       // 16-byte pieces per hi-plane row
  constexpr int PER_THREAD = JT * PPRH / 256;
  static_assert(64 * PPR == JT * PPRH, "the 64 sampled two-plane rows fill one tile buffer");
  constexpr int NBUF = 4;              // ring of key tiles in LDS: tile t+3 is requested during tile t

  __shared__ __attribute__((aligned(16))) unsigned lds_k[NBUF][JT * ROWH];
  // per 64 keys of a tile: eight copies of a_j (fp16) per key, b_j - 2^18 a_j per key, bmax of
  // the two sub-tiles
  __shared__ __attribute__((aligned(16))) unsigned lds_aux[NBUF][NREC * kAuxWords];

  // variant chosen on the device: the launch of the variant that was not chosen ends here
  if (args.sel_pred && args.sel[kSelWord] != args.sel_want) return;

  int bid = blockIdx.x;
  const bool second = bid >= args.blocks0;
  if (second) bid -= args.blocks0;
  const Side& sd = second ? args.side[1] : args.side[0];
  // With carried margins both forms are enqueued, and the state words say which one runs for a
  // side: this one while the potentials still move.
  bool write_entries = false;
  if (sd.margins != nullptr) {
    const float ls = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
    if (margins_settled(args.sel, sd.ps_q, ls)) return;
    // the switch is near (the change about halves from launch to launch): leave entries behind
    write_entries = args.sel[kSelBump + sd.ps_q] == 0u && args.sel[kSelGen + sd.ps_q] <= 255u &&
                    side_dmax(args.sel, sd.ps_q) * ls < kEntriesBelow;
    if (bid == 0 && threadIdx.x == 0) args.sel[kSelForm + sd.ps_q] = 1u;  // for the merge kernel
  }
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
  const int ntiles = (j_end - j_begin + JT - 1) / JT;

  // MFMAs produce raw products of the scaled planes; lscale turns them into base-2 logits
  const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
  const float inv_lscale = 1.0f / lscale;
  const float skip_below = args.skip_log2 * inv_lscale;  // the 2^40 distance in raw units (< 0)

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

  // Bound on the two cross products of a row, in raw units.  With X, Y the scaled matrices
  // (|.| < 2^15) and hi/lo their planes: |Y_lo| <= 8 (half an ulp of [2^14, 2^15)) and
  // |X_lo| <= 2^-11 |X_hi| (+ 2^-24 for subnormal hi), hence
  //   sum_k |Y_lo X_hi| + |Y_hi X_lo| <= (8 + 16) * (1 + 2^-10) * sum_k |X_hi| + DP * 2^-9,
  // rounded up generously; one base-2 unit of slack covers the fp32 roundings of the chain.
  float corr[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float l1 = 0.f;
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) {
      const f16x8 hv = __builtin_bit_cast(f16x8, xq[rb][0][kk]);
#pragma unroll
      for (int e = 0; e < 8; ++e) l1 += fabsf((float)hv[e]);
    }
    l1 += xor32(l1);
    corr[rb] = 24.5f * l1 + (float)DP * 0x1p-9f + inv_lscale;
  }

  // run_m: running maximum in raw units; run_c = -run_m * lscale as rounded once, the offset
  // every exponent of the row uses (rescaling by differences of run_c stays consistent)
  float run_m[RB], run_s[RB], run_c[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) run_m[rb] = run_s[rb] = run_c[rb] = 0.f;

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
  auto ds_write16 = [&](unsigned* p, u32x4 v) {
    asm volatile("ds_write_b128 %0, %1" : : "v"(lds_addr(p)), "v"(v) : "memory");
  };
  auto wait_lds = [&]() { __builtin_amdgcn_s_waitcnt(0xC07F); };   // lgkmcnt(0)
  // The compiler takes the result of a hand-written ds_read for valid right after the
  // statement.  Passing the registers through an empty statement placed after the wait makes
  // every later use depend on a point behind it.
  auto pin4 = [](u32x4& v) { asm volatile("" : "+v"(v)); };
  auto pin1 = [](float& v) { asm volatile("" : "+v"(v)); };
  auto wait_all = [&]() { __builtin_amdgcn_s_waitcnt(0x0070); };   // vmcnt(0) and lgkmcnt(0)
  // everything but the newest key tile has landed (loads complete in issue order), and lgkmcnt(0)
  auto wait_older_tiles = [&]() { __builtin_amdgcn_s_waitcnt(0x0070 | PER_THREAD); };
  auto barrier = [&]() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  // slot permutation of LDS row r when a row has `ppr` 16-byte pieces: b128 reads of 32
  // consecutive rows at one piece index then spread over all banks
  auto swz_of = [](int r, int ppr) {
    return ppr >= 16 ? (r & 15) : (ppr == 8 ? ((r >> 1) & 7) : (ppr == 4 ? ((r >> 2) & 3) : ((r >> 3) & 1)));
  };
  auto swz = [&](int r) { return swz_of(r, PPR); };    // the sampled two-plane rows
  auto swzh = [&](int r) { return swz_of(r, PPRH); };  // hi-plane rows of a key tile

  // ---- key tiles: lane idx of instruction c fills LDS slot idx and fetches the piece that
  // belongs there (slot = piece ^ swz(row)); the plane buffers end in zero rows, so tiles past
  // the chunk are fetched like any other and masked by their bias ----
  const unsigned* kp[PER_THREAD];
#pragma unroll
  for (int c = 0; c < PER_THREAD; ++c) {
    const int idx = tid + 256 * c;
    const int r = idx / PPRH;
    const int piece = (idx % PPRH) ^ swzh(r);  // a piece of the hi plane, the first half of the row
    kp[c] = sd.kplanes + (size_t)(j_begin + r) * (size_t)ROWW + piece * 4;
  }
  auto issue_tile = [&](int buf) {  // the next tile in sequence
#pragma unroll
    for (int c = 0; c < PER_THREAD; ++c) {
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)kp[c],
          (__attribute__((address_space(3))) void*)(&lds_k[buf][(c * 256 + wave * 64) * 4]), 16, 0,
          0);
      kp[c] += JT * ROWW;
    }
  };

  // ---- key bias: coarse_bias_kernel has written, per 64-key tile, the record that the tile's
  // LDS buffer takes (a_j, b_j - 2^18 a_j, bmax; raw units); wavefront 0 brings it in with two
  // direct loads, issued before the tile's keys so that the same wait covers both ----
  const float kc0 = sd.kc0, kc1 = sd.kc1, kc2 = sd.kc2;
  const bool has_kb1 = sd.kb1 != nullptr, has_kb2 = sd.kb2 != nullptr;
  const float* kb1p = has_kb1 ? sd.kb1 : sd.kb0;
  const float* kb2p = has_kb2 ? sd.kb2 : sd.kb0;
  const unsigned* auxp = sd.key_aux + (size_t)(j_begin / 64) * kAuxWords + lane * 4;
  auto issue_aux = [&](int buf) {  // the next tile in sequence
    if (wave == 0) {  // every instruction with all 64 lanes: 16, 4 and 4 bytes per lane
#pragma unroll
      for (int rec = 0; rec < NREC; ++rec) {
        const unsigned* src = auxp + rec * kAuxWords;  // auxp: word 4 * lane of the record
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)src,
            (__attribute__((address_space(3))) void*)(&lds_aux[buf][rec * kAuxWords + kAuxA]), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(src - 3 * lane + kAuxB),
            (__attribute__((address_space(3))) void*)(&lds_aux[buf][rec * kAuxWords + kAuxB]), 4, 0, 0);
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(src - 3 * lane + kAuxMax),
            (__attribute__((address_space(3))) void*)(&lds_aux[buf][rec * kAuxWords + kAuxMax]), 4, 0, 0);
      }
    }
    auxp += NREC * kAuxWords;
  };
  // word `what` (+ key k of the sub-tile) in the record that holds sub-tile js of buffer buf
  auto aux_at = [&](int buf, int js, int what) {
    return &lds_aux[buf][(js >> 1) * kAuxWords + what];
  };

  auto mfma16 = [](const u32x4& a, const u32x4& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  };
  // 16-byte piece (step kk, half h) of the hi plane of key row js*32 + li of a key tile
  auto read_hi = [&](u32x4 (&dst)[KK16], int buf, int js) {
    const unsigned* yrow = lds_k[buf] + (js * 32 + li) * ROWH;
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk)
      dst[kk] = ds_read16(yrow + (((2 * kk + h) ^ swzh(li)) << 2));  // swzh(js*32 + li) == swzh(li)
  };
  // the same of either plane of sampled two-plane row js*32 + li (buffer 0)
  auto read_sampled = [&](u32x4 (&dst)[KK16], int js, int plane) {
    const unsigned* yrow = lds_k[0] + (js * 32 + li) * ROWW;
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) {
      const int piece = plane * (DP / 8) + 2 * kk + h;
      dst[kk] = ds_read16(yrow + ((piece ^ swz(li)) << 2));
    }
  };
  // v_permlane32_swap exchanges lanes 32..63 of its first operand with lanes 0..31 of its
  // second: (a, b) = (t, t) becomes (low half twice, high half twice)
  auto swap_halves = [&](float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  };
  auto max16 = [](const f32x16& a) {
    const float m0 = fmaxf(fmaxf(a[0], a[1]), a[2]);
    const float m1 = fmaxf(fmaxf(a[3], a[4]), a[5]);
    const float m2 = fmaxf(fmaxf(a[6], a[7]), a[8]);
    const float m3 = fmaxf(fmaxf(a[9], a[10]), a[11]);
    const float m4 = fmaxf(fmaxf(a[12], a[13]), a[14]);
    return fmaxf(fmaxf(fmaxf(m0, m1), a[15]), fmaxf(fmaxf(m2, m3), m4));
  };
  // the key bias of sub-tile js added to every query column: A = [bias_j, 1], B = [1, 0]
  auto add_bias = [&](const f32x16& acc, float bias_lane) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(h ? 1.0f : bias_lane, h ? 0.0f : 1.0f, acc, 0, 0, 0);
  };

  u32x4 KH[2][KK16];  // hi planes of the sub-tile in work and the next one
  u32x4 KA[2];        // their a_j pieces (the same piece in both half-waves)
  // query side of the a_j step: 2^15 in the eight slots of the lower half-wave, nothing above
  const unsigned qcw = h ? 0u : 0x78007800u;
  const u32x4 QC = {qcw, qcw, qcw, qcw};
  u32x4 KL[KK16];     // lo plane of the sub-tile in work, read when a unit of it goes on
  float kbias = 0.f;  // bias of key js*32 + li of that sub-tile, read together with KL
  float bmax[2] = {0.f, 0.f};  // largest bias of the sub-tiles whose hi planes are in KH

  // ---- where the running maxima start (sums start empty): coarse_bias_kernel has computed it ----
  const bool track = sd.best_key != nullptr;
  int best_j[RB];
  float warm[RB];
  bool have = track;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    best_j[rb] = -1;
    warm[rb] = -3.0e38f;
    if (track) {
      warm[rb] = sd.seed[min(row0 + rb * 32 + li, sd.nq - 1)];
      have = have && warm[rb] > -3.0e38f;
    }
  }
  // a workgroup with a row that has no key yet also samples 64 keys spread over the whole key set
  const bool cold = __syncthreads_or(have ? 0 : 1) != 0;
  if (cold) {
    const int stride = sd.nk / 64;  // sampled keys: 0, stride, 2 stride, ...
    if (wave == 0) {
      const int j = lane * stride;
      float b = kc0 * sd.kb0[j] + (has_kb1 ? kc1 * kb1p[j] : 0.f);
      b += (has_kb2 ? kc2 * kb2p[j] : 0.f);
      ds_write4(reinterpret_cast<float*>(&lds_aux[0][kAuxB + lane]),
                fmaxf(fmaxf(b, kNegBig) * inv_lscale, -3.0e38f));
    }
#pragma unroll
    for (int c = 0; c < PER_THREAD; ++c) {
      const int idx = tid + 256 * c;
      const int r = idx / PPR;
      const int piece = (idx % PPR) ^ swz(r);
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(sd.kplanes + (size_t)(r * stride) *
                                                                          (size_t)ROWW + piece * 4),
          (__attribute__((address_space(3))) void*)(&lds_k[0][(c * 256 + wave * 64) * 4]), 16, 0, 0);
    }
    wait_all();
    barrier();
#pragma unroll
    for (int js = 0; js < 2; ++js) {
      read_sampled(KH[0], js, 0);
      read_sampled(KL, js, 1);
      kbias = ds_read4(reinterpret_cast<const float*>(&lds_aux[0][kAuxB + js * 32 + li]));
      wait_lds();
#pragma unroll
      for (int kk = 0; kk < KK16; ++kk) {
        pin4(KH[0][kk]);
        pin4(KL[kk]);
      }
      pin1(kbias);
      FS_LC_FENCE();
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < KK16; ++kk) acc = mfma16(KL[kk], xq[rb][0][kk], acc);
#pragma unroll
        for (int kk = 0; kk < KK16; ++kk) acc = mfma16(KH[0][kk], xq[rb][1][kk], acc);
#pragma unroll
        for (int kk = 0; kk < KK16; ++kk) acc = mfma16(KH[0][kk], xq[rb][0][kk], acc);
        acc = add_bias(acc, kbias);
        const float mx = max16(acc);
        float a = mx, b = mx;
        swap_halves(a, b);
        const float m = fmaxf(a, b);
        if (track && (js == 0 || wave_any(m > run_m[rb]))) {  // as in go_on below
          int rr = 0;
#pragma unroll
          for (int r = 1; r < 16; ++r) rr = (acc[r] == mx) ? r : rr;
          if (js == 0 || m > run_m[rb])
            best_j[rb] = (mx == m) ? (js * 32 + 8 * (rr >> 2) + 4 * h + (rr & 3)) * stride : -1;
        }
        run_m[rb] = js == 0 ? m : fmaxf(run_m[rb], m);
      }
    }
    barrier();  // buffer 0 is free again
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    if (!cold || warm[rb] > run_m[rb]) {  // the row's key of the last launch stays until exceeded
      run_m[rb] = warm[rb];
      best_j[rb] = -1;
    }
    float c = -run_m[rb] * lscale;
    asm volatile("" : "+v"(c));  // the rounded product itself, nothing fused into later uses
    run_c[rb] = c;
  }

  // margin entries of this wavefront (see margin_entry): entry 2 s + rb for sub-tile s of the chunk
  // (everything here is the same in all lanes and kept in scalar registers)
  unsigned* ent = nullptr;
  unsigned far_entry = 0u, gen_word = 0u;
  const float far_raw = kEntryMargin * inv_lscale;
  if (write_entries) {
    const int wrow = __builtin_amdgcn_readfirstlane(row0 / 64);
    ent = reinterpret_cast<unsigned*>(sd.margins) +
          ((size_t)wrow * (size_t)sd.margin_stride + (size_t)(j_begin / 32)) * 2;
    const float cum2 = 2.002f * (__builtin_bit_cast(float, args.sel[kSelCum + sd.ps_q]) +
                                 side_dmax(args.sel, sd.ps_q));
    float sl = 0.f;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) sl = fmaxf(sl, corr[rb] * 0x1p-6f + 2.0f * inv_lscale);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sl = fmaxf(sl, __shfl_xor(sl, o, 64));
    const float wslack = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, sl)));
    gen_word = args.sel[kSelGen + sd.ps_q];
    far_entry = margin_entry(far_raw, wslack, cum2, gen_word);
  }

  unsigned n_ended = 0;
  f32x16 H[4];  // hi*hi products (on top of 2^18 a_j): sub-tile s, row block rb in H[2 (s & 1) + rb]

  // Start of tile t: the keys and the bias record of tile t+1 have landed (only those of tile t+2
  // may still be in flight); after the barrier tile t+1 is visible and every wavefront is done
  // with tile t-1, whose buffer takes tile t+3.
  auto start_of_tile = [&](int t) {
    wait_older_tiles();
    barrier();
    issue_aux((t + 3) & 3);
    issue_tile((t + 3) & 3);
  };
  // hi plane, a_j piece and bmax of sub-tile js of the tile in buffer b, into register set k
  auto request = [&](int k, int b, int js) {
    read_hi(KH[k], b, js);
    KA[k] = ds_read16(aux_at(b, js, kAuxA + ((js & 1) * 32 + li) * 4));
    bmax[k] = ds_read4(reinterpret_cast<const float*>(aux_at(b, js, kAuxMax + (js & 1))));
  };
  auto arrived = [&](int k) {  // after a wait: every later use of set k sits behind this point
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) pin4(KH[k][kk]);
    pin4(KA[k]);
    pin1(bmax[k]);
  };

  // Operands of the units of sub-tile js (buffer b) that go on, pipelined form: the hi plane and
  // the per-key biases again from LDS (the register set the sub-tile was multiplied from has
  // moved on), the lo plane from global memory (the second half of a key's two-plane row; the
  // compiler places that wait).
  auto fetch_full = [&](u32x4 (&KX)[KK16], int b, int js, int kbase) {
    const unsigned* lrow = sd.kplanes + (size_t)(kbase + li) * (size_t)ROWW + DP / 2 + 4 * h;
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) KL[kk] = *reinterpret_cast<const u32x4*>(lrow + 8 * kk);
    read_hi(KX, b, js);
    kbias = ds_read4(reinterpret_cast<const float*>(aux_at(b, js, kAuxB + (js & 1) * 32 + li)));
    wait_lds();
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) pin4(KX[kk]);
    pin1(kbias);
  };
  // A unit that goes on: the two cross products and the key bias on top of its hi*hi product,
  // then its soft-max.  Everything it computes lives and dies here.
  auto unit_full = [&](const f32x16& hh, const u32x4 (&KX)[KK16], const u32x4 (&KLx)[KK16], float kb,
                       int rb, int kbase) {
    FS_LC_FENCE();
    f32x16 L = mfma16(KX[0], xq[rb][1][0], hh);
#pragma unroll
    for (int kk = 1; kk < KK16; ++kk) L = mfma16(KX[kk], xq[rb][1][kk], L);
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) L = mfma16(KLx[kk], xq[rb][0][kk], L);
    L = add_bias(L, kb);
    FS_LC_FENCE();
    const float mx = max16(L);  // this lane's 16 keys
    // every logit of the unit more than the 2^40 distance below its row's running maximum:
    // its exponentials would not change the fp32 row sums
    if (wave_any(mx - run_m[rb] > skip_below)) {
      float a = mx, b2 = mx;
      swap_halves(a, b2);
      const float m_new = fmaxf(fmaxf(a, b2), run_m[rb]);
      if (track && wave_any(m_new > run_m[rb])) {
        // the maximum of a row moves: the half-wave that holds the new one notes its key (register
        // r of a lane is key 8 (r / 4) + 4 h + r % 4 of the sub-tile), the other half forgets its own
        int rr = 0;
#pragma unroll
        for (int r = 1; r < 16; ++r) rr = (L[r] == mx) ? r : rr;
        if (m_new > run_m[rb]) best_j[rb] = (mx == m_new) ? kbase + 8 * (rr >> 2) + 4 * h + (rr & 3) : -1;
      }
      float cx = -m_new * lscale;
      asm volatile("" : "+v"(cx));  // rounded once, see run_c
      float ps0 = 0.f, ps1 = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        ps0 += fast_exp2(__builtin_fmaf(L[r], lscale, cx));
        ps1 += fast_exp2(__builtin_fmaf(L[r + 1], lscale, cx));
      }
      run_s[rb] = run_s[rb] * fast_exp2(cx - run_c[rb]) + (ps0 + ps1);
      run_m[rb] = m_new;
      run_c[rb] = cx;
    }
  };

  // One step = one 32-key sub-tile s (parity c = s & 1, in LDS buffer b): the hi*hi products of
  // sub-tile s+1 go to the matrix pipe, with the tests of sub-tile s (whose products finished
  // during the last step) placed between them in program order; then the units of s that go on.
  // nb, njs: buffer and sub-tile index of s+2, whose hi plane is requested into the set that
  // sub-tile s was multiplied from.
  auto step = [&](auto c_c, int b, int js, int nb, int njs, int kbase) {
    constexpr int c = decltype(c_c)::value, n = c ^ 1;
    wait_lds();  // set n (sub-tile s+1), requested during the last step
    arrived(n);
    const float lim = skip_below - bmax[c];  // read before the request below replaces bmax[c]
    request(c, nb, njs);
    FS_LC_FENCE();
    f32x16 z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0.f;
    const f32x16& t0 = H[2 * c], &t1 = H[2 * c + 1];
    f32x16 &a = H[2 * n], &bq = H[2 * n + 1];
    a = mfma16(KA[n], QC, z);
    FS_LC_FENCE();
    const float p0 = fmaxf(fmaxf(t0[0], t0[1]), t0[2]), p1 = fmaxf(fmaxf(t0[3], t0[4]), t0[5]);
    FS_LC_FENCE();
    bq = mfma16(KA[n], QC, z);
    FS_LC_FENCE();
    const float p2 = fmaxf(fmaxf(t0[6], t0[7]), t0[8]), p3 = fmaxf(fmaxf(t0[9], t0[10]), t0[11]);
    FS_LC_FENCE();
    a = mfma16(KH[n][0], xq[0][0][0], a);
    FS_LC_FENCE();
    const float p4 = fmaxf(fmaxf(t0[12], t0[13]), t0[14]), p5 = fmaxf(fmaxf(p0, p1), t0[15]);
    FS_LC_FENCE();
    bq = mfma16(KH[n][0], xq[1][0][0], bq);
    FS_LC_FENCE();
    const float mx0 = fmaxf(p5, fmaxf(fmaxf(p2, p3), p4));
    const bool full0 = wave_any(mx0 > run_m[0] + lim - corr[0]);
    FS_LC_FENCE();
    float q0 = 0.f, q1 = 0.f, q2 = 0.f, q3 = 0.f, q4 = 0.f, q5 = 0.f;
#pragma unroll
    for (int kk = 1; kk < KK16; ++kk) {
      a = mfma16(KH[n][kk], xq[0][0][kk], a);
      FS_LC_FENCE();
      if (kk == 1) {
        q0 = fmaxf(fmaxf(t1[0], t1[1]), t1[2]);
        q1 = fmaxf(fmaxf(t1[3], t1[4]), t1[5]);
        q2 = fmaxf(fmaxf(t1[6], t1[7]), t1[8]);
      }
      FS_LC_FENCE();
      bq = mfma16(KH[n][kk], xq[1][0][kk], bq);
      FS_LC_FENCE();
      if (kk == 1) {
        q3 = fmaxf(fmaxf(t1[9], t1[10]), t1[11]);
        q4 = fmaxf(fmaxf(t1[12], t1[13]), t1[14]);
        q5 = fmaxf(fmaxf(q0, q1), t1[15]);
      }
      FS_LC_FENCE();
    }
    if (KK16 == 1) {  // narrow rows: no MFMA left to sit behind
      q0 = fmaxf(fmaxf(t1[0], t1[1]), t1[2]);
      q1 = fmaxf(fmaxf(t1[3], t1[4]), t1[5]);
      q2 = fmaxf(fmaxf(t1[6], t1[7]), t1[8]);
      q3 = fmaxf(fmaxf(t1[9], t1[10]), t1[11]);
      q4 = fmaxf(fmaxf(t1[12], t1[13]), t1[14]);
      q5 = fmaxf(fmaxf(q0, q1), t1[15]);
    }
    const float mx1 = fmaxf(q5, fmaxf(fmaxf(q2, q3), q4));
    const bool full1 = wave_any(mx1 > run_m[1] + lim - corr[1]);
    n_ended += (full0 ? 0u : 1u) + (full1 ? 0u : 1u);
    FS_LC_FENCE();
    if (write_entries) {
      // (wave-uniform) a unit that ended by at least kEntryMargin gets an entry that says so:
      // one more comparison per unit, where the exact margin would take a reduction over the
      // wavefront (lse_sparse_kernel visits the others once and then knows theirs exactly)
      const bool far0 = !wave_any(mx0 > run_m[0] + lim - corr[0] - far_raw);
      const bool far1 = !wave_any(mx1 > run_m[1] + lim - corr[1] - far_raw);
      if (lane == 0) {
        unsigned* e = ent + (kbase - j_begin) / 16;  // two entries per 32-key sub-tile
        // (a unit that went on is marked as such: the generation alone, no margin)
        e[0] = far0 ? far_entry : (full0 ? gen_word : 0u);
        e[1] = far1 ? far_entry : (full1 ? gen_word : 0u);
      }
    }
    FS_LC_FENCE();
    // the set that sub-tile s+1 was just multiplied from is free until the next step's request
    if (full0 || full1) fetch_full(KH[n], b, js, kbase);
    if (full0) unit_full(t0, KH[n], KL, kbias, 0, kbase);
    if (full1) unit_full(t1, KH[n], KL, kbias, 1, kbase);
    FS_LC_FENCE();
  };

  // ---- prologue: tiles 0 and 1 published, tiles 2 and 3 on their way; hi*hi of sub-tile 0 ----
  issue_aux(0);
  issue_tile(0);
  issue_aux(1);
  issue_tile(1);
  issue_aux(2);
  issue_tile(2);
  start_of_tile(0);
  request(0, 0, 0);
  request(1, 0, 1);
  wait_lds();
  arrived(0);
  arrived(1);
  FS_LC_FENCE();
  {
    f32x16 z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0.f;
    H[0] = mfma16(KA[0], QC, z);
    H[1] = mfma16(KA[0], QC, z);
#pragma unroll
    for (int kk = 0; kk < KK16; ++kk) {
      H[0] = mfma16(KH[0][kk], xq[0][0][kk], H[0]);
      H[1] = mfma16(KH[0][kk], xq[1][0][kk], H[1]);
    }
  }
  for (int t = 0; t < ntiles; ++t) {
    if (t > 0) start_of_tile(t);
    const int b = t & 3, nb = (t + 1) & 3;
    const int kb = j_begin + t * JT;
    // sub-tile js multiplies sub-tile js+1 and requests sub-tile js+2 (the last two: of tile t+1)
    step(std::integral_constant<int, 0>{}, b, 0, b, 2, kb);
    step(std::integral_constant<int, 1>{}, b, 1, b, 3, kb + 32);
    step(std::integral_constant<int, 0>{}, b, 2, nb, 0, kb + 64);
    step(std::integral_constant<int, 1>{}, b, 3, nb, 1, kb + 96);
  }
  wait_all();  // tiles fetched past the chunk: let them land before the workgroup ends

  // unit counts of this wavefront for the variant choice on the device; a workgroup that had
  // to sample its starting values says nothing about the launches that follow
  if (args.sel != nullptr && lane == 0 && ntiles > 0) {
    const int slot = blockIdx.x % kSelSlots;
    if (!(track && cold)) {
      atomicAdd(&args.sel[kSelEnded + slot], n_ended);
      atomicAdd(&args.sel[kSelUnits + slot], (unsigned)(ntiles * NSUB * RB));
    }
  }

#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = row0 + rb * 32 + li;
    const float s = run_s[rb] + xor32(run_s[rb]);
    const float M2 = -run_c[rb];
    int bj = best_j[rb];
    const int oj = __shfl_xor(bj, 32, 64);
    if (bj < 0) bj = oj;
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
