// Shared definitions for the gfx950 FlashSinkhorn kernels.
//
// Every streaming kernel computes, for a block of stationary "query" rows q_i and
// a stream of "key" rows k_j, base-2 logits
//     L_ij = qscale * (q_i . k_j) + kbias_j
// and reduces over j with a lane-private online soft-max.  The transport-plan
// operations differ only in what they accumulate next to the running sum.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flash_sinkhorn_hip.h"

#ifndef FS_SETTLE
#define FS_SETTLE 256.0f
#endif
#ifndef FS_ENTRIES_BELOW
#define FS_ENTRIES_BELOW 512.0f
#endif
#ifndef FS_ENTRY_MARGIN
#define FS_ENTRY_MARGIN 1024.0f
#endif

namespace fs {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegBig = -1.0e30f;   // finite stand-in for -inf on masked keys
constexpr float kLazyThresh = 16.0f;  // rescale only when the tile max exceeds 2^16

enum Mode : int { kLse = 0, kVec = 1, kMat = 2, kMat5 = 3, kArgmax = 4 };
enum EpiKind : int { kEpiLse = 0, kEpiApply = 1, kEpiGrad = 2, kEpiArgmax = 3 };

// What to do with a finished row (M, s, O[.]) of base-2 soft-max statistics.
struct Epilogue {
  int kind;
  float* out;            // [nq] (LSE, VEC) or [nq, d] (MAT kinds)
  // kEpiLse: out = alpha*(out_scale*(M+log2 s)) + (1-alpha)*old - shift_coef*shift
  const float* old;
  const float* shift;
  float alpha, out_scale, shift_coef;
  // kEpiApply: out = post * exp2(rc0*r0[i] + rc1*r1[i] + rc2*r2[i] + M) * O
  const float* r0;
  const float* r1;
  const float* r2;
  float rc0, rc1, rc2, post;
  // kEpiApply, scalar outputs only: then out *= mul[i] (if given) and, with add_a,
  // out = add_a[i]*add_b[i] + res_coef*out (the two halves of a Schur-complement product)
  const float* mul;
  const float* add_a;
  const float* add_b;
  float res_coef;
  // kEpiGrad: out = gcoef * gs * w[i] * (q[i,:] - O/s)
  const float* w;
  const float* grad_scale;  // 1-element device array or null
  float gcoef;
  // kEpiArgmax (c-transform): out = -max_j t_ij, idx_out = the smallest j attaining it
  long long* idx_out;
};

// One half of a launch: which rows are stationary, which are streamed.
struct Side {
  const float* q;       // [nq, d] stationary rows
  const float* k;       // [nk, d] streamed rows
  const float* q2;      // kMat5: second stationary operand [nq, d]
  const float* v;       // kVec: [nk]; kMat: [nk, d] or null (values = k rows)
  const float* vscale;  // kMat: optional per-key scale [nk]
  const float* kb0;     // key bias (base 2): kc0*kb0[j] + kc1*kb1[j] + kc2*kb2[j]
  const float* kb1;
  const float* kb2;
  float kc0, kc1, kc2;
  float qscale;         // coord_scale / eps * log2(e)
  int nq, nk;
  int splits;           // number of key chunks
  int chunk;            // keys per chunk (multiple of the key tile)
  int igroups;          // ceil(nq / rows per workgroup)
  const unsigned* qplanes;  // split-bf16 kernels: query rows as packed bf16 planes [nq][NP][DP/2]
  const unsigned* kplanes;  // same for the key rows [nk][NP][DP/2]
  const float* plane_scale; // fp16 planes: power-of-two scales of the two operand matrices [2]
  int ps_q, ps_k;           // which of the two scales belongs to the query / key matrix (a side
                            // may pair a matrix with itself while another matrix is present)
  const unsigned* vplanes;  // plan_gemm_kernel: fp16 planes of the value matrix in operand order
  const float* vplane_scale;  // their power-of-two scale [1]
  const unsigned* q2planes; // plan_gemm_kernel, mat5: chunked fp16 planes of q2
  const float* q2plane_scale;  // scale of q2's planes [1]
  const float* kplane_scale;   // scale of the key matrix alone [1]
  const float* q2norm2;        // mat5: |q2_i|^2 per row [nq]
  const float* kmax2;          // mat5: 64 partial maxima of |k_j|^2
  float* part_ms;       // [splits, nq, 2] partial (M, s) when splits > 1
  // lse_coarse_kernel: per query row, the key that held the row's largest logit in the last
  // launch over these operands (-1: none yet).  The current logit of that key is where the
  // row's running maximum starts: a lower bound of the new maximum whatever the entry holds.
  int* best_key;        // [nq] or null
  int* part_best;       // [splits, nq] when splits > 1: the key behind a partial M, -1 when no
                        // key of the chunk exceeded the starting value
  // lse_coarse_kernel: per 64-key tile, what coarse_bias_kernel derives from the key bias, in
  // the layout the tile's LDS buffer takes (kAuxWords words per tile, kAuxPadTiles tiles past
  // the last key)
  unsigned* key_aux;
  // lse_coarse_kernel, margins carried from launch to launch (all null: none).  margins: per
  // wavefront (64 query rows) and 32-key sub-tile two entries (one per row block), `margin_stride`
  // sub-tiles per wavefront: by how much the sub-tile's logits stayed below the point where they
  // could matter when they were last tested, plus twice the sum of all key-bias changes up to
  // then, tagged with a generation in the low 8 bits.  m_prev: per query row the merged maximum
  // of the last launch (base-2 units).  bias_prev: per key the raw bias of the last launch.
  // Second copy of the key and query planes in MFMA operand order, for kernels that take their
  // operands straight from global memory: per 32 rows, plane and 16-column step one 1 KiB block
  // with lane (h, row % 32)'s 16 bytes at 16 * (32 h + row % 32).
  const unsigned* ktiled;
  const unsigned* qtiled;
  float* margins;
  int margin_stride;
  int sparse_group;     // key chunks one wavefront of the sparse form goes through
  float* m_prev;
  float* bias_prev;
  float* seed;          // per query row: where this launch's running maximum starts (raw units)
  // lse_sparse_kernel: per (64-row group, key range) how many of the range's partial results it
  // wrote (the merge kernel reads only those); index row group * ranges + range
  unsigned char* npieces;
  float* part_o;        // [splits, nq, DP] partial O when splits > 1 (MAT kinds) or [splits,nq] (VEC)
  Epilogue ep;
};

struct LaunchArgs {
  Side side[2];
  int blocks0;   // blocks belonging to side[0]; the rest belong to side[1]
  int blocks_all;  // lse_gemm_kernel: work items of both sides (its grid is rounded up to 8 k)
  int d;         // true feature dimension
  int vec_ok;    // rows are 16-byte aligned (d % 4 == 0 and aligned bases)
  int nss;       // column-sliced kernels: super-slices of 1536 columns (1 unless d > 1536)
  int pstride;   // GEMM-shaped kernels: words per row of the chunked fp16 planes
  float out_scale;  // finish_argmax_kernel: units of the partial values (1, or the plane scale)
  float skip_log2;  // lse2_kernel: tiles whose logits all lie this far (base 2, negative) below
                    // the running maxima skip their exponentials; -inf-like to switch it off
  // Log-sum-exp kernels, variant chosen on the device: a launch with `sel` and `sel_pred` set
  // runs only when sel[kSelWord] == sel_want (its workgroups return at once otherwise).  The
  // variant with the coarse tile test counts its units into the slots of the same state block.
  unsigned* sel;
  unsigned sel_want;
  int sel_pred;  // 0: the launch runs whatever the state says (it still counts into it)
  unsigned tag[2];  // per side: what the carried margins depend on (operands, scales, coefficients)
  // lse_sparse_kernel: its grid, how many sides it serves, and its work queues (kQueueWords
  // words per side and XCD, zeroed by coarse_bias_kernel before every launch)
  int blocks_sparse, sparse_sides;
  unsigned* queue;
  // Two-sided steps whose sides are the two orders of one pair of matrices, on prepared planes:
  // lse_sweep_kernel computes both sides' sums from one sweep over the logits when the state
  // words allow it (sweep != 0: the step has such a launch; the two-sided kernel then only runs
  // when that one did not, or failed).  col_part: [side[0].igroups][side[0].nk] sums over the
  // query rows of a workgroup for every key.
  int sweep;            // 1, or 2 when the variant is chosen on the device (the one-sweep form
                        // then belongs to the plain variant)
  int sw_splits, sw_chunk;  // key chunks of the one-sweep launch (its own: at most side[0].splits)
  float* col_part;
  // sweep_self: every side is a problem of a matrix with itself (q == k, a symmetric matrix of
  // logits once both biases are inside): the one-sweep launch only visits key tiles at or beyond
  // a workgroup's own 256 rows, a row's sum is its partial row sums plus the column sums that the
  // row groups before its own took for it.  Side 1 (if any) has its own chunks and column sums;
  // sw_items0 / sw_items: work items of side 0 / of the launch.
  int sweep_self;
  int sw_splits_b, sw_chunk_b;
  float* col_part_b;
  int sw_items0, sw_items;
  int sw_part_mult;  // partial rows per key chunk (2 for lse_gemm_kernel, else 1; 0 reads as 1)
};

// Row groups (of 256 rows) that have keys at or beyond their first row in key chunk s of a
// matrix paired with itself.
__host__ __device__ inline int self_groups_of_chunk(int s, int chunk, int n, int groups) {
  const long long end = (long long)(s + 1) * chunk < n ? (long long)(s + 1) * chunk : n;
  const int g = (int)((end + 255) / 256);
  return g < groups ? g : groups;
}

// Work queue of lse_sparse_kernel for one (side, XCD): word 0 counts the base items handed out,
// word 16 the remainders pushed, word 32 the remainders popped (one cache line each); from word
// 64 on, kQueueSlots 64-bit slots for the remainders (0: empty, all ones: taken).
constexpr int kQueueBase = 0, kQueueTail = 16, kQueueHead = 32, kQueueSlot0 = 64, kQueueSlots = 224;
constexpr int kQueueWords = kQueueSlot0 + 2 * kQueueSlots;
constexpr size_t kQueueBytes = (size_t)2 * 8 * kQueueWords * 4;
constexpr int kSparseBlocks = 512;

// Record of coarse_bias_kernel per 64 keys: eight fp16 copies of a_j per key (4 words each), then
// b_j - 2^18 a_j per key, then the largest bias of each 32-key sub-tile in the first two of 64
// words: three parts that one wavefront moves with one full instruction each (16, 4 and 4
// bytes per lane).
constexpr int kAuxA = 0, kAuxB = 256, kAuxMax = 320, kAuxWords = 384, kAuxPadTiles = 8;

// Device state of the variant choice (unsigned words), zeroed when the operand planes are
// written: which variant runs (0: coarse tile test, 1: plain), how many decisions were taken,
// running totals, and per-launch counters spread over kSelSlots slots (slot = workgroup % slots).
constexpr int kSelWord = 0, kSelDecisions = 1, kSelCumEnded = 2, kSelCumUnits = 4;  // totals: u64
constexpr int kSelSlots = 64, kSelEnded = 8, kSelUnits = kSelEnded + kSelSlots;
// carried margins, per matrix of the plane set in the role of the query rows (Side::ps_q):
// running sum of the key-bias changes (float), this launch's largest
// change (float bits, by atomic max), the tag the margins were taken under, their generation
// (1..255; 0 never valid), and whether this launch started a generation
constexpr int kSelCum = kSelUnits + kSelSlots, kSelTag = kSelCum + 2;
constexpr int kSelGen = kSelTag + 2, kSelBump = kSelGen + 2;
constexpr int kSelMode = kSelBump + 2;  // likewise: the last launch ran in the sparse form
constexpr int kSelSkip = kSelMode + 2;  // per-launch slots: units the sparse form did not visit
constexpr int kSelCumSkipped = 6;       // their running total (u64), part of kSelCumEnded's
// likewise (per matrix in the role of the query rows): which kernel wrote the partial results of
// the launch under way (0: lse2_kernel, 1: lse_coarse_kernel, 2: lse_sparse_kernel), for the merge
constexpr int kSelForm = kSelSkip + kSelSlots;
// this launch's largest key-bias change per matrix in the role of the query rows: kDmaxSlots words
// each (float bits, by atomic max; the wavefronts of coarse_bias_kernel spread over the slots, or
// a thousand atomics on one word would take longer than the rest of that kernel)
constexpr int kDmaxSlots = 16;
constexpr int kSelDmax = kSelForm + 2;
// likewise per role: margin entries of the current generation exist (lse_coarse_kernel left them
// behind, or lse_sparse_kernel ran); without them the sparse form would visit every unit
constexpr int kSelHave = kSelDmax + 2 * kDmaxSlots;
// the share of units the plain kernel left out in the first launch of its current stretch, in
// 65536ths plus one (0: not taken yet)
constexpr int kSelBase = kSelHave + 2;
// The one-sweep form of a two-sided step (lse_sweep_kernel): whether this step may run it (set by
// the merge of the step before), whether its sums left the range it is exact in (the two-sided
// kernel then redoes the step), the merge kernel's count of workgroups that are done, and the
// step's largest and smallest log2 of a row or column sum (float bits of the largest and of minus
// the smallest, by atomic max, spread over slots)
constexpr int kSelSweep = kSelBase + 1, kSelSweepFail = kSelSweep + 1, kSelSweepDone = kSelSweep + 2;
constexpr int kSweepSlots = 8;
constexpr int kSelSweepHi = kSelSweep + 3, kSelSweepLo = kSelSweepHi + kSweepSlots;
// which variant's kernels ran in the step under way (1: the plain one, one-sweep form included;
// 0: the one with the coarse tile test), written by them for the merge kernel, whose first
// workgroup may change kSelWord while the others still need to know
constexpr int kSelRan = kSelSweepLo + kSweepSlots;
// the extremes of the last step of the plain variant (float bits of the largest log2 of a sum
// and of minus the smallest), kept for the next step's permission and for diagnostics
constexpr int kSelSweepLast = kSelRan + 1;
// how many steps of the one-sweep form the two-sided kernel had to redo so far (diagnostics)
constexpr int kSelSweepRedone = kSelSweepLast + 2;
constexpr int kSelWords = kSelSweepRedone + 1;
static_assert(kSelWords <= 512, "one workgroup clears the state block, two words per thread");
// log2 of the sums (each about a row's or column's weight times 2^(twice the change of its
// potential in this step, in base-2 units)): the one-sweep form's exponentials have no running
// maximum under them, so terms below 2^-126 are lost and sums above 2^127 overflow.  Its
// results count while every sum lies in [2^-80, 2^60] (what is lost is then below 2^-29 of any
// sum even with a million terms), and the step after a step whose sums all lie in [2^-56, 2^24]
// may run it, under whatever eps that step comes with: on a flat plan (large eps) the sums
// hardly move when eps changes, which is where a schedule of decreasing eps spends its first
// steps; where they do move, the check above catches it and the permission is gone until a
// two-sided step has given it again.
constexpr float kSweepFailLo = -80.f, kSweepFailHi = 60.f, kSweepOkLo = -56.f, kSweepOkHi = 24.f;
// lse_coarse_kernel leaves margin entries behind once a side's largest bias change is below this
// many base-2 units (lse_sparse_kernel takes over below 256)
constexpr float kSettleBelow = FS_SETTLE, kUnsettleAbove = 4.0f * FS_SETTLE;
constexpr float kEntriesBelow = FS_ENTRIES_BELOW;
// ... for the units that end at the test by at least this many base-2 units
constexpr float kEntryMargin = FS_ENTRY_MARGIN;
constexpr unsigned kSelDecideSteps = 3;  // which counted launch of the coarse variant decides
constexpr unsigned kSelMinPercent = 40;  // keep it while this share of units ends at the test
// Back to it once the plain kernel leaves out the exponentials of a larger share of its units
// than in its first launch of this stretch, by this many 65536ths (4 %).  The plain kernel finds
// its running maxima on the way and always leaves out the padding, so its share says little by
// itself (1 - 2 % on a flat plan, 7 - 20 % where the coarse variant would end 80 %), but its
// growth does; measured against the stretch's own first launch, a plan that stays as it is
// never sends the choice back and forth.
constexpr unsigned kSelBackStep16 = 2621;

// One wavefront: add the launch's counters to the totals and clear them.  Only workgroups whose
// rows all started from a key of the previous launch count, and the share of ended units climbs
// over the first launches that have such keys: the kSelDecideSteps-th launch with counts decides,
// and leaves the coarse variant when too few of its units ended at the test.
// After a launch that used carried margins: this launch's bias change joins the running sum.
// Which form of lse_coarse_kernel runs for a side: the sparse one once the side's largest bias
// change since its last launch is below 256 base-2 units (the change about halves from step to
// step of a solve, so margins of a few times that outlast the rest of it; on a peaked plan most
// are larger), and on until it is above 1024 again; the pipelined one before, and when a
// generation starts.
// lscale: base-2 units per raw unit.
// The launch's largest key-bias change for a side (raw units): the largest of its slots (bit
// patterns of non-negative floats, or of +inf, order like unsigned integers).
__device__ __forceinline__ float side_dmax(const unsigned* st, int side) {
  unsigned m = 0u;
#pragma unroll
  for (int i = 0; i < kDmaxSlots; ++i) m = max(m, st[kSelDmax + side * kDmaxSlots + i]);
  return __builtin_bit_cast(float, m);
}

__device__ __forceinline__ bool margins_settled(const unsigned* st, int side, float lscale) {
  if (st[kSelBump + side] != 0u || st[kSelGen + side] > 255u || st[kSelHave + side] == 0u) return false;
  const float d = side_dmax(st, side) * lscale;
  return d < (st[kSelMode + side] != 0u ? kUnsettleAbove : kSettleBelow);  // false when d is not a number
}

// What the merge kernel does to the state words after a launch, by one wavefront.  Every word is
// read before any is written (they live in one buffer, and loads placed behind stores to it would
// each wait for their own round trip: the chain used to be the longest thing in the kernel).
//   * the launch's unit counters join the totals and are cleared; the kSelDecideSteps-th launch
//     of the coarse variant with counts decides, and leaves it when too few of its units ended;
//     the plain kernel counts the units whose exponentials it left out, and a launch that left
//     out clearly more than the first of its stretch hands the next one back to the coarse variant;
//   * per side with carried margins (`commit_sides` of them, their matrices' roles in
//     `role`, base-2 units per raw unit in `lscale`): the launch's largest bias change joins the
//     running sum (or starts it, after a launch that began a generation), and the form that ran
//     is remembered for the hysteresis of margins_settled.
__device__ __forceinline__ void state_after_launch(unsigned* st, int lane, int commit_sides,
                                                   const int (&role)[2], const float (&lscale)[2]) {
  // ---- loads ----
  const unsigned e = st[kSelEnded + lane], u = st[kSelUnits + lane], k = st[kSelSkip + lane];
  const unsigned long long* cum64 = reinterpret_cast<const unsigned long long*>(st + kSelCumEnded);
  const unsigned long long c0 = cum64[0], c1 = cum64[1], c2 = cum64[2];
  const unsigned seen = st[kSelDecisions], word = st[kSelWord], base = st[kSelBase];
  unsigned bump[2] = {0u, 0u}, gen[2] = {0u, 0u}, mode[2] = {0u, 0u}, dmax[2] = {0u, 0u}, cum[2] = {0u, 0u};
  unsigned have[2] = {0u, 0u};
#pragma unroll
  for (int i = 0; i < 2; ++i)
    if (i < commit_sides) {
      bump[i] = st[kSelBump + role[i]];
      gen[i] = st[kSelGen + role[i]];
      mode[i] = st[kSelMode + role[i]];
      cum[i] = st[kSelCum + role[i]];
      have[i] = st[kSelHave + role[i]];
    }
  // (lanes 0..31: the slots of both roles)
  unsigned dslot = lane < 2 * kDmaxSlots ? st[kSelDmax + lane] : 0u;
  // ---- the decision ----
  unsigned long long es = e, us = u, ks = k;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    es += __shfl_xor(es, o, 64);
    us += __shfl_xor(us, o, 64);
    ks += __shfl_xor(ks, o, 64);
  }
#pragma unroll
  for (int o = kDmaxSlots / 2; o > 0; o >>= 1) dslot = max(dslot, (unsigned)__shfl_xor((int)dslot, o, 64));
  const unsigned d_role0 = (unsigned)__shfl((int)dslot, 0, 64), d_role1 = (unsigned)__shfl((int)dslot, kDmaxSlots, 64);
#pragma unroll
  for (int i = 0; i < 2; ++i)
    if (i < commit_sides) dmax[i] = role[i] ? d_role1 : d_role0;
  st[kSelEnded + lane] = 0u;
  st[kSelUnits + lane] = 0u;
  st[kSelSkip + lane] = 0u;
  // the slots of the roles that are committed below start the next launch at zero
#pragma unroll
  for (int i = 0; i < 2; ++i)
    if (i < commit_sides && lane >= role[i] * kDmaxSlots && lane < (role[i] + 1) * kDmaxSlots)
      st[kSelDmax + lane] = 0u;
  if (lane == 0 && us > 0) {
    unsigned long long* out = reinterpret_cast<unsigned long long*>(st + kSelCumEnded);
    out[0] = c0 + es;
    out[1] = c1 + us;
    out[2] = c2 + ks;
    if (word == 0u) {
      if (seen < kSelDecideSteps) {  // the share of the last of these launches decides
        st[kSelDecisions] = seen + 1u;
        if (seen + 1u == kSelDecideSteps && es * 100ull < us * (unsigned long long)kSelMinPercent) {
          st[kSelWord] = 1u;
          st[kSelBase] = 0u;  // the plain kernel's next launch sets the mark for the way back
        }
      }
    } else {
      const unsigned share16 = (unsigned)((es << 16) / us);
      if (base == 0u) {
        st[kSelBase] = share16 + 1u;
      } else if (share16 >= base - 1u + kSelBackStep16) {
        // the plain kernel leaves out clearly more than when this stretch began: the plan has
        // become peaked (eps went down), and the coarse variant gets its launches with counts again
        st[kSelWord] = 0u;
        st[kSelDecisions] = 0u;
        st[kSelBase] = 0u;
        st[kSelSweep] = 0u;  // (the one-sweep form's permission is not kept up by the other variant)
      }
    }
  }
  // ---- carried margins ----
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      if (i < commit_sides && !(i == 1 && role[1] == role[0])) {
        const float d = __builtin_bit_cast(float, dmax[i]) * lscale[i];
        const bool settled = bump[i] == 0u && gen[i] <= 255u && have[i] != 0u &&
                             d < (mode[i] != 0u ? kUnsettleAbove : kSettleBelow);  // margins_settled
        st[kSelMode + role[i]] = settled ? 1u : 0u;
        // entries of this generation: none after a launch that began one; there once the sparse
        // form ran or lse_coarse_kernel left some behind (its own condition, see there)
        const bool wrote = settled || (bump[i] == 0u && gen[i] <= 255u && d < kEntriesBelow);
        st[kSelHave + role[i]] = bump[i] != 0u ? 0u : ((have[i] != 0u || wrote) ? 1u : 0u);
        const float cnew = bump[i] ? 0.f : __builtin_bit_cast(float, cum[i]) + __builtin_bit_cast(float, dmax[i]);
        st[kSelCum + role[i]] = __builtin_bit_cast(unsigned, cnew);
        st[kSelBump + role[i]] = 0u;
      }
  }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Smallest value over the wavefront (DPP row shifts, then row broadcasts; lane 63 holds it).
__device__ __forceinline__ float wave_min_f32(float v) {
  int x = __builtin_bit_cast(int, v);
#define FS_MIN_STEP(ctrl, rmask, bmask)                                                          \
  {                                                                                               \
    const int o = __builtin_amdgcn_update_dpp(x, x, ctrl, rmask, bmask, false);                   \
    x = __builtin_bit_cast(int, fminf(__builtin_bit_cast(float, x), __builtin_bit_cast(float, o))); \
  }
  FS_MIN_STEP(0x111, 0xf, 0xf)  // row_shr:1
  FS_MIN_STEP(0x112, 0xf, 0xf)  // row_shr:2
  FS_MIN_STEP(0x114, 0xf, 0xe)  // row_shr:4
  FS_MIN_STEP(0x118, 0xf, 0xc)  // row_shr:8
  FS_MIN_STEP(0x142, 0xa, 0xf)  // row_bcast:15
  FS_MIN_STEP(0x143, 0xc, 0xf)  // row_bcast:31
#undef FS_MIN_STEP
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(x, 63));
}

// Carried margins of lse_coarse_kernel / lse_sparse_kernel.  A unit (32 keys x 32 query rows)
// that ended at the coarse test with margin mg (how far its bound stayed below the point where
// a logit could matter, the smallest over its rows; negative: the unit went on) gets the entry
//   mg - wslack + cum2,   cum2 = 2.002 * (sum of the largest key-bias changes of all launches
//                                         of this generation up to and including this one),
// rounded down into the upper 24 bits of a word whose low 8 bits name the generation.  Between
// two launches a logit rises by at most the largest bias change D, and a row's starting value
// (its logit at the key that held its maximum) lies at most D + wslack below that maximum: the
// unit ends again for as long as its entry exceeds the cum2 of the launch that asks.  0: no entry.
__device__ __forceinline__ unsigned margin_entry(float mg, float wslack, float cum2, unsigned gen) {
  const float v = mg - wslack + cum2;
  if (!(mg >= 0.f) || !(v > 0.f) || !(v <= 3.0e38f)) return 0u;
  return (__builtin_bit_cast(unsigned, v) & ~0xFFu) | gen;
}

__device__ __forceinline__ bool margin_entry_holds(unsigned w, unsigned gen, unsigned cum2_bits) {
  return (w & 0xFFu) == gen && (int)(w & ~0xFFu) > (int)cum2_bits;
}

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

__device__ __forceinline__ bool wave_any(bool p) { return __builtin_amdgcn_ballot_w64(p) != 0ull; }

// Power of two that maps a largest magnitude `mx` into [2^14, 2^15); 1 for zero / denormal
// / non-finite maxima, exponent clamped to +-40.
__device__ __forceinline__ float f16_plane_scale(float mx) {
  const int e = (int)((__builtin_bit_cast(unsigned, mx) >> 23) & 255u);
  if (e == 0 || e == 255) return 1.0f;
  int se = 14 - (e - 127);
  se = max(-40, min(40, se));
  return __builtin_bit_cast(float, (unsigned)(127 + se) << 23);
}

__device__ __forceinline__ unsigned pack_f16(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, f16x2));
}

}  // namespace fs
