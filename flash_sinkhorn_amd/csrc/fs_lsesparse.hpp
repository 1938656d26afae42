// Log-sum-exp on settled potentials: the form of the coarse tile test that visits only the units
// (32 keys x 32 query rows) whose carried margin may have been used up (fp16 planes, d <= 64).
//
// lse_coarse_kernel tests every unit after its hi*hi plane product.  Once the potentials move
// little from launch to launch, nearly every unit ends at that test again and again, by about the
// same margin.  This kernel keeps the margins (one 32-bit entry per unit, see margin_entry) and
// skips a unit for as long as its entry proves that it would end: what is left per launch are the
// units that hold logits near their rows' maxima (a few per cent on a peaked plan) and those
// whose margin the bias changes since their last test have used up.
//
// Work comes in items: 64 query rows (two blocks of 32, planes in registers) against one key
// range (several key chunks in a row; the merge kernel gets one partial result per piece of an
// item and is told how many there are).  The lists of units to visit differ a lot in length
// from item to item (a few rows far from every cluster have near keys everywhere), so items
// are not tied to workgroups: the launch is two workgroups per CU whose wavefronts stay and
// take items from a counter, one queue per XCD and side (workgroup id % 8 is the XCD, and each
// XCD serves its own key ranges, whose keys stay in its L2).  A wavefront that finds a list
// much longer than kPiece units cuts it: it pushes the remainder (the same rows against the
// rest of the range, as a partial result of its own) into the XCD's second queue, works
// through its piece, and takes the remainder back unless a wavefront that had run out of items
// has taken it in the meantime.  Nothing ever waits for anything: a pushed remainder is claimed
// with one atomic exchange by whoever gets there first, its owner included.
// Per item a wavefront
//   1. reads the entries of its two row blocks for the range together with its query planes and
//      starting values (one round of loads), and keeps, as bit masks in LDS, which units it has
//      to visit: a unit is visited unless its own entry holds and every row of its own block
//      starts where the row's last maximum says (a block with a row for which that fails visits
//      all its units and only writes entries);
//   2. walks the list with the operands of three 32-key sub-tiles in flight, read straight from
//      the copy of the planes in MFMA operand order (hi and lo plane, the a_j piece and the
//      biases of coarse_bias_kernel's records: ten 1 KiB loads per sub-tile);
//   3. per listed unit: the a_j step and the hi*hi product, the test, then either the new entry
//      or the two cross products, the exact bias and the soft-max (as in lse_coarse_kernel).
//
// Everything is exact: a unit that is not visited is one that would have ended at the test; the
// pieces of a list are disjoint sets of keys with partial results of their own, and which
// wavefront works on a piece changes nothing in it.
#pragma once

#include "fs_common.hpp"
#include "fs_stream.hpp"

namespace fs {

#ifndef FS_PIECE
#define FS_PIECE 48
#endif
constexpr int kPiece = FS_PIECE;  // units after which a long list is cut (at the next 32 sub-tiles)

template <int DP>
__global__ __launch_bounds__(256, 2) void lse_sparse_kernel(const LaunchArgs args) {
  static_assert(DP == 16 || DP == 32 || DP == 64, "two-plane rows of at most 64 columns");
  constexpr int RB = 2;            // blocks of 32 query rows per wavefront
  constexpr int KK16 = DP / 16;    // MFMAs of one plane product
  constexpr int kActWords = 64;    // list of units to visit: 32 sub-tiles (64 units) per word
  constexpr int kUpFront = 8;      // words of the list whose entries are read with the planes
  constexpr unsigned long long kTaken = ~0ull;

  __shared__ unsigned long long lds_act[4][kActWords];
  // and which of the listed units went on to the soft-max when they were last visited
  __shared__ unsigned long long lds_full[4][kActWords];
  __shared__ unsigned lds_cnt[4];  // the workgroup's unit counts, wavefronts done

  // the device chose the plain kernel: nothing to do
  if (args.sel_pred && args.sel[kSelWord] != args.sel_want) return;

  const int xcd = blockIdx.x & 7;
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int h = lane >> 5;
  if (tid < 4) lds_cnt[tid] = 0u;
  __syncthreads();  // the only barrier of this kernel

  auto mfma16 = [](const u32x4& a, const u32x4& b, const f32x16& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
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
  auto uniform = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
  // query side of the a_j step: 2^15 in the eight slots of the lower half-wave, nothing above
  const unsigned qcw = h ? 0u : 0x78007800u;
  const u32x4 QC = {qcw, qcw, qcw, qcw};

  unsigned tot_ended = 0, tot_skipped = 0, tot_units = 0;  // over all items of this wavefront

  // one side after the other (with half of the workgroups starting on either side, an XCD's L2
  // had to hold a key range of each matrix at once, and the launch was slower)
  for (int s_idx = 0; s_idx < args.sparse_sides; ++s_idx) {
    const Side& sd = args.side[s_idx];
    // ---- the state words: does this form run for the side? ----
    const int side_i = sd.ps_q;  // the margins' state goes with the matrix that holds the query rows
    const unsigned* st = args.sel;
    const unsigned gen = st[kSelGen + side_i];
    const float dnow = side_dmax(st, side_i);
    // MFMAs produce raw products of the scaled planes; lscale turns them into base-2 logits
    const float lscale = sd.qscale / (sd.plane_scale[sd.ps_q] * sd.plane_scale[sd.ps_k]);
    if (!margins_settled(st, side_i, lscale)) continue;  // the pipelined form runs this launch
    const float inv_lscale = 1.0f / lscale;
    const float skip_below = args.skip_log2 * inv_lscale;  // the 2^40 distance in raw units (< 0)
    const float cum2 = 2.002f * (__builtin_bit_cast(float, st[kSelCum + side_i]) + dnow);
    const unsigned cum2_bits = __builtin_bit_cast(unsigned, cum2);  // not finite: no entry holds
    const bool track = sd.best_key != nullptr;
    if (blockIdx.x == 0 && tid == 0) args.sel[kSelForm + side_i] = 2u;  // for the merge kernel

    // Base items of the side, key range slowest: item i = (range i / nwv, row group i % nwv).
    // Each XCD takes a contiguous run of them (with eight ranges: one range).
    const int group = sd.sparse_group;
    const int nsplit = (sd.splits + group - 1) / group;
    const int nwv = sd.igroups * 4;
    const int n_items = nwv * nsplit;
    const int per_xcd = (n_items + 7) / 8;
    // (a wavefront that went on to another XCD's queue once its own was empty made the launch
    // slower: far keys cost more than the idling at the end)
    const int it_begin = xcd * per_xcd, it_end = min(n_items, it_begin + per_xcd);
    unsigned* q = args.queue + (size_t)(s_idx * 8 + xcd) * kQueueWords;
    unsigned long long* slots = reinterpret_cast<unsigned long long*>(q + kQueueSlot0);
    auto pop_base = [&]() -> int {
      int v = 0;
      if (lane == 0)
        v = (int)__hip_atomic_fetch_add(q + kQueueBase, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return it_begin + uniform(v);
    };
    // a remainder from the second queue: (row group, piece, first list word), or -1
    auto pop_rest = [&](int& p, int& g0) -> int {
      unsigned long long v = 0ull;
      if (lane == 0) {
        const unsigned hd = __hip_atomic_load(q + kQueueHead, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned tl = __hip_atomic_load(q + kQueueTail, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (hd < min(tl, (unsigned)kQueueSlots)) {
          const unsigned i = __hip_atomic_fetch_add(q + kQueueHead, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (i < (unsigned)kQueueSlots)
            v = __hip_atomic_exchange(slots + i, kTaken, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          else
            v = 1ull;  // past the end: nothing there, nothing to come
        } else {
          v = 1ull;    // empty right now: whoever pushes later looks after it himself
        }
      }
      const unsigned lo32 = (unsigned)uniform((int)(unsigned)v), hi32 = (unsigned)uniform((int)(unsigned)(v >> 32));
      if (hi32 == 0u && lo32 == 1u) return -1;        // queue empty
      if ((hi32 == 0u && lo32 == 0u) || (hi32 == ~0u && lo32 == ~0u)) return -2;  // a slot without an item
      p = (int)(hi32 >> 16) & 0xFF;
      g0 = (int)(hi32 & 0xFFFFu);
      return (int)lo32;
    };

    int cur = pop_base();
    for (;;) {
      // ---- the next item ----
      int item_w, item_r, piece = 0, g_first = 0;
      if (cur < it_end) {
        item_r = cur / nwv;
        item_w = cur % nwv;
        cur = pop_base();  // (the answer is not needed before this item is done)
      } else {
        const int got = pop_rest(piece, g_first);
        if (got == -1) break;
        if (got == -2) continue;
        item_r = got / nwv;
        item_w = got % nwv;
      }
      const int split = item_r * group;
      const int row0 = item_w * (32 * RB);
      const int j_begin = split * sd.chunk;
      const int j_end = min(sd.nk, j_begin + group * sd.chunk);
      const int n_sub = ((j_end - j_begin + 127) / 128) * 4;  // whole 128-key tiles, as the other form
      const int n_groups = (n_sub + 31) / 32;
      if (n_sub <= 0) continue;

      // ---- one round of loads: query planes, starting values, last maxima, entries ----
      u32x4 xq[RB][2][KK16];  // [block][plane][16-column step], from the copy in operand order
      float warm[RB], mprev[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int row = min(row0 + rb * 32 + li, sd.nq - 1);
        const unsigned* qt = sd.qtiled + (size_t)(row / 32) * (2 * KK16 * 256) + (h * 32 + row % 32) * 4;
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int kk = 0; kk < KK16; ++kk)
            xq[rb][p][kk] = *reinterpret_cast<const u32x4*>(qt + (p * KK16 + kk) * 256);
        warm[rb] = track ? sd.seed[row] : -3.0e38f;
        mprev[rb] = sd.m_prev[row];
      }
      // this item's entries: entry 2 s + rb for sub-tile s (counted from the range's first key)
      unsigned* ent = reinterpret_cast<unsigned*>(sd.margins) +
                      ((size_t)item_w * (size_t)sd.margin_stride + (size_t)(j_begin / 32)) * 2;
      unsigned ew[kUpFront];
#pragma unroll
      for (int u = 0; u < kUpFront; ++u) ew[u] = ent[min((g_first + u) * 64 + lane, 2 * n_sub - 1)];

      // Bound on the two cross products of a row, in raw units (see lse_coarse_kernel).
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

      // ---- which units to visit ----
      const bool fits = n_groups <= kActWords;  // else: everything is visited, list or no list
      bool have = track;  // a row without a key (first launches on new planes) starts from nothing
      float wslack = 0.f;
      unsigned long long blk_ok[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        have = have && warm[rb] > -3.0e38f;
        const float sl = corr[rb] * 0x1p-6f + 2.0f * inv_lscale;
        wslack = fmaxf(wslack, sl);
        // the row starts where its last maximum says (overwritten keys fail this)
        const bool ok = track && warm[rb] > -3.0e38f &&
                        warm[rb] >= mprev[rb] * inv_lscale - 1.001f * dnow - sl;
        blk_ok[rb] = __builtin_amdgcn_ballot_w64(ok) == ~0ull ? ~0ull : 0ull;
      }
      const bool cold = __builtin_amdgcn_ballot_w64(!have) != 0ull;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) wslack = fmaxf(wslack, __shfl_xor(wslack, o, 64));
      // units of list word g that exist: two bits per sub-tile, block 0 in the even one
      auto group_mask = [&](int g) -> unsigned long long {
        const int left = n_sub - g * 32;
        return left >= 32 ? ~0ull : ((1ull << (2 * left)) - 1ull);
      };
      const bool listed = fits && track && !cold;  // else: every unit is visited
      // entries of blocks that may not use theirs count as used up
      const unsigned long long usable_bits = (blk_ok[0] & 0x5555555555555555ull) |
                                             (blk_ok[1] & 0xAAAAAAAAAAAAAAAAull);
      if (fits) {
#pragma unroll
        for (int u = 0; u < kUpFront; ++u) {
          const int g = g_first + u;
          const unsigned long long v = __builtin_amdgcn_ballot_w64(
              g * 64 + lane < 2 * n_sub && margin_entry_holds(ew[u], gen, cum2_bits));
          const unsigned long long f = __builtin_amdgcn_ballot_w64(ew[u] == gen);
          if (g < n_groups && lane == 0) {
            lds_act[wave][g] = listed ? (~(v & usable_bits) & group_mask(g)) : group_mask(g);
            lds_full[wave][g] = f;
          }
        }
        for (int g = g_first + kUpFront; g < n_groups; ++g) {  // longer ranges: the rest of the list
          const unsigned w = ent[min(g * 64 + lane, 2 * n_sub - 1)];
          const unsigned long long v = __builtin_amdgcn_ballot_w64(
              g * 64 + lane < 2 * n_sub && margin_entry_holds(w, gen, cum2_bits));
          const unsigned long long f = __builtin_amdgcn_ballot_w64(w == gen);
          if (lane == 0) {
            lds_act[wave][g] = listed ? (~(v & usable_bits) & group_mask(g)) : group_mask(g);
            lds_full[wave][g] = f;
          }
        }
      }
      auto uniform64 = [&](unsigned long long m) -> unsigned long long {
        const unsigned lo32 = (unsigned)uniform((int)(unsigned)m), hi32 = (unsigned)uniform((int)(unsigned)(m >> 32));
        return ((unsigned long long)hi32 << 32) | lo32;
      };
      auto list_word = [&](int g) -> unsigned long long {
        return fits ? uniform64(lds_act[wave][g]) : group_mask(g);
      };
      auto full_word = [&](int g) -> unsigned long long {
        return fits ? uniform64(lds_full[wave][g]) : 0ull;
      };

      // run_m: running maximum in raw units; run_c = -run_m * lscale as rounded once, the offset
      // every exponent of the row uses (rescaling by differences of run_c stays consistent)
      float run_m[RB], run_s[RB], run_c[RB];
      int best_j[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        run_m[rb] = warm[rb];
        run_s[rb] = 0.f;
        best_j[rb] = -1;
        float c = -run_m[rb] * lscale;
        asm volatile("" : "+v"(c));  // the rounded product itself, nothing fused into later uses
        run_c[rb] = c;
      }

      unsigned n_ended = 0, n_visited = 0;

      // One listed unit: row block rb against the sub-tile whose operands are (hi, lo, ka, bm, kb).
      // was_full: the unit went on to the soft-max when it was last visited, and will again: no
      // test, the exact logits right away.
      auto unit = [&](const u32x4 (&hi)[KK16], const u32x4 (&lo)[KK16], const u32x4& ka, float bm,
                      float kb, int rb, int kbase, bool was_full) -> unsigned {
        f32x16 L;
#pragma unroll
        for (int r = 0; r < 16; ++r) L[r] = 0.f;
        L = mfma16(ka, QC, L);  // 2^18 a_j on every query column
#pragma unroll
        for (int kk = 0; kk < KK16; ++kk) L = mfma16(hi[kk], xq[rb][0][kk], L);
        if (!was_full) {
          const float thr = run_m[rb] + (skip_below - bm) - corr[rb];
          const float mxh = max16(L);
          if (!wave_any(mxh > thr)) {  // ends again: by how much
            ++n_ended;
            return margin_entry(wave_min_f32(thr - mxh), wslack, cum2, gen);
          }
        }
        // goes on: the two cross products and the exact key bias on top, then the soft-max
#pragma unroll
        for (int kk = 0; kk < KK16; ++kk) L = mfma16(hi[kk], xq[rb][1][kk], L);
#pragma unroll
        for (int kk = 0; kk < KK16; ++kk) L = mfma16(lo[kk], xq[rb][0][kk], L);
        // the key bias added to every query column: A = [bias_j, 1], B = [1, 0]
        L = __builtin_amdgcn_mfma_f32_32x32x2f32(h ? 1.0f : kb, h ? 0.0f : 1.0f, L, 0, 0, 0);
        const float mx = max16(L);  // this lane's 16 keys
        // every logit of the unit more than the 2^40 distance below its row's running maximum:
        // its exponentials would not change the fp32 row sums
        if (!wave_any(mx - run_m[rb] > skip_below)) {
          // The exact logits say so: the unit gets an entry from them (they rise and the rows'
          // starting values fall like the bounds of the test do; see margin_entry), and is not
          // visited again while that holds.
          ++n_ended;
          return margin_entry(wave_min_f32(run_m[rb] + skip_below - mx), wslack, cum2, gen);
        }
        {
          float a = mx, b2 = mx;
          swap_halves(a, b2);
          const float m_new = fmaxf(fmaxf(a, b2), run_m[rb]);
          if (track && wave_any(m_new > run_m[rb])) {
            // the maximum of a row moves: the half-wave that holds the new one notes its key
            // (register r of a lane is key 8 (r / 4) + 4 h + r % 4 of the sub-tile), the other
            // half forgets its own
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
        return gen;  // no margin: visited again next launch, and then without the test
      };

      // Operands of a listed sub-tile come straight from global memory (key planes and bias
      // records are L2 residents), NSET sub-tiles ahead; the slots of a wavefront that has run
      // out of sub-tiles reload its first one, so that every pass issues the same loads.
      constexpr int NSET = 3;
      u32x4 SH[NSET][KK16], SL[NSET][KK16], SA[NSET];
      float SB[NSET], SK[NSET];
      int SS[NSET];
      unsigned SN[NSET];
      auto load_set = [&](u32x4 (&hi)[KK16], u32x4 (&lo)[KK16], u32x4& ka, float& bm, float& kb, int s2) {
        const int sc = max(s2, 0);
        const int kbase = j_begin + 32 * sc;
        const unsigned* blk = sd.ktiled + (size_t)(kbase / 32) * (2 * KK16 * 256) + lane * 4;
#pragma unroll
        for (int kk = 0; kk < KK16; ++kk) hi[kk] = *reinterpret_cast<const u32x4*>(blk + kk * 256);
        const unsigned* rec = sd.key_aux + (size_t)(kbase / 64) * kAuxWords;
        ka = *reinterpret_cast<const u32x4*>(rec + kAuxA + ((sc & 1) * 32 + li) * 4);
        bm = __builtin_bit_cast(float, rec[kAuxMax + (sc & 1)]);
#pragma unroll
        for (int kk = 0; kk < KK16; ++kk) lo[kk] = *reinterpret_cast<const u32x4*>(blk + (KK16 + kk) * 256);
        kb = __builtin_bit_cast(float, rec[kAuxB + (sc & 1) * 32 + li]);
      };

      // ---- the list, piece by piece: words [g_it, g_stop) at a time ----
      int g_it = g_first, g_stop = n_groups;
      const int my_piece = piece;  // which partial result of the range this wavefront fills; a
                                   // remainder handed to somebody else fills the next one
      for (;;) {
        // A list much longer than a piece is cut at a word boundary and the rest offered to
        // wavefronts that have run out of items.
        int pushed = -1;
        unsigned long long pushed_item = 0ull;
        g_stop = n_groups;
        if (my_piece + 1 < group) {
          int total = 0, g_cut = -1;
          for (int g = g_it; g < n_groups; ++g) {
            total += __builtin_popcountll(list_word(g));
            if (g_cut < 0 && total >= kPiece) g_cut = g + 1;
          }
          if (g_cut > 0 && g_cut < n_groups && total > kPiece + kPiece / 2) {
            pushed_item = ((unsigned long long)(((unsigned)(my_piece + 1) << 16) | (unsigned)g_cut) << 32) |
                          (unsigned)(item_r * nwv + item_w);
            int slot = -1;
            if (lane == 0) {
              const unsigned t = __hip_atomic_fetch_add(q + kQueueTail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              if (t < (unsigned)kQueueSlots) {
                const unsigned long long was = __hip_atomic_exchange(slots + t, pushed_item, __ATOMIC_RELAXED,
                                                                     __HIP_MEMORY_SCOPE_AGENT);
                // (a wavefront that looked into the slot before the item was there has marked it:
                // nobody will come for it)
                if (was == 0ull) slot = (int)t;
              }
            }
            pushed = uniform(slot);
            if (pushed >= 0) g_stop = g_cut;
          }
        }
        // ---- walk words [g_it, g_stop) ----
        int base_it = 0;
        unsigned long long m_it = 0ull;
        unsigned long long f_it = 0ull;
        // (need: bits 0, 1 = the listed units of the sub-tile, bits 2, 3 = which of them went on last time)
        auto next = [&](unsigned& need) -> int {
          while (m_it == 0ull) {
            if (g_it >= g_stop) return -1;
            m_it = list_word(g_it);
            f_it = full_word(g_it);
            base_it = g_it * 32;
            ++g_it;
          }
          const int k = __builtin_ctzll(m_it) >> 1;
          need = ((unsigned)(m_it >> (2 * k)) & 3u) | (((unsigned)(f_it >> (2 * k)) & 3u) << 2);
          m_it &= ~(3ull << (2 * k));
          return base_it + k;
        };
#pragma unroll
        for (int i = 0; i < NSET; ++i) {
          SN[i] = 0u;
          SS[i] = next(SN[i]);
          load_set(SH[i], SL[i], SA[i], SB[i], SK[i], SS[i]);
        }
        while (SS[0] >= 0) {
#pragma unroll
          for (int i = 0; i < NSET; ++i) {
            if (SS[i] >= 0) {
              const int kbase = j_begin + 32 * SS[i];
              if (SN[i] & 1u) {
                const unsigned e = unit(SH[i], SL[i], SA[i], SB[i], SK[i], 0, kbase, (SN[i] & 4u) != 0u);
                if (lane == 0) ent[2 * SS[i]] = e;
                ++n_visited;
              }
              if (SN[i] & 2u) {
                const unsigned e = unit(SH[i], SL[i], SA[i], SB[i], SK[i], 1, kbase, (SN[i] & 8u) != 0u);
                if (lane == 0) ent[2 * SS[i] + 1] = e;
                ++n_visited;
              }
            }
            SS[i] = SS[i] >= 0 ? next(SN[i]) : -1;
            load_set(SH[i], SL[i], SA[i], SB[i], SK[i], SS[i]);
          }
        }
        if (pushed < 0) break;  // that was the rest of the range
        // the remainder: still there?  Then it is this wavefront's again (same rows, same partial
        // result, and the piece number it carried was never used); else somebody else has it,
        // with a partial result of its own, and looks after the rest of the range.
        unsigned long long was = 0ull;
        if (lane == 0)
          was = __hip_atomic_exchange(slots + pushed, kTaken, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool mine = uniform((int)(was == pushed_item)) != 0;
        if (!mine) break;
      }
      const bool to_the_end = g_stop >= n_groups;  // this wavefront did the last piece of the range

      // units of this piece (words [g_first, g_it)) for the counters
      const unsigned n_units = (unsigned)((min(g_it * 32, n_sub) - g_first * 32) * RB);
      if (!(track && cold)) {
        tot_ended += n_ended + (n_units - n_visited);
        tot_skipped += n_units - n_visited;
        tot_units += n_units;
      }

      // ---- the partial result of this piece ----
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int row = row0 + rb * 32 + li;
        const float s = run_s[rb] + xor32(run_s[rb]);
        const float M2 = -run_c[rb];
        int bj = best_j[rb];
        const int oj = __shfl_xor(bj, 32, 64);
        if (bj < 0) bj = oj;
        if (row < sd.nq && h == 0) {
          const size_t pr = (size_t)(split + my_piece) * (size_t)sd.nq + (size_t)row;
          *reinterpret_cast<float2*>(&sd.part_ms[2 * pr]) = make_float2(M2, s);
          if (sd.part_best != nullptr) sd.part_best[pr] = bj;
        }
      }
      // the wavefront that reaches the end of the range says how many partial results it has
      if (to_the_end && lane == 0) sd.npieces[(size_t)item_w * nsplit + item_r] = (unsigned char)(my_piece + 1);
    }
  }

  // unit counts for the variant choice on the device.  The wavefronts of a workgroup end at
  // different times: they add up in LDS, and the last one out hands the workgroup's counts to
  // the state words (a quarter of the atomics)
  if (lane == 0) {
    const int slot = blockIdx.x % kSelSlots;
    atomicAdd(&lds_cnt[0], tot_ended);
    atomicAdd(&lds_cnt[1], tot_skipped);
    atomicAdd(&lds_cnt[2], tot_units);
    if (atomicAdd(&lds_cnt[3], 1u) == 3u && lds_cnt[2] != 0u) {
      atomicAdd(&args.sel[kSelEnded + slot], lds_cnt[0]);
      atomicAdd(&args.sel[kSelSkip + slot], lds_cnt[1]);
      atomicAdd(&args.sel[kSelUnits + slot], lds_cnt[2]);
    }
  }
}

}  // namespace fs
