// extern "C" entry points: argument checks, launch planning and kernel dispatch.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "flash_sinkhorn_hip.h"
#include "fs_common.hpp"
#include "fs_dispatch.hpp"
#include "fs_stream.hpp"

// Scratch of fs_symmetric_step_noalloc: lives in the code object, one copy per GPU that loads
// the library, held until the process ends.  In host code the name is only a handle for
// hipGetSymbolAddress; kernels and copies get the per-device address it returns.
constexpr size_t kScratchBytes = (size_t)48 << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace fs {
namespace {

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];  // address of `scratch` on each device, looked up once
std::mutex g_scratch_mutex;

// Address of the built-in scratch buffer on the current device (set-up on the first call there).
int scratch_on_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return FS_ERR_LAUNCH_FAILED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr)
      return FS_ERR_LAUNCH_FAILED;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return FS_OK;
}

constexpr int kMaxStreamD = 128;    // register-stationary streaming kernels
constexpr int kMaxSlicedD = 16384;  // widest supported rows
constexpr int kSlicedSpan = 1536;   // columns one workgroup of the column-sliced kernels spans
constexpr int kPlanePadRowsApi = 512;  // must match kPlanePadRows of the plane-splitting kernels
// after the planes: absmax partials [2][256], plane scales [4] (+4 spare), variant-choice state
// (a multiple of 256 bytes: the margin entries, queues and their 64-bit slots come right behind)
constexpr size_t kPlaneAuxBytes = ((2 * 256 + 8 + kSelWords) * sizeof(float) + 255) / 256 * 256;
static_assert(kSelWords <= 512, "the state is cleared by one workgroup");

inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

inline int padded_d(int64_t d) {
  if (d <= 8) return 8;
  if (d <= 16) return 16;
  if (d <= 32) return 32;
  if (d <= 64) return 64;
  return 128;
}

// Blocks a launch should reach before key splitting stops (8 and 4 per CU).
int target_blocks(bool has_o) { return has_o ? 1024 : 2048; }

struct SidePlan {
  int rb, igroups, splits, chunk;
};

// Which kernel family serves feature dimension d, and its tile geometry.
struct Family {
  int nss;       // sliced only: super-slices of kSlicedSpan columns
  bool sliced;
  int dp;        // padded feature width (also the width of partial O rows)
  int jt;        // keys per tile
  int nw, nsl;   // sliced only: wavefronts per workgroup, 32-column blocks per wavefront
};

Family family_for(int64_t d) {
  Family f;
  f.sliced = d > kMaxStreamD;
  f.nw = f.nsl = 0;
  f.nss = 1;
  if (!f.sliced) {
    f.dp = padded_d(d);
    f.jt = (f.dp >= 128) ? 32 : 64;
    return f;
  }
  if (d <= 256) { f.nw = 4; f.nsl = 2; }
  else if (d <= 512) { f.nw = 8; f.nsl = 2; }
  else if (d <= 1024) { f.nw = 8; f.nsl = 4; }
  else { f.nw = 8; f.nsl = 6; f.nss = ceil_div(d, kSlicedSpan); }
  f.dp = f.nss * f.nw * f.nsl * 32;
  f.jt = 32;
  return f;
}

// Rows per wavefront (RB blocks of 32) and the key split for one side.
SidePlan plan_side(int mode, int64_t nq, int64_t nk, const Family& fam, int rb_force = 0,
                   int min_splits = 1) {
  SidePlan p;
  const bool has_o = (mode == kMat || mode == kMat5);
  const int dp = fam.dp;
  const int jt = fam.jt;
  p.rb = 1;
  int target = target_blocks(has_o);
  if (fam.sliced) {
    p.igroups = ceil_div(nq, 32);
    target = 512;  // one workgroup of nw wavefronts per CU, two rounds
  } else {
    if (mode == kLse || mode == kVec) p.rb = (dp <= 64 && nq >= 2048) ? 2 : 1;
    if (mode == kMat) p.rb = (dp <= 32 && nq >= 2048) ? 2 : 1;
    if (rb_force > 0) p.rb = rb_force;
    p.igroups = ceil_div(nq, 128 * p.rb);
  }
  const int max_splits = (int)std::max<int64_t>(1, nk / (4 * jt));
  const int cap = has_o ? 16 : 64;
  int s = 1;
  while (p.igroups * s < target && s * 2 <= max_splits && s * 2 <= cap) s *= 2;
  s = std::max(s, min_splits);
  p.chunk = ceil_div(ceil_div(nk, s), jt) * jt;
  p.splits = ceil_div(nk, p.chunk);
  return p;
}

// Per-tile records of the key bias for lse_coarse_kernel (see coarse_bias_kernel).
size_t coarse_aux_bytes(int64_t nk) {
  return (size_t)(ceil_div(nk, 64) + kAuxPadTiles) * kAuxWords * sizeof(unsigned);
}

size_t side_ws_floats(int mode, const SidePlan& p, int64_t nq, int dp) {
  if (p.splits <= 1) return 0;
  size_t f = (size_t)p.splits * (size_t)nq * 2;
  if (mode == kVec || mode == kLse) f += (size_t)p.splits * (size_t)nq;  // kLse: Side::part_best
  if (mode == kMat || mode == kMat5) f += (size_t)p.splits * (size_t)nq * (size_t)dp;
  return (f + 3) & ~(size_t)3;  // keep the next region 16-byte aligned
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

template <int MODE, int DP, int RB, bool SEPV>
int launch_one(const LaunchArgs& a, int blocks, hipStream_t st) {
  hipLaunchKernelGGL((stream_kernel<MODE, DP, RB, SEPV>), dim3(blocks), dim3(256), 0, st, a);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

template <int MODE, int DP, bool SEPV>
int launch_rb(const LaunchArgs& a, int rb, int blocks, hipStream_t st) {
  if constexpr (MODE == kLse || MODE == kVec) {
    if constexpr (DP <= 64) {
      if (rb == 2) return launch_one<MODE, DP, 2, SEPV>(a, blocks, st);
    }
  }
  if constexpr (MODE == kMat) {
    if constexpr (DP <= 32) {
      if (rb == 2) return launch_one<MODE, DP, 2, SEPV>(a, blocks, st);
    }
  }
  return launch_one<MODE, DP, 1, SEPV>(a, blocks, st);
}

template <int MODE, bool SEPV>
int launch_dp(const LaunchArgs& a, int dp, int rb, int blocks, hipStream_t st) {
  switch (dp) {
    case 8: return launch_rb<MODE, 8, SEPV>(a, rb, blocks, st);
    case 16: return launch_rb<MODE, 16, SEPV>(a, rb, blocks, st);
    case 32: return launch_rb<MODE, 32, SEPV>(a, rb, blocks, st);
    case 64: return launch_rb<MODE, 64, SEPV>(a, rb, blocks, st);
    case 128: return launch_rb<MODE, 128, SEPV>(a, rb, blocks, st);
  }
  return FS_ERR_UNSUPPORTED;
}


// ---- 16-bit operand planes of the LSE kernels ----
// The workspace of an LSE operation starts with the planes of its distinct operand matrices in
// canonical order (ascending address), then the absmax partials and plane scales.  The layout
// depends only on (matrices, d, precision), never on which matrix is the stationary one, so
// planes written once by fs_prepare_operands serve every later step on the same operands.
struct LseConfig {
  bool gemm;    // lse_gemm_kernel (128 < d <= 1536, fp16 planes)
  int prec;     // Prec of lse2_kernel: kF32 (0) fp32 operands, kH3 (3) two fp16 planes
  int dp;       // padded columns of a plane row
  int np;       // planes per operand
};

// Words per row of the chunked fp16 planes: the 32-column chunks (128 bytes) of a row, plus
// one spare chunk when their count is even.  An odd count of 128-byte units per row spreads
// the rows of a stage (same chunk of 256 consecutive rows) over all memory channels.
int chunked_stride(int64_t d) { return (ceil_div(d, 32) | 1) * 32; }

LseConfig lse_config(int64_t d, uint32_t flags) {
  LseConfig c;
  c.prec = (flags & FS_FLAG_FP32_MFMA) ? 0 : 3;
  c.gemm = d > kMaxStreamD && c.prec == 3;
  c.dp = c.gemm ? chunked_stride(d) : std::max(padded_d(d), 16);
  c.np = 2;
  return c;
}

struct PlaneSet {
  int n;  // distinct matrices, 0 when the configuration uses no planes
  const float* src[2];
  int rows[2];
  size_t off[2];
  size_t aux_off, end;
  size_t margin_off, margin_slot;  // two slots of carried margins behind the aux block (0: none)
  size_t queue_off;                // behind them: the work queues of lse_sparse_kernel
  int margin_stride;               // sub-tiles per wavefront row of a slot
};

// Bytes of one matrix's planes alone, and of its whole region: the planes, then one int per row
// (the key behind the row's largest logit, kept from launch to launch of lse_coarse_kernel).
size_t planes_only_bytes(int64_t rows, const LseConfig& c) {
  return (((size_t)(rows + kPlanePadRowsApi) * (size_t)c.np * (size_t)(c.dp / 2) * 4) + 15) & ~(size_t)15;
}

// One 4-byte value per row, 16-byte aligned; a matrix keeps four such arrays behind its planes:
// the key behind each row's largest logit, that logit (the merged maximum of the last launch
// with the matrix as the stationary one), the row's bias of the last launch as a key, and where
// the row's running maximum starts in the launch under way.
size_t row_array_bytes(int64_t rows) { return ((size_t)rows * 4 + 15) & ~(size_t)15; }

// Second copy of two-plane rows of at most 64 columns in MFMA operand order (Side::ktiled),
// whole blocks of 32 rows.
size_t tiled_bytes(int64_t rows, const LseConfig& c) {
  if (c.gemm || c.prec != 3 || c.dp > 64) return 0;
  return (size_t)ceil_div(rows + kPlanePadRowsApi, 32) * 32 * (size_t)c.dp * 4;
}

size_t plane_bytes(int64_t rows, const LseConfig& c) {
  return planes_only_bytes(rows, c) + 4 * row_array_bytes(rows) + tiled_bytes(rows, c);
}

// Carried margins of lse_coarse_kernel: per wavefront (64 rows) and 32-key sub-tile two entries.
// A slot serves any pairing of the set's matrices as (stationary, streamed).
int margin_stride_for(int64_t max_rows) { return (ceil_div(max_rows, 128) + 1) * 4; }
size_t margin_slot_bytes(int64_t max_rows, const LseConfig& c) {
  if (c.gemm || c.prec != 3 || c.dp > 64) return 0;
  // wavefront rows in whole workgroups of four: the last workgroup's spare wavefronts keep entries too
  const size_t b = (size_t)ceil_div(max_rows, 256) * 4 * (size_t)margin_stride_for(max_rows) * 8;
  return b <= ((size_t)128 << 20) ? b : 0;
}

// Column sums of lse_sweep_kernel: one row of sums (over the keys) per workgroup row group of
// 256 query rows (n = m = 50,000: 39 MB, read once by the merge); problems with more row groups
// than this (262,144 rows: 1 GiB at as many keys) stay on the two-sided kernel.
constexpr int kSweepMaxGroups = 1024;
size_t sweep_col_bytes(int64_t nq, int64_t nk) {
  const int64_t groups = ceil_div(nq, 256);
  if (groups > kSweepMaxGroups || nq < 2048 || nk < 2048) return 0;
  return (((size_t)groups * (size_t)nk * 4) + 63) & ~(size_t)63;
}

// Piece counts of lse_sparse_kernel for one side of a launch: one byte per 64-row group and key
// range (at most 64 ranges).
size_t npieces_bytes(int64_t max_rows) { return ((size_t)ceil_div(max_rows, 256) * 4 * 64 + 15) & ~(size_t)15; }

// Everything behind the aux block that belongs to the carried margins: the two slots, the work
// queues of lse_sparse_kernel (64-bit slots: every part is a multiple of 16 bytes) and its piece
// counts for either side.
size_t margin_region_bytes(int64_t max_rows, const LseConfig& c) {
  const size_t slot = margin_slot_bytes(max_rows, c);
  return slot > 0 ? 2 * slot + kQueueBytes + 2 * npieces_bytes(max_rows) : 0;
}

// Distinct (pointer, rows) operands among up to four candidates, in canonical order.
int make_plane_set(const float* const* ptrs, const int* rows, int count, const LseConfig& c,
                   PlaneSet& ps) {
  ps.n = 0;
  ps.aux_off = ps.end = 0;
  ps.margin_off = ps.margin_slot = 0;
  ps.queue_off = 0;
  ps.margin_stride = 0;
  if (c.prec == 0) return FS_OK;
  for (int k = 0; k < count; ++k) {
    bool seen = false;
    for (int i = 0; i < ps.n; ++i) seen = seen || (ps.src[i] == ptrs[k] && ps.rows[i] == rows[k]);
    if (seen) continue;
    if (ps.n == 2) return FS_ERR_BAD_ARGUMENT;
    ps.src[ps.n] = ptrs[k];
    ps.rows[ps.n] = rows[k];
    ++ps.n;
  }
  if (ps.n == 2 && (ps.src[1] < ps.src[0] || (ps.src[1] == ps.src[0] && ps.rows[1] < ps.rows[0]))) {
    std::swap(ps.src[0], ps.src[1]);
    std::swap(ps.rows[0], ps.rows[1]);
  }
  size_t need = 0;
  for (int i = 0; i < ps.n; ++i) {
    ps.off[i] = need;
    need += plane_bytes(ps.rows[i], c);
  }
  ps.aux_off = need;
  ps.end = need + kPlaneAuxBytes;
  int64_t max_rows = 0;
  for (int i = 0; i < ps.n; ++i) max_rows = std::max<int64_t>(max_rows, ps.rows[i]);
  ps.margin_off = ps.end;
  ps.margin_slot = ps.n > 0 ? margin_slot_bytes(max_rows, c) : 0;
  ps.margin_stride = margin_stride_for(max_rows);
  ps.queue_off = ps.end + 2 * ps.margin_slot;
  ps.end += ps.n > 0 ? margin_region_bytes(max_rows, c) : 0;
  return FS_OK;
}

int plane_index(const PlaneSet& ps, const float* src, int rows) {
  for (int i = 0; i < ps.n; ++i)
    if (ps.src[i] == src && ps.rows[i] == rows) return i;
  return 0;
}

const float* plane_scales(const PlaneSet& ps, void* ws) {
  return reinterpret_cast<const float*>(static_cast<char*>(ws) + ps.aux_off) + 2 * 256;
}

unsigned* select_state(const PlaneSet& ps, void* ws) {
  return reinterpret_cast<unsigned*>(static_cast<char*>(ws) + ps.aux_off) + 2 * 256 + 8;
}

const unsigned* plane_of(const PlaneSet& ps, void* ws, const float* src, int rows) {
  for (int i = 0; i < ps.n; ++i)
    if (ps.src[i] == src && ps.rows[i] == rows)
      return reinterpret_cast<const unsigned*>(static_cast<char*>(ws) + ps.off[i]);
  return nullptr;
}

int* best_keys_of(const PlaneSet& ps, const LseConfig& c, void* ws, const float* src, int rows) {
  for (int i = 0; i < ps.n; ++i)
    if (ps.src[i] == src && ps.rows[i] == rows)
      return reinterpret_cast<int*>(static_cast<char*>(ws) + ps.off[i] + planes_only_bytes(rows, c));
  return nullptr;
}

float* row_array_of(const PlaneSet& ps, const LseConfig& c, void* ws, const float* src, int rows,
                    int which) {  // 1: last maxima, 2: last biases, 3: this launch's starting values
  int* keys = best_keys_of(ps, c, ws, src, rows);
  if (keys == nullptr) return nullptr;
  return reinterpret_cast<float*>(reinterpret_cast<char*>(keys) + which * row_array_bytes(rows));
}

unsigned* tiled_of(const PlaneSet& ps, const LseConfig& c, void* ws, const float* src, int rows) {
  if (tiled_bytes(rows, c) == 0) return nullptr;
  int* keys = best_keys_of(ps, c, ws, src, rows);
  if (keys == nullptr) return nullptr;
  return reinterpret_cast<unsigned*>(reinterpret_cast<char*>(keys) + 4 * row_array_bytes(rows));
}

// Writes the planes (and, for fp16, the scales) of every matrix of the set.  `keep`: the planes
// outlive the call (fs_prepare_operands): the carried margins start empty and the second copy
// in operand order, which only launches on kept planes read, is written too.
int launch_plane_set(const PlaneSet& ps, const LseConfig& c, int64_t d, void* ws, hipStream_t st,
                     bool keep = false, bool start_plain = false) {
  if (ps.n == 0) return FS_OK;
  char* base = static_cast<char*>(ws);
  int rc = FS_OK;
  if (keep && ps.margin_slot > 0)
    rc = launch_fill_zero(reinterpret_cast<unsigned*>(base + ps.margin_off),
                          (long long)(2 * ps.margin_slot / 4), st);
  if (rc != FS_OK) return rc;
  {
    float* partial = reinterpret_cast<float*>(base + ps.aux_off);
    float* scales = partial + 2 * 256;
    const bool two = ps.n > 1;
    rc = launch_absmax(ps.src[0], (long long)ps.rows[0] * d, two ? ps.src[1] : ps.src[0],
                       two ? (long long)ps.rows[1] * d : 0, partial, st);
    for (int i = 0; i < ps.n && rc == FS_OK; ++i)
      rc = launch_split_planes_f16(ps.src[i], reinterpret_cast<unsigned*>(base + ps.off[i]),
                                   ps.rows[i], (int)d, c.dp, partial + 256 * i, scales + i,
                                   two ? nullptr : scales + 1, c.gemm ? 1 : 0,
                                   i == 0 ? select_state(ps, ws) : nullptr,
                                   best_keys_of(ps, c, ws, ps.src[i], ps.rows[i]),
                                   keep ? tiled_of(ps, c, ws, ps.src[i], ps.rows[i]) : nullptr, st,
                                   start_plain ? 1 : 0);
  }
  return rc;
}

int side_plane_set(const Side* sides, int nsides, const LseConfig& c, PlaneSet& ps) {
  const float* ptrs[4];
  int rows[4];
  int cnt = 0;
  for (int s = 0; s < nsides; ++s) {
    ptrs[cnt] = sides[s].q; rows[cnt++] = sides[s].nq;
    ptrs[cnt] = sides[s].k; rows[cnt++] = sides[s].nk;
  }
  return make_plane_set(ptrs, rows, cnt, c, ps);
}

// ---- large-d LSE on chunked fp16 planes (lse_gemm_kernel) ----
constexpr int kGemmTile = 256;  // query rows per workgroup and keys per tile
constexpr int kGemmSweepSplits = 64;  // most key chunks of a one-sweep launch on a matrix with itself

struct GemmPlan {
  int igroups, bsplits, chunk;
};

GemmPlan gemm_plan(int64_t nq, int64_t nk, int total_igroups) {
  GemmPlan p;
  p.igroups = ceil_div(nq, kGemmTile);
  int s = 1;
  while ((int64_t)total_igroups * s < 512 && nk / (2 * s) >= kGemmTile && s < 32) s *= 2;
  p.chunk = ceil_div(ceil_div(nk, s), kGemmTile) * kGemmTile;
  p.bsplits = ceil_div(nk, p.chunk);
  return p;
}

// Workspace: plane region (see above), then per side 2*bsplits partial (M, s) rows.
int run_lse_gemm(int mode, Side* sides, int nsides, int64_t d, const LseConfig& cfg, bool prepared,
                 void* ws, size_t ws_bytes, hipStream_t st, uint32_t flags) {
  const bool vec = (mode == kVec);
  PlaneSet ps;
  int rc = side_plane_set(sides, nsides, cfg, ps);
  if (rc != FS_OK) return rc;
  size_t need = ps.end;
  int total_ig = 0;
  for (int s = 0; s < nsides; ++s) total_ig += ceil_div(sides[s].nq, kGemmTile);
  GemmPlan plans[2];
  for (int s = 0; s < nsides; ++s) plans[s] = gemm_plan(sides[s].nq, sides[s].nk, total_ig);
  // The one-sweep form of a two-sided step (lse_gemm_kernel<3>) on prepared planes, whose state
  // words hold the permission: the sides are the two orders of one pair of matrices ...
  const bool sweep_base = mode == kLse && prepared && !(flags & FS_FLAG_NO_SWEEP);
  bool sweep_pair = sweep_base && nsides == 2;
  if (sweep_pair) {
    const Side &s0 = sides[0], &s1 = sides[1];
    sweep_pair = s0.q == s1.k && s0.k == s1.q && s0.nq == s1.nk && s0.nk == s1.nq && s0.qscale == s1.qscale &&
                 sweep_col_bytes(s0.nq, s0.nk) > 0;
  }
  // ... or every side is a problem of a matrix with itself, of whose symmetric matrix of logits
  // the launch visits the 256 x 256 tiles on and above the diagonal only
  bool sweep_self = sweep_base && !sweep_pair;
  for (int s = 0; s < nsides && sweep_self; ++s)
    sweep_self = sides[s].q == sides[s].k && sides[s].nq == sides[s].nk &&
                 sweep_col_bytes(sides[s].nq, sides[s].nk) > 0;
  const bool sweep = sweep_pair || sweep_self;
  // Key chunks of the one-sweep launch.  Pair: one workgroup per CU where the keys allow, never
  // more chunks than side 0 has partial rows for.  Self: the number of items per chunk grows
  // along the keys, so the chunks are made as small as fills the CUs' rounds best (down to one
  // tile; at most kGemmSweepSplits chunks), all sides alike.
  int sw_bs[2] = {0, 0}, sw_chunk[2] = {0, 0}, sw_items[2] = {0, 0};
  if (sweep_pair) {
    int s = 1;
    while (plans[0].igroups * s < 256 && sides[0].nk / (2 * s) >= kGemmTile && 2 * s <= plans[0].bsplits) s *= 2;
    sw_chunk[0] = ceil_div(ceil_div(sides[0].nk, s), kGemmTile) * kGemmTile;
    sw_bs[0] = ceil_div(sides[0].nk, sw_chunk[0]);
  } else if (sweep_self) {
    double best = 0.0;
    for (int tiles = 1; tiles <= 64; tiles *= 2) {
      const int chunk = tiles * kGemmTile;
      long long items = 0;
      bool ok = true;
      for (int s = 0; s < nsides; ++s) {
        const int bs = ceil_div(sides[s].nk, chunk);
        ok = ok && bs <= kGemmSweepSplits;
        for (int c = 0; c < bs; ++c) items += self_groups_of_chunk(c, chunk, sides[s].nk, plans[s].igroups);
      }
      if (!ok) continue;
      const double cost = std::ceil((double)items / 256.0) * tiles;  // rounds of one workgroup per CU
      if (best == 0.0 || cost < best - 1e-9) {
        best = cost;
        for (int s = 0; s < nsides; ++s) {
          sw_chunk[s] = chunk;
          sw_bs[s] = ceil_div(sides[s].nk, chunk);
        }
      }
    }
    if (best == 0.0) return FS_ERR_UNSUPPORTED;  // (64 tiles x kGemmSweepSplits chunks cover every size accepted)
    for (int s = 0; s < nsides; ++s)
      for (int c = 0; c < sw_bs[s]; ++c)
        sw_items[s] += self_groups_of_chunk(c, sw_chunk[s], sides[s].nk, plans[s].igroups);
  }
  size_t part_off[2], part_o_off[2] = {0, 0};
  for (int s = 0; s < nsides; ++s) {
    const int prows = 2 * std::max(plans[s].bsplits, sweep_self ? sw_bs[s] : 0);  // partial rows per row
    part_off[s] = need;
    need += (((size_t)prows * (size_t)sides[s].nq * 2 * sizeof(float)) + 15) & ~(size_t)15;
    if (vec) {  // one weighted sum per partial row
      part_o_off[s] = need;
      need += (((size_t)2 * plans[s].bsplits * (size_t)sides[s].nq * sizeof(float)) + 15) & ~(size_t)15;
    }
  }
  need = (need + 63) & ~(size_t)63;
  const size_t col_off = need;
  if (sweep) need += sweep_col_bytes(sides[0].nq, sides[0].nk);
  const size_t col_off_b = need;
  if (sweep_self && nsides == 2) need += sweep_col_bytes(sides[1].nq, sides[1].nk);
  if (need > ws_bytes || ws == nullptr) return FS_ERR_WORKSPACE_TOO_SMALL;
  char* base = static_cast<char*>(ws);

  LaunchArgs a;
  std::memset(&a, 0, sizeof(a));
  a.d = (int)d;
  a.pstride = cfg.dp;
  int blocks[2] = {0, 0};
  for (int s = 0; s < nsides; ++s) {
    Side& sd = sides[s];
    sd.splits = 2 * plans[s].bsplits;
    sd.chunk = plans[s].chunk;
    sd.igroups = plans[s].igroups;
    sd.part_ms = reinterpret_cast<float*>(base + part_off[s]);
    sd.part_o = vec ? reinterpret_cast<float*>(base + part_o_off[s]) : nullptr;
    sd.plane_scale = plane_scales(ps, ws);
    sd.ps_q = plane_index(ps, sd.q, sd.nq);
    sd.ps_k = plane_index(ps, sd.k, sd.nk);
    sd.qplanes = plane_of(ps, ws, sd.q, sd.nq);
    sd.kplanes = plane_of(ps, ws, sd.k, sd.nk);
    blocks[s] = plans[s].igroups * plans[s].bsplits;
    a.side[s] = sd;
  }
  if (nsides == 1) a.side[1] = a.side[0];
  a.blocks0 = blocks[0];
  const int total = blocks[0] + blocks[1];
  a.blocks_all = total;
  if (total <= 0) return FS_OK;

  if (!prepared) rc = launch_plane_set(ps, cfg, d, ws, st);
  if (sweep) {
    // enqueued ahead of the two-sided launch, which only runs when this one did not, or failed
    a.sel = select_state(ps, ws);
    a.sweep = 1;
    a.col_part = reinterpret_cast<float*>(base + col_off);
    a.sw_part_mult = 2;
    a.sw_chunk = sw_chunk[0];
    a.sw_splits = 2 * sw_bs[0];
    if (sweep_self) {
      a.sweep_self = 1;
      a.sw_items0 = a.sw_items = sw_items[0];
      if (nsides == 2) {
        a.sw_chunk_b = sw_chunk[1];
        a.sw_splits_b = 2 * sw_bs[1];
        a.sw_items += sw_items[1];
        a.col_part_b = reinterpret_cast<float*>(base + col_off_b);
      }
    }
    if (rc == FS_OK) rc = launch_lse_gemm_sweep(a, st);
    if (rc == FS_OK) rc = launch_finish_sweep(a, st);
  }
  if (rc == FS_OK) rc = launch_lse_gemm(a, mode, total, st);
  if (rc != FS_OK) return rc;
  const int items0 = a.side[0].nq, items1 = (nsides == 2) ? a.side[1].nq : 0;
  if (mode == kArgmax) {  // one side; the partial values are already in output units
    a.out_scale = 1.0f;
    hipLaunchKernelGGL((finish_argmax_kernel<0>), dim3(ceil_div(items0, 256)), dim3(256), 0, st, a);
    return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
  }
  hipLaunchKernelGGL((finish_kernel<false>), dim3(ceil_div(items0 + items1, 256)), dim3(256), 0, st,
                     a, cfg.dp, items0, items1);
  return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
}

size_t gemm_ws_bytes(int64_t n, int64_t m, int64_t d, bool both, bool either, bool with_sweep = false) {
  LseConfig c;
  c.gemm = true; c.prec = 3; c.dp = chunked_stride(d); c.np = 2;
  size_t planes = plane_bytes(n, c) + plane_bytes(m, c) + kPlaneAuxBytes;
  auto part = [&](int64_t nq, int64_t nk, int total_ig) {
    const GemmPlan p = gemm_plan(nq, nk, total_ig);
    // (with_sweep: a matrix with itself may take up to kGemmSweepSplits chunks)
    const int bs = (with_sweep && nq == nk) ? std::max(p.bsplits, kGemmSweepSplits) : p.bsplits;
    return (size_t)2 * bs * (size_t)nq * 3 * sizeof(float) + 32;  // (M, s) and a weighted sum
  };
  const int ig_n = ceil_div(n, kGemmTile), ig_m = ceil_div(m, kGemmTile);
  // (the one-sweep form of a two-sided step: either matrix may hold the query rows)
  const size_t col = with_sweep ? std::max(sweep_col_bytes(n, m), sweep_col_bytes(m, n)) + 64 : 0;
  if (both) return planes + part(n, m, ig_n + ig_m) + part(m, n, ig_n + ig_m) + 64 + col;
  if (either) return planes + std::max(part(n, m, ig_n), part(m, n, ig_m)) + 64;
  return planes + part(n, m, ig_n) + 64;
}

// ---- large-d plan-matrix products on fp16 planes (plan_gemm_kernel) ----
constexpr int kPgTile = 256;       // keys per tile
constexpr int kPgRowsApi = 32;     // query rows per workgroup
constexpr size_t kPgAuxBytes = 2048;  // 256 partial maxima + the scale of a value matrix

struct PgPlan {
  int igroups, splits, chunk;
};

// Column blocks per wavefront, column groups and the row stride of partial outputs.
void pg_columns(int64_t d, int& cb, int& ncg, int& dpo) {
  const int ncb = ceil_div(d, 32);
  cb = (ncb <= 16) ? 2 : ((ncb <= 32) ? 4 : 6);
  ncg = ceil_div(ncb, 8 * cb);
  dpo = ncg * 8 * cb * 32;
}

// Planned per side, independent of what else shares the launch, so that the workspace a
// caller sized with fs_workspace_bytes always fits.
PgPlan pg_plan(int64_t nq, int64_t nk, int ncg) {
  PgPlan p;
  p.igroups = ceil_div(nq, kPgRowsApi);
  // One workgroup per CU at a time: take the smallest power-of-two key split whose grid fills
  // whole rounds of the 256 CUs to 85 % or better, else the best one.
  const double base = (double)p.igroups * ncg / 256.0;
  int s = 1, best = 1;
  double best_eff = 0.0;
  for (int c = 1; c <= 64 && (c == 1 || nk / c >= kPgTile); c *= 2) {
    const double rounds = base * c;
    const double eff = rounds / std::ceil(rounds);
    if (eff > best_eff + 1e-9) {
      best_eff = eff;
      best = c;
    }
    if (eff >= 0.85) {
      best = c;
      break;
    }
  }
  s = best;
  p.chunk = ceil_div(ceil_div(nk, s), kPgTile) * kPgTile;
  p.splits = ceil_div(nk, p.chunk);
  return p;
}

size_t pg_vt_bytes(int64_t nk, int64_t d) {
  return (size_t)ceil_div(nk, kPgTile) * kPgTile * (size_t)ceil_div(d, 32) * 32 * 4;
}

size_t pg_partial_bytes(const PgPlan& p, int64_t nq, int dpo) {
  if (p.splits <= 1) return 0;
  return (size_t)p.splits * (size_t)nq * (size_t)(2 + dpo) * sizeof(float) + 32;
}

// Workspace: plane region of x and y (as for lse_gemm_kernel), then per side the transposed
// value planes with their aux block, then per side the partial (M, s) and O rows.
int run_plan_gemm(int mode, Side* sides, int nsides, int64_t d, const LseConfig& cfg, bool prepared,
                  void* ws, size_t ws_bytes, hipStream_t st) {
  const bool mat5 = (mode == kMat5);
  PlaneSet ps;
  int rc = side_plane_set(sides, nsides, cfg, ps);
  if (rc != FS_OK) return rc;
  int cb, ncg, dpo;
  pg_columns(d, cb, ncg, dpo);
  size_t need = ps.end;
  PgPlan plans[2];
  size_t vt_off[2], part_off[2], q2_off = 0;
  for (int s = 0; s < nsides; ++s) {
    plans[s] = pg_plan(sides[s].nq, sides[s].nk, ncg);
    vt_off[s] = need;
    need += pg_vt_bytes(sides[s].nk, d) + kPgAuxBytes;
  }
  size_t bounds_off = 0;
  if (mat5) {  // chunked planes of the second stationary operand, their aux block, row bounds
    q2_off = need;
    need += plane_bytes(sides[0].nq, cfg) + kPlaneAuxBytes;
    bounds_off = need;
    need += (((size_t)sides[0].nq + 64) * sizeof(float) + 15) & ~(size_t)15;
  }
  for (int s = 0; s < nsides; ++s) {
    part_off[s] = need;
    need += (pg_partial_bytes(plans[s], sides[s].nq, dpo) + 15) & ~(size_t)15;
  }
  if (need > ws_bytes || ws == nullptr) return FS_ERR_WORKSPACE_TOO_SMALL;
  char* base = static_cast<char*>(ws);

  LaunchArgs a;
  std::memset(&a, 0, sizeof(a));
  a.d = (int)d;
  a.pstride = cfg.dp;
  a.nss = ncg;
  bool vec_ok = (d % 4 == 0);
  bool any_split = false;
  int blocks[2] = {0, 0};
  for (int s = 0; s < nsides; ++s) {
    Side& sd = sides[s];
    sd.splits = plans[s].splits;
    sd.chunk = plans[s].chunk;
    sd.igroups = plans[s].igroups;
    sd.part_ms = nullptr;
    sd.part_o = nullptr;
    if (sd.splits > 1) {
      any_split = true;
      sd.part_ms = reinterpret_cast<float*>(base + part_off[s]);
      sd.part_o = sd.part_ms + (((size_t)sd.splits * (size_t)sd.nq * 2 + 3) & ~(size_t)3);
    }
    sd.plane_scale = plane_scales(ps, ws);
    sd.ps_q = plane_index(ps, sd.q, sd.nq);
    sd.ps_k = plane_index(ps, sd.k, sd.nk);
    sd.qplanes = plane_of(ps, ws, sd.q, sd.nq);
    sd.kplanes = plane_of(ps, ws, sd.k, sd.nk);
    sd.vplanes = reinterpret_cast<const unsigned*>(base + vt_off[s]);
    sd.vplane_scale =
        reinterpret_cast<const float*>(base + vt_off[s] + pg_vt_bytes(sd.nk, d)) + 256;
    sd.kplane_scale = sd.plane_scale + plane_index(ps, sd.k, sd.nk);
    if (mat5) {
      sd.q2planes = reinterpret_cast<const unsigned*>(base + q2_off);
      sd.q2plane_scale =
          reinterpret_cast<const float*>(base + q2_off + plane_bytes(sd.nq, cfg)) + 2 * 256;
      vec_ok = vec_ok && aligned16(sd.q2);
      sd.kmax2 = reinterpret_cast<const float*>(base + bounds_off);
      sd.q2norm2 = sd.kmax2 + 64;
    }
    vec_ok = vec_ok && aligned16(sd.q) && aligned16(sd.ep.out);
    blocks[s] = plans[s].igroups * plans[s].splits * ncg;
    a.side[s] = sd;
  }
  if (nsides == 1) a.side[1] = a.side[0];
  a.blocks0 = blocks[0];
  a.vec_ok = vec_ok ? 1 : 0;
  const int total = blocks[0] + blocks[1];
  if (total <= 0) return FS_OK;

  if (!prepared) rc = launch_plane_set(ps, cfg, d, ws, st);
  for (int s = 0; s < nsides && rc == FS_OK; ++s) {
    const Side& sd = sides[s];
    float* aux = reinterpret_cast<float*>(base + vt_off[s] + pg_vt_bytes(sd.nk, d));
    rc = launch_transpose_planes(sd.v ? sd.v : sd.k, sd.vscale,
                                 reinterpret_cast<unsigned*>(base + vt_off[s]), sd.nk, (int)d,
                                 ceil_div(sd.nk, kPgTile) * 8, ceil_div(d, 32), aux, aux + 256, st);
  }
  if (mat5 && rc == FS_OK) {
    const Side& sd = sides[0];
    float* bounds = reinterpret_cast<float*>(base + bounds_off);
    rc = launch_mat5_bounds(sd.q2, sd.nq, (int)d, sd.kb1, sd.nk, bounds + 64, bounds, st);
    if (rc != FS_OK) return rc;
    float* partial = reinterpret_cast<float*>(base + q2_off + plane_bytes(sd.nq, cfg));
    rc = launch_absmax(sd.q2, (long long)sd.nq * d, sd.q2, 0, partial, st);
    if (rc == FS_OK)
      rc = launch_split_planes_f16(sd.q2, reinterpret_cast<unsigned*>(base + q2_off), sd.nq, (int)d,
                                   cfg.dp, partial, partial + 2 * 256, nullptr, 1, nullptr, nullptr, nullptr, st);
  }
  if (rc == FS_OK) rc = launch_plan_gemm(a, mat5, cb, total, st);
  if (rc != FS_OK) return rc;
  if (any_split) {
    int items[2] = {0, 0};
    for (int s = 0; s < nsides; ++s)
      items[s] = (a.side[s].splits > 1) ? a.side[s].nq * (dpo / 4) : 0;
    LaunchArgs f = a;
    if (items[0] == 0 && nsides == 2) {  // only the second side needs merging
      f.side[0] = a.side[1];
      items[0] = items[1];
      items[1] = 0;
    }
    hipLaunchKernelGGL((finish_kernel<true>), dim3(ceil_div(items[0] + items[1], 256)), dim3(256), 0,
                       st, f, dpo, items[0], items[1]);
    if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
  }
  return FS_OK;
}

size_t pg_ws_bytes(int64_t n, int64_t m, int64_t d, bool both, bool either, bool mat5) {
  LseConfig c;
  c.gemm = true; c.prec = 3; c.dp = chunked_stride(d); c.np = 2;
  size_t planes = plane_bytes(n, c) + plane_bytes(m, c) + kPlaneAuxBytes;
  if (mat5) planes += plane_bytes(n, c) + kPlaneAuxBytes + ((size_t)n + 64) * sizeof(float) + 16;
  int cb, ncg, dpo;
  pg_columns(d, cb, ncg, dpo);
  auto side = [&](int64_t nq, int64_t nk) {
    const PgPlan p = pg_plan(nq, nk, ncg);
    return pg_vt_bytes(nk, d) + kPgAuxBytes + pg_partial_bytes(p, nq, dpo) + 16;
  };
  if (both) return planes + side(n, m) + side(m, n) + 64;
  if (either) return planes + std::max(side(n, m), side(m, n)) + 64;
  return planes + side(n, m) + 64;
}

// ---- d <= 128 plan-matrix / plan-vector products and c-transform on fp16 planes (plan_tile_kernel) ----
size_t pt_vt_bytes(int64_t nk, int dpk) {  // V^T operands: 32-key blocks x 32-column blocks x 4 KiB
  return (size_t)ceil_div(nk, 64) * 2 * (size_t)((dpk + 31) / 32) * 4096;
}

// two row blocks per wavefront once the grid is large enough to fill the chip either way
int pt_rows_per_wave(int64_t nq) { return nq >= 16384 ? 2 : 1; }

// Workspace: plane region of x and y (the layout of lse2_kernel, so prepared planes serve),
// then per side the V^T operands with their aux block (kMat), then per side the partial rows.
int run_plan_tile(int mode, Side* sides, int nsides, int64_t d, const LseConfig& cfg,
                  const Family& fam, bool prepared, uint32_t flags, void* ws, size_t ws_bytes,
                  hipStream_t st) {
  PlaneSet ps;
  int rc = side_plane_set(sides, nsides, cfg, ps);
  if (rc != FS_OK) return rc;
  const int dpk = cfg.dp;  // 16, 32, 64 or 128
  int rb = 2;
  for (int s = 0; s < nsides; ++s) rb = std::min(rb, pt_rows_per_wave(sides[s].nq));
  const bool mat5 = (mode == kMat5);
  const bool has_o = (mode == kMat || mat5);
  // one row block where two would spill: 128-column rows and mat5
  if (dpk == 128 || mat5) rb = 1;
  size_t need = ps.end;
  SidePlan plans[2];
  size_t vt_off[2] = {0, 0}, part_off[2], q2_off = 0, bounds_off = 0;
  for (int s = 0; s < nsides; ++s) {
    plans[s] = plan_side(mode, sides[s].nq, sides[s].nk, fam, rb);
    if (has_o) {
      vt_off[s] = need;
      need += pt_vt_bytes(sides[s].nk, dpk) + kPgAuxBytes;
    }
  }
  if (mat5) {  // two-plane rows of the second stationary operand, their aux block, row bounds
    q2_off = need;
    need += plane_bytes(sides[0].nq, cfg) + kPlaneAuxBytes;
    bounds_off = need;
    need += (((size_t)sides[0].nq + 64) * sizeof(float) + 15) & ~(size_t)15;
  }
  for (int s = 0; s < nsides; ++s) {
    part_off[s] = need;
    need += side_ws_floats(mode, plans[s], sides[s].nq, dpk) * sizeof(float);
  }
  if (need > ws_bytes || (need > 0 && ws == nullptr)) return FS_ERR_WORKSPACE_TOO_SMALL;
  char* base = static_cast<char*>(ws);

  LaunchArgs a;
  std::memset(&a, 0, sizeof(a));
  a.d = (int)d;
  a.skip_log2 = (flags & FS_FLAG_NO_TILE_SKIP) ? -3.0e38f : -40.0f;
  bool vec_ok = (d % 4 == 0);
  bool any_split = false, any_seed = false;
  int blocks[2] = {0, 0};
  for (int s = 0; s < nsides; ++s) {
    Side& sd = sides[s];
    const SidePlan& p = plans[s];
    sd.splits = p.splits;
    sd.chunk = p.chunk;
    sd.igroups = p.igroups;
    sd.part_ms = nullptr;
    sd.part_o = nullptr;
    if (p.splits > 1) {
      any_split = true;
      sd.part_ms = reinterpret_cast<float*>(base + part_off[s]);
      sd.part_o = sd.part_ms + (((size_t)p.splits * (size_t)sd.nq * 2 + 3) & ~(size_t)3);
    }
    sd.plane_scale = plane_scales(ps, ws);
    sd.ps_q = plane_index(ps, sd.q, sd.nq);
    sd.ps_k = plane_index(ps, sd.k, sd.nk);
    sd.qplanes = plane_of(ps, ws, sd.q, sd.nq);
    sd.kplanes = plane_of(ps, ws, sd.k, sd.nk);
    if (has_o) {
      sd.vplanes = reinterpret_cast<const unsigned*>(base + vt_off[s]);
      sd.vplane_scale =
          reinterpret_cast<const float*>(base + vt_off[s] + pt_vt_bytes(sd.nk, dpk)) + 256;
      vec_ok = vec_ok && aligned16(sd.q) && aligned16(sd.ep.out);
    }
    if (mat5) {
      sd.kplane_scale = sd.plane_scale + plane_index(ps, sd.k, sd.nk);
      sd.q2planes = reinterpret_cast<const unsigned*>(base + q2_off);
      sd.q2plane_scale =
          reinterpret_cast<const float*>(base + q2_off + plane_bytes(sd.nq, cfg)) + 2 * 256;
      sd.kmax2 = reinterpret_cast<const float*>(base + bounds_off);
      sd.q2norm2 = sd.kmax2 + 64;
    }
    // a caller that knows, per query row, a key with a large logit (the carried keys of a solve):
    // the rows' running maxima start from their logits at those keys
    sd.seed = (sd.best_key != nullptr && mode != kArgmax)
                  ? row_array_of(ps, cfg, ws, sd.q, sd.nq, 3) : nullptr;
    any_seed = any_seed || sd.seed != nullptr;
    blocks[s] = p.igroups * p.splits;
    a.side[s] = sd;
  }
  if (nsides == 1) a.side[1] = a.side[0];
  a.blocks0 = blocks[0];
  a.vec_ok = vec_ok ? 1 : 0;
  const int total = blocks[0] + blocks[1];
  if (total <= 0) return FS_OK;

  if (!prepared) rc = launch_plane_set(ps, cfg, d, ws, st);
  if (any_seed && rc == FS_OK) rc = launch_row_seeds(a, dpk, nsides, st);
  if (mat5 && rc == FS_OK) {
    const Side& sd = sides[0];
    float* partial = reinterpret_cast<float*>(base + q2_off + plane_bytes(sd.nq, cfg));
    float* bounds = reinterpret_cast<float*>(base + bounds_off);
    rc = launch_mat5_bounds(sd.q2, sd.nq, (int)d, sd.kb1, sd.nk, bounds + 64, bounds, st);
    if (rc == FS_OK) rc = launch_absmax(sd.q2, (long long)sd.nq * d, sd.q2, 0, partial, st);
    if (rc == FS_OK)
      rc = launch_split_planes_f16(sd.q2, reinterpret_cast<unsigned*>(base + q2_off), sd.nq, (int)d,
                                   cfg.dp, partial, partial + 2 * 256, nullptr, 0, nullptr, nullptr, nullptr, st);
  }
  for (int s = 0; s < nsides && rc == FS_OK && has_o; ++s) {
    const Side& sd = sides[s];
    float* aux = reinterpret_cast<float*>(base + vt_off[s] + pt_vt_bytes(sd.nk, dpk));
    rc = launch_transpose_planes(sd.v ? sd.v : sd.k, sd.vscale,
                                 reinterpret_cast<unsigned*>(base + vt_off[s]), sd.nk, (int)d,
                                 ceil_div(sd.nk, 64) * 2, (dpk + 31) / 32, aux, aux + 256, st);
  }
  if (rc == FS_OK) rc = launch_plan_tile(a, mode, dpk, rb, total, st);
  if (rc != FS_OK) return rc;
  if (any_split && mode == kArgmax) {
    a.out_scale = 1.0f;
    hipLaunchKernelGGL((finish_argmax_kernel<0>), dim3(ceil_div(a.side[0].nq, 256)), dim3(256), 0, st,
                       a);
    return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
  }
  if (any_split) {
    const int per_row = has_o ? dpk / 4 : 1;
    int items[2] = {0, 0};
    for (int s = 0; s < nsides; ++s)
      items[s] = (a.side[s].splits > 1) ? a.side[s].nq * per_row : 0;
    LaunchArgs f = a;
    if (items[0] == 0 && nsides == 2) {  // only the second side needs merging
      f.side[0] = a.side[1];
      items[0] = items[1];
      items[1] = 0;
    }
    const int grid = ceil_div(items[0] + items[1], 256);
    if (has_o)
      hipLaunchKernelGGL((finish_kernel<true>), dim3(grid), dim3(256), 0, st, f, dpk, items[0], items[1]);
    else
      hipLaunchKernelGGL((finish_kernel<false>), dim3(grid), dim3(256), 0, st, f, dpk, items[0], items[1]);
    if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
  }
  return FS_OK;
}

size_t pt_ws_bytes(int mode, int64_t n, int64_t m, int64_t d, bool both, bool either,
                   const Family& fam) {
  const int dpk = std::max(padded_d(d), 16);
  LseConfig c;
  c.gemm = false; c.prec = 3; c.dp = dpk; c.np = 2;
  const size_t planes = plane_bytes(n, c) + plane_bytes(m, c) + 64 + kPlaneAuxBytes +
                        margin_region_bytes(std::max(n, m), c);  // the whole plane set
  auto side = [&](int64_t nq, int64_t nk) {
    size_t b = 0;
    for (int rb = 1; rb <= 2; ++rb)
      b = std::max(b, side_ws_floats(mode, plan_side(mode, nq, nk, fam, rb), nq, dpk) * sizeof(float));
    if (mode == kMat || mode == kMat5) b += pt_vt_bytes(nk, dpk) + kPgAuxBytes;
    if (mode == kMat5)  // planes of the second operand, aux, row bounds
      b += plane_bytes(nq, c) + kPlaneAuxBytes + ((size_t)nq + 64) * 4 + 64;
    return b + 16;
  };
  if (both) return planes + side(n, m) + side(m, n) + 64;
  if (either) return planes + std::max(side(n, m), side(m, n)) + 64;
  return planes + side(n, m) + 64;
}

// Plans, carves the workspace, launches the streaming kernel over one or two
// sides and, when keys were split, the merge kernel.
int run_stream(int mode, bool sepv, Side* sides, int nsides, int64_t d, void* ws, size_t ws_bytes,
               hipStream_t st, uint32_t flags = 0) {
  if (d > kMaxSlicedD) return FS_ERR_UNSUPPORTED;
  const Family fam = family_for(d);
  const int dp = fam.dp;
  const LseConfig cfg = lse_config(d, flags);
  const bool prepared = (flags & FS_FLAG_OPERANDS_PREPARED) != 0;
  if ((mode == kLse || mode == kVec || mode == kArgmax) && cfg.gemm)
    return run_lse_gemm(mode, sides, nsides, d, cfg, prepared, ws, ws_bytes, st, flags);
  if (mode == kArgmax && fam.sliced) return FS_ERR_UNSUPPORTED;  // d > 128 runs on fp16 planes only
  if ((mode == kMat || mode == kMat5) && cfg.gemm)
    return run_plan_gemm(mode, sides, nsides, d, cfg, prepared, ws, ws_bytes, st);
  // the plan-vector product at <= 64 columns rides on the pipelined log-sum-exp kernel
  const bool vec_lse2 = mode == kVec && cfg.prec == 3 && cfg.dp <= 64 && !fam.sliced;
  if (mode != kLse && !vec_lse2 && !fam.sliced && cfg.prec == 3)
    return run_plan_tile(mode, sides, nsides, d, cfg, fam, prepared, flags, ws, ws_bytes, st);
  LaunchArgs a;
  std::memset(&a, 0, sizeof(a));
  a.d = (int)d;
  bool vec_ok = (d % 4 == 0);
  int rb = 2;
  SidePlan plans[2];
  size_t need = 0;
  for (int s = 0; s < nsides; ++s) {
    plans[s] = plan_side(mode, sides[s].nq, sides[s].nk, fam);
    rb = std::min(rb, plans[s].rb);
  }
  bool aligned = (d % 4 == 0);
  for (int s = 0; s < nsides; ++s) aligned = aligned && aligned16(sides[s].q) && aligned16(sides[s].k);
  const int prec = cfg.prec;
  // pipelined LSE kernel: the 16-bit plane modes take any d <= 128, the fp32 mode needs aligned rows
  const bool lse2 = vec_lse2 || (mode == kLse && !fam.sliced && (prec != 0 || (aligned && dp >= 16)));
  const int dp2 = cfg.dp;
  // the kernel variant with the coarse tile test: asked for, or left to the device.  The device's
  // choice lives in state that belongs to prepared planes (a call that writes its own planes
  // would start it afresh), so without them FS_FLAG_COARSE_AUTO means the plain kernel.
  // (rows of 65 .. 128 columns: lse_coarse128_kernel, without carried margins)
  const bool can_coarse = lse2 && mode == kLse && prec == 3 && dp2 <= 128 && !(flags & FS_FLAG_NO_TILE_SKIP);
  const bool wide = dp2 == 128;
  const bool coarse = (flags & FS_FLAG_COARSE_TEST) && can_coarse;
  const bool auto_sel = (flags & FS_FLAG_COARSE_AUTO) && can_coarse && !coarse && prepared;
  Family fam_plan = fam;
  // carried margins: prepared planes only (they are state)
  bool margins = (coarse || auto_sel) && prepared && !wide;
  int min_splits[2] = {1, 1};
  if (coarse || auto_sel) {  // that kernel works on two row blocks per wavefront and 128-key tiles
    rb = 2;                  // (64-key tiles at 128 columns)
    fam_plan.jt = wide ? 64 : 128;
    for (int s = 0; s < nsides; ++s) {
      min_splits[s] = 2;  // the merge kernel carries the margins' state from launch to launch
      if (sides[s].nk < 2 * 128) margins = false;
    }
    for (int s = 0; s < nsides; ++s)
      plans[s] = plan_side(mode, sides[s].nq, sides[s].nk, fam_plan, rb, margins ? min_splits[s] : 1);
  }
  PlaneSet ps;
  ps.n = 0;
  ps.end = 0;
  if (lse2 && prec != 0) {
    const int prc = side_plane_set(sides, nsides, cfg, ps);
    if (prc != FS_OK) return prc;
    need = ps.end;
  }
  const size_t need_planes_end = need;
  for (int s = 0; s < nsides; ++s) {
    // both sides run in one launch and must share the rows-per-wave template
    if (!fam.sliced && plans[s].rb != rb)
      plans[s] = plan_side(mode, sides[s].nq, sides[s].nk, fam_plan, rb, margins ? min_splits[s] : 1);
    need += side_ws_floats(mode, plans[s], sides[s].nq, dp) * sizeof(float);
  }
  // The sparse form's wavefronts go through several chunks each (at most 2048 sub-tiles: its
  // list of sub-tiles to visit): eight key ranges, one per XCD and its L2, or more when the
  // launch would otherwise be fewer than about four wavefronts per slot of the chip.
  int sparse_group[2] = {1, 1};
  {
    int64_t waves = 0;
    for (int s = 0; s < nsides; ++s) {
      waves += (int64_t)plans[s].igroups * 4;
      if (plans[s].splits <= 1 || ps.margin_slot == 0 || plans[s].chunk > 65536) margins = false;
    }
    const int want = (int)std::max<int64_t>(8, ceil_div(4 * 2048, std::max<int64_t>(waves, 1)));
    for (int s = 0; s < nsides; ++s)
      sparse_group[s] = std::max(1, std::min(ceil_div(plans[s].splits, want), 65536 / std::max(plans[s].chunk, 1)));
  }
  // lse_coarse_kernel: per-tile records of the key bias, behind the partial rows
  const size_t aux_off = need;
  size_t aux_bytes[2] = {0, 0};
  if (coarse || auto_sel)
    for (int s = 0; s < nsides; ++s) {
      aux_bytes[s] = coarse_aux_bytes(sides[s].nk);
      need += aux_bytes[s];
    }
  // The one-sweep form of a two-sided step: the sides are the two orders of one pair of matrices
  // on prepared planes (the permission to run it is state, like the variant choice), two row
  // blocks per wavefront, keys split on both sides.
  // (rows of 65 .. 128 columns: lse_sweep128_kernel, whose workgroups take 256 query rows like
  // lse_sweep_kernel's whatever the two-sided kernel's plan says)
  const bool sweep_base = lse2 && mode == kLse && prec == 3 && dp2 <= 128 && prepared && !coarse &&
                          !(flags & FS_FLAG_NO_SWEEP) && ps.n > 0 && (rb == 2 || wide);
  auto groups256 = [&](int s) { return ceil_div(sides[s].nq, 256); };
  bool sweep_pair = sweep_base && nsides == 2;
  if (sweep_pair) {
    const Side &s0 = sides[0], &s1 = sides[1];
    sweep_pair = s0.q == s1.k && s0.k == s1.q && s0.nq == s1.nk && s0.nk == s1.nq && s0.qscale == s1.qscale &&
                 (wide || (plans[0].rb == 2 && plans[1].rb == 2)) && plans[0].splits > 1 && plans[1].splits > 1 &&
                 groups256(0) <= kSweepMaxGroups && sweep_col_bytes(s0.nq, s0.nk) > 0;
  }
  // ... or every side is a problem of a matrix with itself (the self problems of a debiased
  // loss): a symmetric matrix of logits, of which the one-sweep launch visits the tiles on and
  // above the diagonal of 256 x 256 blocks only
  bool sweep_self = sweep_base && !sweep_pair;
  for (int s = 0; s < nsides && sweep_self; ++s)
    sweep_self = sides[s].q == sides[s].k && sides[s].nq == sides[s].nk && (wide || plans[s].rb == 2) &&
                 plans[s].splits > 1 && groups256(s) <= kSweepMaxGroups &&
                 sweep_col_bytes(sides[s].nq, sides[s].nk) > 0;
  const bool sweep = sweep_pair || sweep_self;
  const size_t col_off = need;
  if (sweep) need += sweep_col_bytes(sides[0].nq, sides[0].nk);
  const size_t col_off_b = need;
  if (sweep_self && nsides == 2) need += sweep_col_bytes(sides[1].nq, sides[1].nk);
  if (need > ws_bytes || (need > 0 && ws == nullptr)) return FS_ERR_WORKSPACE_TOO_SMALL;
  float* wsp = reinterpret_cast<float*>(static_cast<char*>(ws) + need_planes_end);
  bool any_split = false;
  int blocks[2] = {0, 0};
  for (int s = 0; s < nsides; ++s) {
    Side& sd = sides[s];
    const SidePlan& p = plans[s];
    sd.splits = p.splits;
    sd.chunk = p.chunk;
    sd.igroups = p.igroups;
    sd.best_key = nullptr;
    sd.part_best = nullptr;
    sd.key_aux = nullptr;
    sd.margins = nullptr;
    sd.npieces = nullptr;
    sd.seed = nullptr;
    sd.sparse_group = 1;
    sd.ktiled = sd.qtiled = nullptr;
    sd.m_prev = nullptr;
    sd.bias_prev = nullptr;
    sd.part_ms = nullptr;
    sd.part_o = nullptr;
    if (p.splits > 1) {
      any_split = true;
      sd.part_ms = wsp;
      size_t off = (size_t)p.splits * (size_t)sd.nq * 2;
      if (mode != kLse) sd.part_o = wsp + ((off + 3) & ~(size_t)3);
      else sd.part_best = reinterpret_cast<int*>(wsp + off);
      wsp += side_ws_floats(mode, p, sd.nq, dp);
    }
    vec_ok = vec_ok && aligned16(sd.q) && aligned16(sd.k) && aligned16(sd.ep.out);
    if (sd.q2) vec_ok = vec_ok && aligned16(sd.q2);
    if (mode == kMat && sd.v) vec_ok = vec_ok && aligned16(sd.v);
    blocks[s] = p.igroups * p.splits * ((fam.sliced && (mode == kMat || mode == kMat5)) ? fam.nss : 1);
    if (ps.n > 0) {
      sd.qplanes = plane_of(ps, ws, sd.q, sd.nq);
      sd.kplanes = plane_of(ps, ws, sd.k, sd.nk);
      sd.plane_scale = plane_scales(ps, ws);
      sd.ps_q = plane_index(ps, sd.q, sd.nq);
      sd.ps_k = plane_index(ps, sd.k, sd.nk);
      if (coarse || auto_sel) {
        sd.best_key = best_keys_of(ps, cfg, ws, sd.q, sd.nq);
        sd.seed = row_array_of(ps, cfg, ws, sd.q, sd.nq, 3);
        sd.key_aux = reinterpret_cast<unsigned*>(static_cast<char*>(ws) + aux_off + (s == 1 ? aux_bytes[0] : 0));
      }
      if (margins) {
        // (slot and state words go with the matrix that holds the query rows)
        sd.margins = reinterpret_cast<float*>(static_cast<char*>(ws) + ps.margin_off + sd.ps_q * ps.margin_slot);
        sd.margin_stride = ps.margin_stride;
        sd.sparse_group = sparse_group[s];
        sd.ktiled = tiled_of(ps, cfg, ws, sd.k, sd.nk);
        sd.qtiled = tiled_of(ps, cfg, ws, sd.q, sd.nq);
        sd.npieces = reinterpret_cast<unsigned char*>(static_cast<char*>(ws) + ps.queue_off + kQueueBytes) +
                     (size_t)s * npieces_bytes(std::max(ps.rows[0], ps.n > 1 ? ps.rows[1] : 0));
        sd.m_prev = row_array_of(ps, cfg, ws, sd.q, sd.nq, 1);
        sd.bias_prev = row_array_of(ps, cfg, ws, sd.k, sd.nk, 2);
        // what the margins depend on: the pairing of matrices, the scale of the dot products
        // and the coefficients of the bias terms
        auto bits = [](float v) { unsigned u; std::memcpy(&u, &v, 4); return u; };
        unsigned t = 0x9e3779b9u * (unsigned)(1 + sd.ps_q + 2 * sd.ps_k);
        for (unsigned w : {bits(sd.qscale), bits(sd.kc0), bits(sd.kc1), bits(sd.kc2),
                           (unsigned)(sd.kb1 != nullptr) + 2u * (unsigned)(sd.kb2 != nullptr),
                           (unsigned)sd.nq, (unsigned)sd.nk, (unsigned)p.chunk})
          t = (t ^ w) * 0x85ebca6bu + 0xc2b2ae35u;
        a.tag[s] = t | 1u;  // never 0, the cleared state
      }
    }
    a.side[s] = sd;
  }
  if (nsides == 1) a.side[1] = a.side[0];
  a.blocks0 = blocks[0];
  // lse_sparse_kernel: wavefronts that stay and take (row group, key range) items from queues,
  // two workgroups per CU
  a.sparse_sides = nsides;
  a.blocks_sparse = kSparseBlocks;
  a.queue = margins ? reinterpret_cast<unsigned*>(static_cast<char*>(ws) + ps.queue_off) : nullptr;
  a.vec_ok = vec_ok ? 1 : 0;
  a.nss = fam.nss;
  const int total = blocks[0] + blocks[1];
  if (total <= 0) return FS_OK;

  int rc;
  if (fam.sliced) {
    rc = launch_sliced(mode, a, fam.nw, fam.nsl, total, st);
  } else if (lse2) {
    rc = prepared ? FS_OK : launch_plane_set(ps, cfg, d, ws, st);
    a.skip_log2 = (flags & FS_FLAG_NO_TILE_SKIP) ? -3.0e38f : -40.0f;
    if (sweep) {
      // enqueued ahead of the two-sided kernel, which only runs when this one did not, or failed
      a.sel = select_state(ps, ws);
      a.sweep = auto_sel ? 2 : 1;
      a.col_part = reinterpret_cast<float*>(static_cast<char*>(ws) + col_off);
      // Its own key split (it has half the workgroups of the two-sided launch, or fewer): of
      // the counts down to half of the side's, the one that fills the last round of workgroups
      // best (two workgroups per CU at a time)
      auto choose = [&](int sidx, int items_before, int& splits_out, int& chunk_out) {
        const int nk = a.side[sidx].nk, ig = groups256(sidx), smax = a.side[sidx].splits;
        double best = -1.0;
        int best_items = 0;
        for (int s = smax; s >= std::max(1, smax / 2); --s) {
          const int chunk = ceil_div(ceil_div(nk, s), 64) * 64;
          const int real = ceil_div(nk, chunk);
          if (real > smax) continue;
          int items = ig * real;
          if (sweep_self) {
            items = 0;
            for (int c = 0; c < real; ++c) items += self_groups_of_chunk(c, chunk, nk, ig);
          }
          const double rounds = (double)(items_before + items) / 512.0;
          const double eff = rounds / std::ceil(rounds);
          if (eff > best + 1e-9) {
            best = eff;
            splits_out = real;
            chunk_out = chunk;
            best_items = items;
          }
        }
        return best_items;
      };
      const int items0 = choose(0, 0, a.sw_splits, a.sw_chunk);
      if (sweep_self) {
        a.sweep_self = 1;
        a.sw_items0 = a.sw_items = items0;
        if (nsides == 2) {
          a.sw_items += choose(1, items0, a.sw_splits_b, a.sw_chunk_b);
          a.col_part_b = reinterpret_cast<float*>(static_cast<char*>(ws) + col_off_b);
        }
      }
      // (its row groups are of 256 rows; the two-sided kernel's may be of 128)
      LaunchArgs asw = a;
      for (int s = 0; s < nsides; ++s) asw.side[s].igroups = groups256(s);
      if (nsides == 1) asw.side[1] = asw.side[0];
      if (rc == FS_OK) rc = launch_lse_sweep(asw, dp2, st);
    }
    // device-chosen variant: both are enqueued, the one the state word names runs
    if (auto_sel) {
      a.sel = select_state(ps, ws);
      a.sel_pred = 1;
      a.sel_want = 1u;
      if (wide) {
        // the plain kernel at 128 columns works on one row block per wavefront: the same key
        // chunks and partial rows, twice the row groups
        LaunchArgs ap = a;
        int pb[2] = {0, 0};
        for (int s = 0; s < nsides; ++s) pb[s] = ceil_div(a.side[s].nq, 128) * a.side[s].splits;
        ap.blocks0 = pb[0];
        if (rc == FS_OK) rc = launch_lse2(ap, dp2, 1, prec, false, false, pb[0] + pb[1], st);
      } else if (rc == FS_OK) {
        rc = launch_lse2(a, dp2, rb, prec, false, false, total, st);
      }
      a.sel_want = 0u;
      if (rc == FS_OK) rc = launch_lse2(a, dp2, rb, prec, false, true, total, st);
    } else if (rc == FS_OK) {
      if (coarse && prepared) a.sel = select_state(ps, ws);  // the forced variant counts as well
      rc = launch_lse2(a, dp2, rb, prec, mode == kVec, coarse, total, st);
    }
  } else
  switch (mode) {
    case kLse: rc = launch_dp<kLse, false>(a, dp, rb, total, st); break;
    case kVec: rc = launch_dp<kVec, false>(a, dp, rb, total, st); break;
    case kMat:
      rc = sepv ? launch_dp<kMat, true>(a, dp, rb, total, st)
                : launch_dp<kMat, false>(a, dp, rb, total, st);
      break;
    case kMat5: rc = launch_dp<kMat5, false>(a, dp, rb, total, st); break;
    case kArgmax: rc = launch_dp<kArgmax, false>(a, dp, rb, total, st); break;
    default: rc = FS_ERR_BAD_ARGUMENT;
  }
  if (rc != FS_OK) return rc;

  if (any_split && mode == kArgmax) {
    a.out_scale = 1.0f;
    hipLaunchKernelGGL((finish_argmax_kernel<0>), dim3(ceil_div(a.side[0].nq, 256)), dim3(256), 0, st,
                       a);
    return hipGetLastError() == hipSuccess ? FS_OK : FS_ERR_LAUNCH_FAILED;
  }
  if (a.sel != nullptr && !any_split) {  // no merge launch to carry the decision
    hipLaunchKernelGGL((coarse_decide_kernel<0>), dim3(1), dim3(64), 0, st, a.sel);
    if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
  }
  if (any_split) {
    // sides that were not split already wrote their output; give them no items
    const bool has_o = (mode == kMat || mode == kMat5);
    const int per_row = has_o ? dp / 4 : 1;
    int items[2] = {0, 0};
    for (int s = 0; s < nsides; ++s)
      items[s] = (a.side[s].splits > 1) ? a.side[s].nq * per_row : 0;
    LaunchArgs f = a;
    if (items[0] == 0 && nsides == 2) {  // only the second side needs merging
      f.side[0] = a.side[1];
      items[0] = items[1];
      items[1] = 0;
    }
    const int tot = items[0] + items[1];
    const int grid = ceil_div(tot, 256);
    if (has_o)
      hipLaunchKernelGGL((finish_kernel<true>), dim3(grid), dim3(256), 0, st, f, dp, items[0], items[1]);
    else
      hipLaunchKernelGGL((finish_kernel<false>), dim3(grid), dim3(256), 0, st, f, dp, items[0], items[1]);
    if (hipGetLastError() != hipSuccess) return FS_ERR_LAUNCH_FAILED;
  }
  return FS_OK;
}

// Launch planning counts work items (rows x 4-column groups of the padded row) and workgroups
// in 32-bit ints: sizes whose counts would not fit are refused.
bool bad_sizes(int64_t n, int64_t m, int64_t d) {
  if (n <= 0 || m <= 0 || d <= 0 || n > (1 << 30) || m > (1 << 30) || d > (1 << 20)) return true;
  const int64_t dp = d <= 128 ? 128 : ((d + 1535) / 1536) * 1536;
  return std::max(n, m) * (dp / 4) > (int64_t)INT32_MAX;
}

Side lse_side(const float* q, const float* k, const float* kb0, float kc0, const float* kb1,
              float kc1, int64_t nq, int64_t nk, float qscale) {
  Side s;
  std::memset(&s, 0, sizeof(s));
  s.q = q; s.k = k;
  s.kb0 = kb0; s.kc0 = kc0;
  s.kb1 = kb1; s.kc1 = kc1;
  s.nq = (int)nq; s.nk = (int)nk;
  s.qscale = qscale;
  return s;
}

void lse_epilogue(Side& s, float* out, const float* old, float alpha, float eps, float damping,
                  const float* shift) {
  s.ep.kind = kEpiLse;
  s.ep.out = out;
  s.ep.old = (alpha != 1.0f) ? old : nullptr;
  s.ep.alpha = alpha;
  s.ep.out_scale = -eps * damping * kLn2;
  s.ep.shift = (shift && damping < 1.0f) ? shift : nullptr;
  s.ep.shift_coef = alpha * (1.0f - damping);
}

}  // namespace
}  // namespace fs

using namespace fs;

extern "C" {

int fs_version(void) { return 1; }

const char* fs_error_string(int code) {
  switch (code) {
    case FS_OK: return "ok";
    case FS_ERR_NULL_POINTER: return "null pointer argument";
    case FS_ERR_BAD_SIZE: return "size out of range";
    case FS_ERR_BAD_ARGUMENT: return "bad argument";
    case FS_ERR_WORKSPACE_TOO_SMALL: return "workspace too small";
    case FS_ERR_LAUNCH_FAILED: return "kernel launch failed";
    case FS_ERR_UNSUPPORTED: return "unsupported configuration";
    case FS_ERR_SCRATCH_TOO_SMALL: return "problem too large for the built-in scratch buffer";
  }
  return "unknown error";
}

}  // extern "C"

// with_sweep: room for the column sums of lse_sweep_kernel (prepared planes only)
static size_t workspace_bytes(int op, int64_t n, int64_t m, int64_t d, bool with_sweep) {
  if (bad_sizes(n, m, d) || d > kMaxSlicedD) return 0;
  const Family fam = family_for(d);
  const int dp = fam.dp;
  int mode;
  bool both = false, either = false;
  switch (op) {
    case FS_OP_LSE: mode = kLse; either = true; break;
    case FS_OP_SYMMETRIC_STEP: mode = kLse; both = true; break;
    case FS_OP_GRAD: mode = kMat; both = true; break;
    case FS_OP_APPLY_VEC: mode = kVec; either = true; break;
    case FS_OP_APPLY_MAT: mode = kMat; either = true; break;
    case FS_OP_MAT5: mode = kMat5; break;
    case FS_OP_C_TRANSFORM: mode = kArgmax; break;
    default: return 0;
  }
  // rb may be lowered when two sides share a launch: size for the rb=1 plan too
  auto side_bytes = [&](int64_t nq, int64_t nk) {
    size_t b = 0;  // the launch may settle on any rows-per-wave count: size for the largest
    for (int rb = 0; rb <= 3; ++rb)
      b = std::max(b, side_ws_floats(mode, plan_side(mode, nq, nk, fam, rb), nq, dp));
    if (mode == kLse && !fam.sliced && dp <= 128) {  // the plans of lse_coarse_kernel / lse_coarse128_kernel
      Family f2 = fam;
      f2.jt = dp <= 64 ? 128 : 64;
      b = std::max(b, side_ws_floats(mode, plan_side(mode, nq, nk, f2, 2), nq, dp));
      b = std::max(b, side_ws_floats(mode, plan_side(mode, nq, nk, f2, 2, 2), nq, dp));  // with carried margins
    }
    return b * sizeof(float);
  };
  size_t planes = 0;  // two fp16 planes of x and y for the pipelined LSE kernel
  if (mode == kLse && !fam.sliced) {
    LseConfig c;
    c.gemm = false; c.prec = 3; c.dp = std::max(dp, 16); c.np = 2;
    planes = plane_bytes(n, c) + plane_bytes(m, c) + 64 + kPlaneAuxBytes +
             margin_region_bytes(std::max(n, m), c);
  }
  if (mode == kLse && !fam.sliced) planes += coarse_aux_bytes(n) + coarse_aux_bytes(m);
  // (the one-sweep form of the symmetric step: either matrix may hold the query rows)
  if (op == FS_OP_SYMMETRIC_STEP && !fam.sliced && dp <= 128 && with_sweep)
    planes += std::max(sweep_col_bytes(n, m), sweep_col_bytes(m, n));
  const size_t a = side_bytes(n, m) + planes, b = side_bytes(m, n) + planes;
  size_t gemm = ((mode == kLse || mode == kVec || mode == kArgmax) && fam.sliced)
                    ? gemm_ws_bytes(n, m, d, both, either, with_sweep && op == FS_OP_SYMMETRIC_STEP) : 0;
  if ((mode == kMat || mode == kMat5) && fam.sliced)
    gemm = pg_ws_bytes(n, m, d, both, either, mode == kMat5);
  if ((mode == kMat || mode == kVec || mode == kArgmax || mode == kMat5) && !fam.sliced)
    gemm = pt_ws_bytes(mode, n, m, d, both, either, fam);
  if (both) return std::max(a + b - planes + 64, gemm);
  if (either) return std::max(std::max(a, b) + 64, gemm);
  return std::max(a + 64, gemm);
}

extern "C" {

size_t fs_workspace_bytes(int op, int64_t n, int64_t m, int64_t d) {
  return workspace_bytes(op, n, m, d, true);
}

int fs_prepare_operands(const float* x, const float* y, int64_t n, int64_t m, int64_t d,
                        uint32_t flags, void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !y) return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (d > kMaxSlicedD) return FS_ERR_UNSUPPORTED;
  const LseConfig cfg = lse_config(d, flags);
  const float* ptrs[2] = {x, y};
  const int rows[2] = {(int)n, (int)m};
  PlaneSet ps;
  const int rc = make_plane_set(ptrs, rows, 2, cfg, ps);
  if (rc != FS_OK || ps.n == 0) return rc;
  if (ps.end > workspace_bytes || workspace == nullptr) return FS_ERR_WORKSPACE_TOO_SMALL;
  return launch_plane_set(ps, cfg, d, workspace, (hipStream_t)stream, true,
                          (flags & FS_FLAG_START_PLAIN) != 0);
}

size_t fs_variant_state_offset(const float* x, const float* y, int64_t n, int64_t m, int64_t d,
                               uint32_t flags) {
  if (!x || !y || bad_sizes(n, m, d) || d > kMaxSlicedD) return 0;
  const LseConfig cfg = lse_config(d, flags);
  const float* ptrs[2] = {x, y};
  const int rows[2] = {(int)n, (int)m};
  PlaneSet ps;
  if (make_plane_set(ptrs, rows, 2, cfg, ps) != FS_OK || ps.n == 0) return 0;
  return ps.aux_off + (2 * 256 + 8) * sizeof(float);
}

size_t fs_best_keys_offset(const float* x, const float* y, int64_t n, int64_t m, int64_t d,
                           uint32_t flags, int which) {
  if (!x || !y || bad_sizes(n, m, d) || d > kMaxSlicedD || (which != 0 && which != 1)) return 0;
  const LseConfig cfg = lse_config(d, flags);
  if (cfg.gemm || cfg.dp > 128) return 0;
  const float* ptrs[2] = {x, y};
  const int rows[2] = {(int)n, (int)m};
  PlaneSet ps;
  if (make_plane_set(ptrs, rows, 2, cfg, ps) != FS_OK || ps.n == 0) return 0;
  const int i = plane_index(ps, ptrs[which], rows[which]);
  return ps.off[i] + planes_only_bytes(rows[which], cfg);
}

int fs_lse(const float* x, const float* y, const float* bias, float* out, int64_t n, int64_t m,
           int64_t d, float eps, float coord_scale, float damping, uint32_t flags,
           void* workspace, size_t workspace_bytes, void* stream) {
  (void)flags;
  if (!x || !y || !bias || !out) return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (!(eps > 0.f)) return FS_ERR_BAD_ARGUMENT;
  Side s = lse_side(x, y, bias, kLog2e, nullptr, 0.f, n, m, coord_scale / eps * kLog2e);
  lse_epilogue(s, out, nullptr, 1.0f, eps, damping, nullptr);
  return run_stream(kLse, false, &s, 1, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
}

int fs_lse_fused(const float* x, const float* y, const float* pot_hat, const float* log_w,
                 float* out, int64_t n, int64_t m, int64_t d, float eps, float coord_scale,
                 float damping, uint32_t flags, void* workspace, size_t workspace_bytes,
                 void* stream) {
  (void)flags;
  if (!x || !y || !pot_hat || !log_w || !out) return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (!(eps > 0.f)) return FS_ERR_BAD_ARGUMENT;
  Side s = lse_side(x, y, pot_hat, kLog2e / eps, log_w, kLog2e, n, m,
                    coord_scale / eps * kLog2e);
  lse_epilogue(s, out, nullptr, 1.0f, eps, damping, nullptr);
  return run_stream(kLse, false, &s, 1, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
}

int fs_symmetric_step(const float* x, const float* y, const float* f_hat, const float* g_hat,
                      const float* log_a, const float* log_b, float* f_out, float* g_out,
                      const float* shift_x, const float* shift_y, int64_t n, int64_t m,
                      int64_t d, float eps, float alpha, float damp_f, float damp_g,
                      float coord_scale, uint32_t flags, void* workspace,
                      size_t workspace_bytes, void* stream) {
  (void)flags;
  if (!x || !y || !f_hat || !g_hat || !log_a || !log_b || !f_out || !g_out)
    return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (!(eps > 0.f)) return FS_ERR_BAD_ARGUMENT;
  if (f_out == f_hat || g_out == g_hat) return FS_ERR_BAD_ARGUMENT;
  // Self problem OT(x, x): when every paired argument aliases, the two half-updates are the
  // same computation and it is done once (f_out == g_out receives it).
  const bool self = (x == y && f_hat == g_hat && log_a == log_b && f_out == g_out &&
                     shift_x == shift_y && n == m && damp_f == damp_g);
  if (f_out == g_out && !self) return FS_ERR_BAD_ARGUMENT;
  const float qs = coord_scale / eps * kLog2e;
  Side s[2];
  s[0] = lse_side(x, y, g_hat, kLog2e / eps, log_b, kLog2e, n, m, qs);
  lse_epilogue(s[0], f_out, f_hat, alpha, eps, damp_f, shift_x);
  if (self)
    return run_stream(kLse, false, s, 1, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
  s[1] = lse_side(y, x, f_hat, kLog2e / eps, log_a, kLog2e, m, n, qs);
  lse_epilogue(s[1], g_out, g_hat, alpha, eps, damp_g, shift_y);
  return run_stream(kLse, false, s, 2, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
}

int fs_symmetric_step_noalloc(const float* x, const float* y, const float* f_hat,
                              const float* g_hat, const float* log_a, const float* log_b,
                              float* f_out, float* g_out, const float* shift_x,
                              const float* shift_y, int64_t n, int64_t m, int64_t d, float eps,
                              float alpha, float damp_f, float damp_g, float coord_scale,
                              uint32_t flags, void* stream) {
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (d > kMaxSlicedD) return FS_ERR_UNSUPPORTED;
  const size_t need = workspace_bytes(FS_OP_SYMMETRIC_STEP, n, m, d, false);
  if (need == 0 || need > kScratchBytes) return FS_ERR_SCRATCH_TOO_SMALL;
  void* buf = nullptr;
  const int rc = scratch_on_current_device(&buf);
  if (rc != FS_OK) return rc;
  // the call writes its own operand planes (which also resets the variant-choice state) and
  // every partial row before reading it: nothing in the buffer has to be cleared beforehand
  flags &= ~(uint32_t)(FS_FLAG_OPERANDS_PREPARED | FS_FLAG_COARSE_AUTO);
  return fs_symmetric_step(x, y, f_hat, g_hat, log_a, log_b, f_out, g_out, shift_x, shift_y, n, m,
                           d, eps, alpha, damp_f, damp_g, coord_scale, flags, buf, kScratchBytes,
                           stream);
}

int fs_symmetric_steps(const float* x, const float* y, const float* f_hat, const float* g_hat,
                       const float* log_a, const float* log_b, float* f_a, float* g_a, float* f_b,
                       float* g_b, const float* shift_x, const float* shift_y, int64_t n,
                       int64_t m, int64_t d, const float* eps, const float* alpha,
                       const float* damp_f, const float* damp_g, int n_steps, float coord_scale,
                       uint32_t flags, void* workspace, size_t workspace_bytes, void* stream) {
  if (!f_a || !g_a || !f_b || !g_b || !eps || !alpha || !damp_f || !damp_g)
    return FS_ERR_NULL_POINTER;
  if (n_steps < 0) return FS_ERR_BAD_ARGUMENT;
  if (f_a == f_b || g_a == g_b || f_a == g_b || f_b == g_a) return FS_ERR_BAD_ARGUMENT;
  const float* f_in = f_hat;
  const float* g_in = g_hat;
  for (int s = 0; s < n_steps; ++s) {
    float* f_out = (s & 1) ? f_b : f_a;
    float* g_out = (s & 1) ? g_b : g_a;
    const int rc = fs_symmetric_step(x, y, f_in, g_in, log_a, log_b, f_out, g_out,
                                     damp_f[s] < 1.0f ? shift_x : nullptr,
                                     damp_g[s] < 1.0f ? shift_y : nullptr, n, m, d, eps[s],
                                     alpha[s], damp_f[s], damp_g[s], coord_scale, flags, workspace,
                                     workspace_bytes, stream);
    if (rc != FS_OK) return rc;
    f_in = f_out;
    g_in = g_out;
  }
  return FS_OK;
}

int fs_self_pair_steps(const float* x, const float* y, const float* fx_hat, const float* fy_hat,
                       const float* log_a, const float* log_b, float* fx_a, float* fy_a,
                       float* fx_b, float* fy_b, const float* shift_x, const float* shift_y,
                       int64_t n, int64_t m, int64_t d, const float* eps_x, const float* eps_y,
                       const float* alpha, const float* damp_x, const float* damp_y, int n_steps,
                       float coord_scale, uint32_t flags, void* workspace, size_t workspace_bytes,
                       void* stream) {
  if (!x || !y || !fx_hat || !fy_hat || !log_a || !log_b || !fx_a || !fy_a || !fx_b || !fy_b ||
      !eps_x || !eps_y || !alpha || !damp_x || !damp_y)
    return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (n_steps < 0) return FS_ERR_BAD_ARGUMENT;
  if (fx_a == fx_b || fy_a == fy_b || fx_a == fx_hat || fx_b == fx_hat || fy_a == fy_hat ||
      fy_b == fy_hat || fx_a == fy_a || fx_a == fy_b || fx_b == fy_a || fx_b == fy_b)
    return FS_ERR_BAD_ARGUMENT;
  const float* fx_in = fx_hat;
  const float* fy_in = fy_hat;
  for (int s = 0; s < n_steps; ++s) {
    if (!(eps_x[s] > 0.f) || !(eps_y[s] > 0.f)) return FS_ERR_BAD_ARGUMENT;
    float* fx_out = (s & 1) ? fx_b : fx_a;
    float* fy_out = (s & 1) ? fy_b : fy_a;
    Side sd[2];
    sd[0] = lse_side(x, x, fx_in, kLog2e / eps_x[s], log_a, kLog2e, n, n,
                     coord_scale / eps_x[s] * kLog2e);
    lse_epilogue(sd[0], fx_out, fx_in, alpha[s], eps_x[s], damp_x[s], shift_x);
    sd[1] = lse_side(y, y, fy_in, kLog2e / eps_y[s], log_b, kLog2e, m, m,
                     coord_scale / eps_y[s] * kLog2e);
    lse_epilogue(sd[1], fy_out, fy_in, alpha[s], eps_y[s], damp_y[s], shift_y);
    const int rc = run_stream(kLse, false, sd, 2, d, workspace, workspace_bytes,
                              (hipStream_t)stream, flags);
    if (rc != FS_OK) return rc;
    fx_in = fx_out;
    fy_in = fy_out;
  }
  return FS_OK;
}

int fs_grad(const float* x, const float* y, const float* f, const float* g, const float* log_a,
            const float* log_b, const float* a, const float* b, const float* x2, const float* y2,
            const float* grad_scale, float* grad_x, float* grad_y, int64_t n, int64_t m,
            int64_t d, float eps, float cost_scale, uint32_t flags, void* workspace,
            size_t workspace_bytes, void* stream) {
  return fs_grad_seeded(x, y, f, g, log_a, log_b, a, b, x2, y2, grad_scale, grad_x, grad_y, n, m, d,
                        eps, cost_scale, nullptr, nullptr, flags, workspace, workspace_bytes, stream);
}

int fs_grad_seeded(const float* x, const float* y, const float* f, const float* g,
                   const float* log_a, const float* log_b, const float* a, const float* b,
                   const float* x2, const float* y2, const float* grad_scale, float* grad_x,
                   float* grad_y, int64_t n, int64_t m, int64_t d, float eps, float cost_scale,
                   const int* keys_x, const int* keys_y, uint32_t flags, void* workspace,
                   size_t workspace_bytes, void* stream) {
  (void)flags;
  if (!x || !y || !f || !g || !log_a || !log_b || !a || !b || !x2 || !y2)
    return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (!(eps > 0.f)) return FS_ERR_BAD_ARGUMENT;
  const float qs = 2.0f * cost_scale / eps * kLog2e;
  Side s[2];
  int ns = 0;
  if (grad_x) {
    Side& sd = s[ns++];
    sd = lse_side(x, y, g, kLog2e / eps, y2, -cost_scale * kLog2e / eps, n, m, qs);
    sd.kb2 = log_b; sd.kc2 = kLog2e;
    sd.ep.kind = kEpiGrad; sd.ep.out = grad_x; sd.ep.w = a; sd.ep.grad_scale = grad_scale;
    sd.ep.gcoef = 2.0f * cost_scale;
    sd.best_key = const_cast<int*>(keys_x);  // read only
  }
  if (grad_y) {
    Side& sd = s[ns++];
    sd = lse_side(y, x, f, kLog2e / eps, x2, -cost_scale * kLog2e / eps, m, n, qs);
    sd.kb2 = log_a; sd.kc2 = kLog2e;
    sd.ep.kind = kEpiGrad; sd.ep.out = grad_y; sd.ep.w = b; sd.ep.grad_scale = grad_scale;
    sd.ep.gcoef = 2.0f * cost_scale;
    sd.best_key = const_cast<int*>(keys_y);
  }
  if (ns == 0) return FS_OK;
  return run_stream(kMat, false, s, ns, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
}

int fs_apply_vec(const float* x, const float* y, const float* f_hat, const float* g_hat,
                 const float* log_a, const float* log_b, const float* vec, float* out,
                 int64_t n, int64_t m, int64_t d, float eps, float coord_scale, int axis,
                 uint32_t flags, void* workspace, size_t workspace_bytes, void* stream) {
  (void)flags;
  if (!x || !y || !f_hat || !g_hat || !log_a || !log_b || !vec || !out)
    return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (!(eps > 0.f) || (axis != 0 && axis != 1)) return FS_ERR_BAD_ARGUMENT;
  const float qs = coord_scale / eps * kLog2e;
  Side s = (axis == 1) ? lse_side(x, y, g_hat, kLog2e / eps, log_b, kLog2e, n, m, qs)
                       : lse_side(y, x, f_hat, kLog2e / eps, log_a, kLog2e, m, n, qs);
  s.v = vec;
  s.ep.kind = kEpiApply; s.ep.out = out; s.ep.post = 1.0f;
  s.ep.r0 = (axis == 1) ? f_hat : g_hat; s.ep.rc0 = kLog2e / eps;
  s.ep.r1 = (axis == 1) ? log_a : log_b; s.ep.rc1 = kLog2e;
  return run_stream(kVec, false, &s, 1, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
}

int fs_schur_matvec(const float* x, const float* y, const float* f_hat, const float* g_hat,
                    const float* log_a, const float* log_b, const float* z, const float* inv_diag_x,
                    const float* denom, float* piz, float* out, int64_t n, int64_t m, int64_t d,
                    float eps, float coord_scale, uint32_t flags, void* workspace,
                    size_t workspace_bytes, void* stream) {
  if (!x || !y || !f_hat || !g_hat || !log_a || !log_b || !z || !inv_diag_x || !denom || !piz ||
      !out)
    return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (!(eps > 0.f) || out == z || piz == inv_diag_x) return FS_ERR_BAD_ARGUMENT;
  const float qs = coord_scale / eps * kLog2e;
  // piz = (P z) / diag_x
  Side s1 = lse_side(x, y, g_hat, kLog2e / eps, log_b, kLog2e, n, m, qs);
  s1.v = z;
  s1.ep.kind = kEpiApply; s1.ep.out = piz; s1.ep.post = 1.0f;
  s1.ep.r0 = f_hat; s1.ep.rc0 = kLog2e / eps;
  s1.ep.r1 = log_a; s1.ep.rc1 = kLog2e;
  s1.ep.mul = inv_diag_x;
  int rc = run_stream(kVec, false, &s1, 1, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
  if (rc != FS_OK) return rc;
  // out = denom * z - P^T piz
  Side s2 = lse_side(y, x, f_hat, kLog2e / eps, log_a, kLog2e, m, n, qs);
  s2.v = piz;
  s2.ep.kind = kEpiApply; s2.ep.out = out; s2.ep.post = 1.0f;
  s2.ep.r0 = g_hat; s2.ep.rc0 = kLog2e / eps;
  s2.ep.r1 = log_b; s2.ep.rc1 = kLog2e;
  s2.ep.add_a = denom; s2.ep.add_b = z; s2.ep.res_coef = -1.0f;
  return run_stream(kVec, false, &s2, 1, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
}

int fs_apply_mat(const float* x, const float* y, const float* f_hat, const float* g_hat,
                 const float* log_a, const float* log_b, const float* mat, const float* scale,
                 float* out, int64_t n, int64_t m, int64_t d, int64_t dv, float eps,
                 float coord_scale, int axis, uint32_t flags, void* workspace,
                 size_t workspace_bytes, void* stream) {
  (void)flags;
  if (!x || !y || !f_hat || !g_hat || !log_a || !log_b || !mat || !out)
    return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (!(eps > 0.f) || (axis != 0 && axis != 1)) return FS_ERR_BAD_ARGUMENT;
  if (axis == 0 && scale) return FS_ERR_BAD_ARGUMENT;
  if (dv != d) return FS_ERR_UNSUPPORTED;
  const float qs = coord_scale / eps * kLog2e;
  Side s = (axis == 1) ? lse_side(x, y, g_hat, kLog2e / eps, log_b, kLog2e, n, m, qs)
                       : lse_side(y, x, f_hat, kLog2e / eps, log_a, kLog2e, m, n, qs);
  const bool sepv = !(mat == s.k && scale == nullptr);
  s.v = sepv ? mat : nullptr;
  s.vscale = scale;
  s.ep.kind = kEpiApply; s.ep.out = out; s.ep.post = 1.0f;
  s.ep.r0 = (axis == 1) ? f_hat : g_hat; s.ep.rc0 = kLog2e / eps;
  s.ep.r1 = (axis == 1) ? log_a : log_b; s.ep.rc1 = kLog2e;
  return run_stream(kMat, sepv, &s, 1, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
}

int fs_c_transform(const float* x, const float* y, const float* bias, float* min_out,
                   int64_t* argmin_out, int64_t n, int64_t m, int64_t d, float coord_scale,
                   uint32_t flags, void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !y || !bias || !min_out || !argmin_out) return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  // min_j [-cs2 x.y + bias_j] = -max_j [cs2 x.y - bias_j]
  Side s = lse_side(x, y, bias, -1.0f, nullptr, 0.f, n, m, coord_scale);
  s.ep.kind = kEpiArgmax;
  s.ep.out = min_out;
  s.ep.idx_out = reinterpret_cast<long long*>(argmin_out);
  // d > 128 runs on the fp16 planes whatever operand mode is asked for
  if (d > kMaxStreamD) flags &= ~(uint32_t)FS_FLAG_FP32_MFMA;
  return run_stream(kArgmax, false, &s, 1, d, workspace, workspace_bytes, (hipStream_t)stream,
                    flags & ~(uint32_t)FS_FLAG_OPERANDS_PREPARED);
}

int fs_mat5(const float* x, const float* y, const float* f_ott, const float* g_ott,
            const float* A, const float* x2, const float* y2, float* out, int64_t n, int64_t m,
            int64_t d, float eps, float cost_scale, uint32_t flags, void* workspace,
            size_t workspace_bytes, void* stream) {
  (void)flags;
  if (!x || !y || !f_ott || !g_ott || !A || !x2 || !y2 || !out) return FS_ERR_NULL_POINTER;
  if (bad_sizes(n, m, d)) return FS_ERR_BAD_SIZE;
  if (!(eps > 0.f)) return FS_ERR_BAD_ARGUMENT;
  const float qs = 2.0f * cost_scale / eps * kLog2e;
  Side s = lse_side(x, y, g_ott, kLog2e / eps, y2, -cost_scale * kLog2e / eps, n, m, qs);
  s.q2 = A;
  s.ep.kind = kEpiApply; s.ep.out = out; s.ep.post = -4.0f * cost_scale / eps;
  s.ep.r0 = f_ott; s.ep.rc0 = kLog2e / eps;
  s.ep.r1 = x2; s.ep.rc1 = -cost_scale * kLog2e / eps;
  return run_stream(kMat5, false, &s, 1, d, workspace, workspace_bytes, (hipStream_t)stream, flags);
}

}  // extern "C"
