// CSR SpMM  C[rows,f] = beta*C + A*B  for gfx950, and the cached handle around it.
//
// Replaces cusparseSpMM(CSRMM_ALG1, alpha = 1, beta = 1) and everything the reference wraps
// around it on every call (sparse-extension/sparse_coo_tensor.cu:136-231): B and C stay row-major,
// nothing is transposed, and the CSR, its transpose and the schedules live in a handle.
//
// Work decomposition
//   task    = a row segment: at most `seg` consecutive stored entries of one row.  One wavefront
//             runs one task.  Rows of degree <= seg are one task and are written straight to C.
//   team    = LPR lanes that together cover the f output columns (VEC floats per lane and chunk).
//             A wavefront holds G = 64/LPR teams; team g takes entries g, g+G, ... of the task and
//             the teams' partial rows are combined with a fixed xor butterfly (no atomics).
//   split rows (degree > seg) write one partial row per task to a workspace; a second kernel adds
//             a row's partials in segment order.  Summation order is a function of the matrix,
//             f and seg only, so results are bit-identical from run to run.
// (col, val) of 64 entries are fetched with one coalesced load per array and handed to the teams
// with lane reads (readlane for G == 1, where the column index becomes a scalar base address).
#include "common.h"
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <new>

namespace cg {

constexpr int kSpmmThreads = 256;
constexpr int kWavesPerBlock = kSpmmThreads / kWave;

struct SpmmArgs {
  const int32_t *rowptr;
  const int32_t *colind;
  const float *val;
  const int32_t *task_row;  // TABLE only
  const int32_t *tbase;     // TABLE only: first task of each row
  const int32_t *pbase;     // TABLE only: first partial slot of each split row
  int64_t ntasks;
  int32_t seg;
  int32_t m;                // number of columns of A (rows of B), for CLAMP
  const float *B;
  int64_t ldb;
  float *C;
  int64_t ldc;
  float *P;                 // partial rows of split rows, row stride f
  int32_t f;
  float beta;
  int32_t tiles;            // feature tiles (1, 2, 4 or 8); tile t is run by XCDs x with x % tiles == t
  int32_t tile_slots;       // VEC-wide slots per tile (the last tile may hold fewer)
  int32_t groups;           // kModeHub: hot column groups (1, 2, 4 or 8); group g runs on XCDs x % groups == g
  int64_t tstart[9];        // kModeHub: tasks of group g are [tstart[g], tstart[g+1])
};

// kModeRows: one task per row, no tables, column indices clamped (one-shot entry point)
// kModeTable: tasks from the schedule tables of a handle
// kModeHub:  tasks of the hot column groups of a hub plan, pinned to XCDs; every task writes a partial row
enum { kModeRows = 0, kModeTable = 1, kModeHub = 2 };

template <int VEC>
struct VecT;
template <>
struct VecT<1> {
  typedef float type;
};
template <>
struct VecT<2> {
  typedef float2 type;
};
template <>
struct VecT<4> {
  typedef float4 type;
};

template <int VEC>
__device__ __forceinline__ void load_vec(const float *p, float (&r)[VEC]) {
  typedef typename VecT<VEC>::type V;
  const V t = *reinterpret_cast<const V *>(p);
  const float *tp = reinterpret_cast<const float *>(&t);
#pragma unroll
  for (int i = 0; i < VEC; ++i) r[i] = tp[i];
}

template <int VEC>
__device__ __forceinline__ void store_vec(float *p, const float (&r)[VEC]) {
  typedef typename VecT<VEC>::type V;
  V t;
  float *tp = reinterpret_cast<float *>(&t);
#pragma unroll
  for (int i = 0; i < VEC; ++i) tp[i] = r[i];
  *reinterpret_cast<V *>(p) = t;
}

template <int VEC, int LPR, int CHUNKS, int MODE>
__global__ __launch_bounds__(kSpmmThreads) void spmm_rowseg_kernel(const SpmmArgs a) {
  static_assert(LPR == 64 || CHUNKS == 1, "several chunks only with a full-wave team");
  constexpr int G = kWave / LPR;
  constexpr bool TABLE = MODE != kModeRows;
  constexpr bool CLAMP = MODE == kModeRows;
  constexpr bool HUB = MODE == kModeHub;
  const int lane = threadIdx.x & (kWave - 1);
  // Workgroups are dealt to the 8 XCDs round robin (workgroup w runs on XCD w % 8), and every XCD
  // has its own L2.  With T feature tiles, XCD x only ever touches tile x % T of B, so its L2 holds
  // a T times narrower slice of B's hot rows: the 8 L2s cache different data instead of 8 copies.
  int tile = 0;
  int64_t tb = blockIdx.x;
  int64_t task_lo = 0, task_hi = a.ntasks;
  if (HUB) {
    // Hot columns are dealt to `groups` groups; group g's rows of B are only ever read by the XCDs
    // x with x % groups == g, so each L2 keeps its own share of the hot rows resident.
    const int x = blockIdx.x & 7;
    const int per = 8 / a.groups;
    const int grp = x % a.groups;
    tb = (int64_t)(blockIdx.x >> 3) * per + x / a.groups;
    task_lo = a.tstart[grp];
    task_hi = a.tstart[grp + 1];
  } else if (a.tiles > 1) {
    const int x = blockIdx.x & 7;
    const int per = 8 / a.tiles;  // XCDs that share a tile
    tile = x % a.tiles;
    tb = (int64_t)(blockIdx.x >> 3) * per + x / a.tiles;
  }
  const int64_t task =
      __builtin_amdgcn_readfirstlane((int)(task_lo + tb * kWavesPerBlock + threadIdx.x / kWave));
  if (task >= task_hi) return;

  int32_t row, sidx, rs, re;
  if (TABLE) {
    row = a.task_row[task];
    sidx = (int32_t)task - a.tbase[row];
  } else {
    row = (int32_t)task;
    sidx = 0;
  }
  rs = a.rowptr[row];
  re = a.rowptr[row + 1];
  const int32_t start = TABLE ? rs + sidx * a.seg : rs;
  const int32_t end = TABLE ? (start + a.seg < re ? start + a.seg : re) : re;
  const bool single = HUB ? false : (TABLE ? (re - rs <= a.seg) : true);
  if (single && start >= end && a.beta == 1.0f) return;  // empty row, C unchanged

  const int g = lane / LPR;   // team
  const int j = lane % LPR;   // position inside the team
  const int slot0 = tile * a.tile_slots;
  int nslots = a.f / VEC - slot0;  // slots of this tile
  nslots = nslots < a.tile_slots ? nslots : a.tile_slots;
  if (nslots <= 0) return;
  bool active[CHUNKS];
  int64_t boff[CHUNKS];  // lane's column offset per chunk; idle lanes re-read the chunk's first slot
#pragma unroll
  for (int ch = 0; ch < CHUNKS; ++ch) {
    active[ch] = (ch * LPR + j) < nslots;
    boff[ch] = (int64_t)(slot0 + ch * LPR + (active[ch] ? j : 0)) * VEC;
  }

  float acc[CHUNKS][VEC];
#pragma unroll
  for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[ch][v] = 0.f;

  constexpr int U = 4;  // entries per team in flight

  // software pipeline: the next 64 (col, val) are in flight while the current 64 are consumed
  int32_t c_next = 0;
  float v_next = 0.f;
  if (start + lane < end) {
    c_next = a.colind[start + lane];
    v_next = a.val[start + lane];
  }
  for (int32_t base = start; base < end; base += kWave) {
    int32_t c = c_next;
    const float v = v_next;
    const int32_t nb = base + kWave + lane;
    c_next = 0;
    v_next = 0.f;
    if (nb < end) {
      c_next = a.colind[nb];
      v_next = a.val[nb];
    }
    if (CLAMP) c = c < 0 ? 0 : (c >= a.m ? a.m - 1 : c);
    const int cnt = (end - base) < kWave ? (end - base) : kWave;  // wave uniform

    if (G == 1) {
      int i = 0;
      for (; i + U <= cnt; i += U) {
        float b[U][CHUNKS][VEC];
        float vv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int32_t cc = __builtin_amdgcn_readlane(c, i + u);
          vv[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i + u));
          const float *brow = a.B + (int64_t)cc * a.ldb;
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch) load_vec<VEC>(brow + boff[ch], b[u][ch]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
            for (int x = 0; x < VEC; ++x) acc[ch][x] = fmaf(vv[u], b[u][ch][x], acc[ch][x]);
      }
      for (; i < cnt; ++i) {
        const int32_t cc = __builtin_amdgcn_readlane(c, i);
        const float vv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i));
        const float *brow = a.B + (int64_t)cc * a.ldb;
        float b[CHUNKS][VEC];
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) load_vec<VEC>(brow + boff[ch], b[ch]);
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
          for (int x = 0; x < VEC; ++x) acc[ch][x] = fmaf(vv, b[ch][x], acc[ch][x]);
      }
    } else {
      int i = 0;
      for (; i + U * G <= cnt; i += U * G) {
        float b[U][VEC];
        float vv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int src = i + u * G + g;
          const int32_t cc = __shfl(c, src, kWave);
          vv[u] = __shfl(v, src, kWave);
          load_vec<VEC>(a.B + (int64_t)cc * a.ldb + boff[0], b[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int x = 0; x < VEC; ++x) acc[0][x] = fmaf(vv[u], b[u][x], acc[0][x]);
      }
      for (; i < cnt; i += G) {
        const int src = i + g;
        const int32_t cc = __shfl(c, src, kWave);  // lanes past cnt hold col 0, val 0
        const float vv = __shfl(v, src, kWave);
        if (src < cnt) {
          float b[VEC];
          load_vec<VEC>(a.B + (int64_t)cc * a.ldb + boff[0], b);
#pragma unroll
          for (int x = 0; x < VEC; ++x) acc[0][x] = fmaf(vv, b[x], acc[0][x]);
        }
      }
    }
  }

  if (G > 1) {  // combine the teams: fixed butterfly, every lane ends with the full sum
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1) {
#pragma unroll
      for (int x = 0; x < VEC; ++x) acc[0][x] += __shfl_xor(acc[0][x], off, kWave);
    }
    if (g != 0) return;
  }

  if (single) {
    float *crow = a.C + (int64_t)row * a.ldc;
#pragma unroll
    for (int ch = 0; ch < CHUNKS; ++ch) {
      if (active[ch]) {
        float out[VEC];
        if (a.beta != 0.f) {
          float old[VEC];
          load_vec<VEC>(crow + boff[ch], old);
#pragma unroll
          for (int x = 0; x < VEC; ++x) out[x] = fmaf(a.beta, old[x], acc[ch][x]);
        } else {
#pragma unroll
          for (int x = 0; x < VEC; ++x) out[x] = acc[ch][x];
        }
        store_vec<VEC>(crow + boff[ch], out);
      }
    }
  } else {
    float *prow = a.P + (HUB ? task : ((int64_t)a.pbase[row] + sidx)) * a.f;
#pragma unroll
    for (int ch = 0; ch < CHUNKS; ++ch)
      if (active[ch]) store_vec<VEC>(prow + boff[ch], acc[ch]);
  }
}

// C[row, :] = beta*C[row, :] + sum over the row's partial rows, in segment order.
__global__ __launch_bounds__(kSpmmThreads) void spmm_reduce_kernel(const int32_t *__restrict__ multi_rows,
                                                                   int64_t nmulti, const int32_t *__restrict__ rowptr,
                                                                   const int32_t *__restrict__ pbase, int32_t seg,
                                                                   const float *__restrict__ P, float *__restrict__ C,
                                                                   int64_t ldc, int32_t f, float beta) {
  const int64_t idx = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  const int64_t mr = idx / f;
  const int32_t col = (int32_t)(idx % f);
  if (mr >= nmulti) return;
  const int32_t row = multi_rows[mr];
  const int32_t deg = rowptr[row + 1] - rowptr[row];
  const int32_t nseg = (deg + seg - 1) / seg;
  const float *p = P + (int64_t)pbase[row] * f + col;
  float s = 0.f;
  for (int32_t i = 0; i < nseg; ++i) s += p[(int64_t)i * f];
  float *c = C + (int64_t)row * ldc + col;
  *c = beta != 0.f ? fmaf(beta, *c, s) : s;
}

// ---------------------------------------------------------------------------------------------
// kernel selection
// ---------------------------------------------------------------------------------------------
struct SpmmShape {
  int vec, lpr, chunks;
};

constexpr int kMaxChunks = 10;

// Tuning knobs (cg_tune_set): 0 = built-in choice.
std::atomic<int> g_tune_seg{0}, g_tune_tiles{0}, g_tune_vec{0}, g_tune_stream{0}, g_tune_win{0};

// Widest vector the operands allow.
static int pick_vec(int32_t f, const float *B, int64_t ldb, const float *C, int64_t ldc) {
  const uintptr_t bits = (uintptr_t)B | (uintptr_t)C;
  const int cap = g_tune_vec.load(std::memory_order_relaxed);
  const int lim = (cap == 1 || cap == 2) ? cap : 4;
  if (lim >= 4 && f % 4 == 0 && ldb % 4 == 0 && ldc % 4 == 0 && bits % 16 == 0) return 4;
  if (lim >= 2 && f % 2 == 0 && ldb % 2 == 0 && ldc % 2 == 0 && bits % 8 == 0) return 2;
  return 1;
}

// Smallest team that covers `slots` vector slots (one tile's worth).
static SpmmShape pick_shape(int vec, int slots) {
  SpmmShape s{vec, 64, 1};
  if (slots <= 64) {
    int lpr = 4;
    while (lpr < slots) lpr <<= 1;
    s.lpr = lpr;
  } else {
    s.chunks = (slots + 63) / 64;
  }
  return s;
}

// Feature tiles per launch.  Wide outputs are split over the XCDs so that each L2 caches its own
// column slice of B; narrow ones (a row of B is a cache line or two) stay whole.
static int pick_tiles(int vec, int slots) {
  const int t = g_tune_tiles.load(std::memory_order_relaxed);
  if (t == 1 || t == 2 || t == 4 || t == 8) return slots >= t ? t : 1;
  (void)vec;
  return slots >= 256 ? 8 : 1;
}

template <int MODE>
static int launch_shape(const SpmmShape &s, const SpmmArgs &a, hipStream_t stream) {
  int64_t blocks = ceil_div64(a.ntasks, kWavesPerBlock);
  if (MODE == kModeHub) {
    int64_t longest = 0;
    for (int g = 0; g < a.groups; ++g) longest = longest > a.tstart[g + 1] - a.tstart[g] ? longest : a.tstart[g + 1] - a.tstart[g];
    blocks = ceil_div64(ceil_div64(longest, kWavesPerBlock), 8 / a.groups) * 8;
  } else if (a.tiles > 1) {
    blocks = ceil_div64(blocks, 8 / a.tiles) * 8;
  }
  if (blocks > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "SpMM grid too large");
  const unsigned grid = (unsigned)blocks;
  if (grid == 0) return CG_OK;
#define CG_CASE(V, L, CH)                                                                          \
  if (s.vec == V && s.lpr == L && s.chunks == CH) {                                                \
    spmm_rowseg_kernel<V, L, CH, MODE><<<grid, kSpmmThreads, 0, stream>>>(a);                      \
    CG_LAUNCH_CHECK();                                                                             \
    return CG_OK;                                                                                  \
  }
#define CG_CASES(V)                                                                                \
  CG_CASE(V, 4, 1) CG_CASE(V, 8, 1) CG_CASE(V, 16, 1) CG_CASE(V, 32, 1) CG_CASE(V, 64, 1)           \
  CG_CASE(V, 64, 2) CG_CASE(V, 64, 3) CG_CASE(V, 64, 4) CG_CASE(V, 64, 5) CG_CASE(V, 64, 6)           \
  CG_CASE(V, 64, 7) CG_CASE(V, 64, 8) CG_CASE(V, 64, 9) CG_CASE(V, 64, 10)
  CG_CASES(1) CG_CASES(2) CG_CASES(4)
#undef CG_CASES
#undef CG_CASE
  CG_FAIL(CG_ERR_UNSUPPORTED, "no SpMM kernel for vec=%d lpr=%d chunks=%d", s.vec, s.lpr, s.chunks);
}

// One launch covers at most tiles * 64 * kMaxChunks slots; wider outputs take several launches
// over column ranges.  Fills the tiling fields of `a` for the range [f0, f0 + ft).
struct SpmmPlan {
  SpmmShape shape;
  int tiles, tile_slots;
};
static SpmmPlan plan_range(int vec, int32_t ft) {
  const int slots = ft / vec;
  SpmmPlan p;
  p.tiles = pick_tiles(vec, slots);
  p.tile_slots = (slots + p.tiles - 1) / p.tiles;
  p.shape = pick_shape(vec, p.tile_slots);
  return p;
}
static int32_t range_cap(int vec) { return kWave * kMaxChunks * vec; }

static int check_dense(const char *who, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f,
                       int64_t brows, int64_t crows) {
  if (f <= 0) CG_FAIL(CG_ERR_SIZE, "%s: f=%d must be positive", who, f);
  if (ldb < f || ldc < f) CG_FAIL(CG_ERR_SIZE, "%s: leading dimension smaller than f (ldb=%lld ldc=%lld f=%d)", who,
                                  (long long)ldb, (long long)ldc, f);
  if ((!B && brows > 0) || (!C && crows > 0)) CG_FAIL(CG_ERR_NULL, "%s: null dense operand", who);
  if (B && C && (const float *)C == B) CG_FAIL(CG_ERR_ALIAS, "%s: C aliases B", who);
  return CG_OK;
}

// ---------------------------------------------------------------------------------------------
// schedules (row segments), built on the device
// ---------------------------------------------------------------------------------------------
// skip_empty: rows without entries get no task (hub plans); otherwise every row has at least one,
// because a beta != 1 launch still has to scale the row of C.
__device__ __forceinline__ uint32_t tasks_of(int32_t deg, int32_t seg, int skip_empty) {
  if (deg <= 0) return skip_empty ? 0u : 1u;
  return deg <= seg ? 1u : (uint32_t)((deg + seg - 1) / seg);
}

__global__ __launch_bounds__(kSpmmThreads) void sched_count_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                   int32_t seg, int skip_empty,
                                                                   uint32_t *__restrict__ ntask,
                                                                   uint32_t *__restrict__ nslot,
                                                                   uint32_t *__restrict__ nmulti) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r >= n) return;
  const uint32_t t = tasks_of(rowptr[r + 1] - rowptr[r], seg, skip_empty);
  ntask[r] = t;
  nslot[r] = t > 1 ? t : 0u;
  nmulti[r] = t > 1 ? 1u : 0u;
}

__global__ __launch_bounds__(kSpmmThreads) void sched_fill_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                  int32_t seg, int skip_empty,
                                                                  const uint32_t *__restrict__ tbase,
                                                                  const uint32_t *__restrict__ mbase,
                                                                  int32_t *__restrict__ task_row,
                                                                  int32_t *__restrict__ multi_rows) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r >= n) return;
  const uint32_t t = tasks_of(rowptr[r + 1] - rowptr[r], seg, skip_empty);
  const uint32_t b = tbase[r];
  for (uint32_t i = 0; i < t; ++i) task_row[b + i] = (int32_t)r;
  if (t > 1) multi_rows[mbase[r]] = (int32_t)r;
}

__global__ __launch_bounds__(kSpmmThreads) void max_degree_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                  int *__restrict__ out) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  int32_t deg = 0;
  if (r < n) deg = rowptr[r + 1] - rowptr[r];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    int32_t o = __shfl_xor(deg, off, kWave);
    deg = o > deg ? o : deg;
  }
  if ((threadIdx.x & (kWave - 1)) == 0 && deg > 0) atomicMax(out, deg);  // integer max: order independent
}

struct Sched {
  int32_t seg = 0;
  int64_t ntasks = 0, nmulti = 0, nslots = 0;
  int32_t *task_row = nullptr, *tbase = nullptr, *pbase = nullptr, *multi_rows = nullptr;
  void release() {
    if (task_row) (void)hipFree(task_row);
    if (tbase) (void)hipFree(tbase);
    if (pbase) (void)hipFree(pbase);
    if (multi_rows) (void)hipFree(multi_rows);
    task_row = tbase = pbase = multi_rows = nullptr;
  }
};

static int dev_alloc(void **p, size_t bytes) {
  hipError_t e = hipMalloc(p, bytes ? bytes : 4);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *p = nullptr;
    set_error("hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
    return CG_ERR_ALLOC;
  }
  return CG_OK;
}

// Task tables for the rows [0, n) described by rowptr.  Synchronises `stream`.
static int make_sched(const int32_t *rowptr, int32_t n, int32_t seg, int skip_empty, Sched &out, hipStream_t stream) {
  Sched sc;
  sc.seg = seg;
  const size_t nb = (size_t)(n + 1) * sizeof(uint32_t);
  uint32_t *d_mbase = nullptr;
  void *d_totals_v = nullptr;
  int st = CG_OK;
  do {
    if ((st = dev_alloc((void **)&sc.tbase, nb)) != CG_OK) break;
    if ((st = dev_alloc((void **)&sc.pbase, nb)) != CG_OK) break;
    if ((st = dev_alloc((void **)&d_mbase, nb)) != CG_OK) break;
    if ((st = scratch_get(stream, kSlotB, 3 * sizeof(uint32_t), &d_totals_v)) != CG_OK) break;
    uint32_t *d_totals = (uint32_t *)d_totals_v;
    uint32_t totals[3] = {0, 0, 0};
    if (n > 0) {
      const unsigned grid = (unsigned)ceil_div64(n, kSpmmThreads);
      sched_count_kernel<<<grid, kSpmmThreads, 0, stream>>>(rowptr, n, seg, skip_empty, (uint32_t *)sc.tbase,
                                                            (uint32_t *)sc.pbase, d_mbase);
      if (hipGetLastError() != hipSuccess) { st = CG_ERR_HIP; set_error("sched_count launch failed"); break; }
      // scanning n + 1 entries puts the grand total behind the last row: tbase[n] == ntasks
      if ((st = hipMemsetAsync((uint32_t *)sc.tbase + n, 0, 4, stream) == hipSuccess ? CG_OK : CG_ERR_HIP) != CG_OK) break;
      if ((st = hipMemsetAsync((uint32_t *)sc.pbase + n, 0, 4, stream) == hipSuccess ? CG_OK : CG_ERR_HIP) != CG_OK) break;
      if ((st = exclusive_scan_u32((uint32_t *)sc.tbase, (uint32_t *)sc.tbase, (int64_t)n + 1, d_totals + 0, stream)) != CG_OK) break;
      if ((st = exclusive_scan_u32((uint32_t *)sc.pbase, (uint32_t *)sc.pbase, (int64_t)n + 1, d_totals + 1, stream)) != CG_OK) break;
      if ((st = exclusive_scan_u32(d_mbase, d_mbase, n, d_totals + 2, stream)) != CG_OK) break;
      if (hipMemcpyAsync(totals, d_totals, sizeof(totals), hipMemcpyDeviceToHost, stream) != hipSuccess ||
          hipStreamSynchronize(stream) != hipSuccess) {
        st = CG_ERR_HIP;
        set_error("schedule totals copy failed");
        break;
      }
    }
    sc.ntasks = totals[0];
    sc.nslots = totals[1];
    sc.nmulti = totals[2];
    if ((st = dev_alloc((void **)&sc.task_row, (size_t)sc.ntasks * sizeof(int32_t))) != CG_OK) break;
    if ((st = dev_alloc((void **)&sc.multi_rows, (size_t)sc.nmulti * sizeof(int32_t))) != CG_OK) break;
    if (n > 0) {
      const unsigned grid = (unsigned)ceil_div64(n, kSpmmThreads);
      sched_fill_kernel<<<grid, kSpmmThreads, 0, stream>>>(rowptr, n, seg, skip_empty, (const uint32_t *)sc.tbase,
                                                           d_mbase, sc.task_row, sc.multi_rows);
      if (hipGetLastError() != hipSuccess) { st = CG_ERR_HIP; set_error("sched_fill launch failed"); break; }
      if (hipStreamSynchronize(stream) != hipSuccess) { st = CG_ERR_HIP; set_error("sched_fill failed"); break; }
    }
  } while (0);
  if (d_mbase) (void)hipFree(d_mbase);
  if (st != CG_OK) {
    sc.release();
    return st;
  }
  out = sc;
  return CG_OK;
}

struct TempFree {
  void *p[16];
  int count = 0;
  ~TempFree() {
    for (int i = 0; i < count; ++i)
      if (p[i]) (void)hipFree(p[i]);
  }
  int alloc(void **out, size_t bytes) {
    CG_TRY(dev_alloc(out, bytes));
    p[count++] = *out;
    return CG_OK;
  }
};

// ---------------------------------------------------------------------------------------------
// streaming over windows of tasks
// ---------------------------------------------------------------------------------------------
// Tasks are contiguous in the entry stream (task t covers [task_start[t], task_start[t+1])), so a
// wavefront that takes a window of consecutive tasks reads one contiguous piece of (colind, val)
// and never pays a task's start-up latency more than once per window.  Windows hold at most 64
// tasks (their metadata lives in one register per lane) and start a new one every `S` entries.
struct StreamTab {
  int32_t S = 0, groups = 0;
  bool hub = false;
  int32_t *task_start = nullptr, *task_dst = nullptr, *wstart = nullptr;
  int64_t nwin = 0;
  int64_t win_first[18] = {0};
  void release() {
    if (task_start) (void)hipFree(task_start);
    if (task_dst) (void)hipFree(task_dst);
    if (wstart) (void)hipFree(wstart);
    task_start = task_dst = wstart = nullptr;
    S = 0;
  }
};

// task_dst: row index (>= 0) when the task is the whole row and goes straight to C, else
// -(partial slot + 1).  In a hub plan every task is partial and its slot is its own index.
__global__ __launch_bounds__(kSpmmThreads) void stream_tasks_kernel(const int32_t *__restrict__ rowptr, int32_t nrows,
                                                                    const int32_t *__restrict__ task_row,
                                                                    const int32_t *__restrict__ tbase,
                                                                    const int32_t *__restrict__ pbase, int32_t seg,
                                                                    int64_t ntasks, int hub,
                                                                    int32_t *__restrict__ task_start,
                                                                    int32_t *__restrict__ task_dst) {
  const int64_t t = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (t > ntasks) return;
  if (t == ntasks) {
    task_start[t] = rowptr[nrows];
    return;
  }
  const int32_t row = task_row[t];
  const int32_t sidx = (int32_t)t - tbase[row];
  const int32_t rs = rowptr[row], re = rowptr[row + 1];
  task_start[t] = rs + sidx * seg;
  task_dst[t] = hub ? -((int32_t)t + 1) : ((re - rs <= seg) ? row : -(pbase[row] + sidx + 1));
}

// flags[t] = 1 where a window starts: every 64th task of a class ...
__global__ __launch_bounds__(kSpmmThreads) void window_flag_tasks_kernel(int64_t t0, int64_t t1,
                                                                         uint32_t *__restrict__ flags) {
  const int64_t t = t0 + (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (t < t1) flags[t] = ((t - t0) & 63) == 0 ? 1u : 0u;
}

// ... and the first task that starts at or after every multiple of S entries of the class.
__global__ __launch_bounds__(kSpmmThreads) void window_flag_entries_kernel(const int32_t *__restrict__ task_start,
                                                                           int64_t t0, int64_t t1, int32_t S,
                                                                           int64_t nbounds,
                                                                           uint32_t *__restrict__ flags) {
  const int64_t j = 1 + (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (j > nbounds) return;
  const int64_t target = (int64_t)task_start[t0] + j * S;
  int64_t lo = t0, hi = t1;  // first t in [t0, t1) with task_start[t] >= target
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (task_start[mid] < target) lo = mid + 1;
    else hi = mid;
  }
  if (lo < t1) flags[lo] = 1u;  // several j may land on the same task: they all store 1
}

__global__ __launch_bounds__(kSpmmThreads) void window_compact_kernel(const uint32_t *__restrict__ flags,
                                                                      const uint32_t *__restrict__ index,
                                                                      int64_t ntasks, int32_t *__restrict__ wstart,
                                                                      uint32_t nwin) {
  const int64_t t = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (t < ntasks && flags[t]) wstart[index[t]] = (int32_t)t;
  if (t == ntasks) wstart[nwin] = (int32_t)ntasks;
}

// class_first[g] .. class_first[g+1]: tasks of class g (nclass == 1 for a plain schedule).
static int build_stream(const Sched &sc, const int32_t *rowptr, int32_t nrows, bool hub, int nclass,
                        const int64_t *class_first, int32_t S, StreamTab &out, hipStream_t stream) {
  out.release();
  const int64_t nt = sc.ntasks;
  CG_TRY(dev_alloc((void **)&out.task_start, (size_t)(nt + 1) * 4));
  CG_TRY(dev_alloc((void **)&out.task_dst, (size_t)(nt + 1) * 4));
  stream_tasks_kernel<<<(unsigned)ceil_div64(nt + 1, kSpmmThreads), kSpmmThreads, 0, stream>>>(
      rowptr, nrows, sc.task_row, sc.tbase, sc.pbase, sc.seg, nt, hub ? 1 : 0, out.task_start, out.task_dst);
  CG_LAUNCH_CHECK();
  out.S = S;
  out.hub = hub;
  out.groups = nclass;
  out.nwin = 0;
  for (int g = 0; g <= nclass; ++g) out.win_first[g] = 0;
  if (nt == 0) {
    CG_TRY(dev_alloc((void **)&out.wstart, 4));
    CG_HIP(hipMemsetAsync(out.wstart, 0, 4, stream));
    CG_HIP(hipStreamSynchronize(stream));
    return CG_OK;
  }
  uint32_t *flags = nullptr, *index = nullptr;
  TempFree tmp;
  CG_TRY(tmp.alloc((void **)&flags, (size_t)(nt + 1) * 4));
  CG_TRY(tmp.alloc((void **)&index, (size_t)(nt + 1) * 4));
  // entry extents of the classes (host needs them to size the boundary launches)
  int32_t ends[18];
  for (int g = 0; g <= nclass; ++g)
    CG_HIP(hipMemcpyAsync(&ends[g], out.task_start + class_first[g], 4, hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  for (int g = 0; g < nclass; ++g) {
    const int64_t t0 = class_first[g], t1 = class_first[g + 1];
    if (t1 <= t0) continue;
    window_flag_tasks_kernel<<<(unsigned)ceil_div64(t1 - t0, kSpmmThreads), kSpmmThreads, 0, stream>>>(t0, t1, flags);
    CG_LAUNCH_CHECK();
    const int64_t nb = ((int64_t)ends[g + 1] - ends[g]) / S;
    if (nb > 0) {
      window_flag_entries_kernel<<<(unsigned)ceil_div64(nb, kSpmmThreads), kSpmmThreads, 0, stream>>>(
          out.task_start, t0, t1, S, nb, flags);
      CG_LAUNCH_CHECK();
    }
  }
  void *d_total_v = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, 4, &d_total_v));
  CG_TRY(exclusive_scan_u32(flags, index, nt, (uint32_t *)d_total_v, stream));
  uint32_t nwin = 0;
  CG_HIP(hipMemcpyAsync(&nwin, d_total_v, 4, hipMemcpyDeviceToHost, stream));
  uint32_t firsts[18] = {0};
  for (int g = 0; g < nclass; ++g)
    if (class_first[g] < nt) CG_HIP(hipMemcpyAsync(&firsts[g], index + class_first[g], 4, hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  for (int g = 0; g < nclass; ++g) out.win_first[g] = class_first[g] < nt ? firsts[g] : nwin;
  out.win_first[nclass] = nwin;
  out.nwin = nwin;
  CG_TRY(dev_alloc((void **)&out.wstart, (size_t)(nwin + 1) * 4));
  window_compact_kernel<<<(unsigned)ceil_div64(nt + 1, kSpmmThreads), kSpmmThreads, 0, stream>>>(flags, index, nt,
                                                                                                out.wstart, nwin);
  CG_LAUNCH_CHECK();
  CG_HIP(hipStreamSynchronize(stream));
  return CG_OK;
}

struct StreamArgs {
  const int32_t *task_start, *task_dst, *wstart;
  const int32_t *colind;
  const float *val;
  int64_t win_first[9];
  int32_t groups;  // 1: windows run anywhere; 2/4/8: windows of class g run on XCDs x % groups == g
  const float *B;
  int64_t ldb;
  float *C;
  int64_t ldc;
  float *P;
  int32_t f;
  float beta;
};

// Full-wave teams (one stored entry per wave step, f covered by CHUNKS x 64 lanes x VEC floats).
template <int VEC, int CHUNKS>
__global__ __launch_bounds__(kSpmmThreads) void spmm_stream_wide_kernel(const StreamArgs a) {
  const int lane = threadIdx.x & (kWave - 1);
  const int x = blockIdx.x & 7;
  const int per = 8 / a.groups;
  const int grp = x % a.groups;
  const int64_t lblock = (int64_t)(blockIdx.x >> 3) * per + x / a.groups;
  const int64_t wl = lblock * kWavesPerBlock + threadIdx.x / kWave;
  if (wl >= a.win_first[grp + 1] - a.win_first[grp]) return;
  const int32_t w = __builtin_amdgcn_readfirstlane((int32_t)(a.win_first[grp] + wl));
  const int32_t t0 = a.wstart[w], t1 = a.wstart[w + 1];
  const int ntask = t1 - t0;  // 1..64
  int32_t m_end = 0, m_dst = 0;
  if (lane < ntask) {
    m_end = a.task_start[t0 + lane + 1];
    m_dst = a.task_dst[t0 + lane];
  }
  const int32_t e_begin = a.task_start[t0];
  const int32_t e_end = __builtin_amdgcn_readlane(m_end, ntask - 1);

  const int nslots = a.f / VEC;
  bool active[CHUNKS];
  int64_t boff[CHUNKS];
#pragma unroll
  for (int ch = 0; ch < CHUNKS; ++ch) {
    active[ch] = (ch * kWave + lane) < nslots;
    boff[ch] = (int64_t)(ch * kWave + (active[ch] ? lane : 0)) * VEC;
  }
  float acc[CHUNKS][VEC];
#pragma unroll
  for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[ch][v] = 0.f;

  constexpr int U = 4;
  int tk = 0;
  int32_t tbeg = e_begin;
  int32_t tend = __builtin_amdgcn_readlane(m_end, 0);

  int32_t c_next = 0;
  float v_next = 0.f;
  if (e_begin + lane < e_end) {
    c_next = a.colind[e_begin + lane];
    v_next = a.val[e_begin + lane];
  }
  for (int32_t base = e_begin;; base += kWave) {
    const int32_t c = c_next;
    const float v = v_next;
    const int32_t nb = base + kWave + lane;
    c_next = 0;
    v_next = 0.f;
    if (nb < e_end) {
      c_next = a.colind[nb];
      v_next = a.val[nb];
    }
    int cnt = e_end - base;
    cnt = cnt > kWave ? kWave : (cnt < 0 ? 0 : cnt);
    int i = 0;
    for (;;) {
      while (tend == base + i) {  // the current task is complete (also true at once for an empty task)
        const int32_t dst = __builtin_amdgcn_readlane(m_dst, tk);
        if (dst >= 0) {
          if (!(tend == tbeg && a.beta == 1.0f)) {  // an empty row leaves C alone when beta == 1
            float *crow = a.C + (int64_t)dst * a.ldc;
#pragma unroll
            for (int ch = 0; ch < CHUNKS; ++ch) {
              if (active[ch]) {
                float out[VEC];
                if (a.beta != 0.f) {
                  float old[VEC];
                  load_vec<VEC>(crow + boff[ch], old);
#pragma unroll
                  for (int q = 0; q < VEC; ++q) out[q] = fmaf(a.beta, old[q], acc[ch][q]);
                } else {
#pragma unroll
                  for (int q = 0; q < VEC; ++q) out[q] = acc[ch][q];
                }
                store_vec<VEC>(crow + boff[ch], out);
              }
            }
          }
        } else {
          float *prow = a.P + (int64_t)(-(dst + 1)) * a.f;
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch)
            if (active[ch]) store_vec<VEC>(prow + boff[ch], acc[ch]);
        }
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
          for (int q = 0; q < VEC; ++q) acc[ch][q] = 0.f;
        if (++tk == ntask) return;
        tbeg = tend;
        tend = __builtin_amdgcn_readlane(m_end, tk);
      }
      if (i >= cnt) break;
      int run = tend - base;
      run = run < cnt ? run : cnt;
      if (run <= i) return;  // cannot happen with monotone task starts; guarantees termination
      for (; i + U <= run; i += U) {
        float b[U][CHUNKS][VEC];
        float vv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int32_t cc = __builtin_amdgcn_readlane(c, i + u);
          vv[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i + u));
          const float *brow = a.B + (int64_t)cc * a.ldb;
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch) load_vec<VEC>(brow + boff[ch], b[u][ch]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
            for (int q = 0; q < VEC; ++q) acc[ch][q] = fmaf(vv[u], b[u][ch][q], acc[ch][q]);
      }
      for (; i < run; ++i) {
        const int32_t cc = __builtin_amdgcn_readlane(c, i);
        const float vv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i));
        const float *brow = a.B + (int64_t)cc * a.ldb;
        float b[CHUNKS][VEC];
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) load_vec<VEC>(brow + boff[ch], b[ch]);
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
          for (int q = 0; q < VEC; ++q) acc[ch][q] = fmaf(vv, b[ch][q], acc[ch][q]);
      }
    }
  }
}

static int launch_stream_wide(int vec, int chunks, const StreamArgs &a, hipStream_t stream) {
  int64_t longest = 0;
  for (int g = 0; g < a.groups; ++g) {
    const int64_t len = a.win_first[g + 1] - a.win_first[g];
    longest = longest > len ? longest : len;
  }
  const int64_t blocks = ceil_div64(ceil_div64(longest, kWavesPerBlock), 8 / a.groups) * 8;
  if (blocks == 0) return CG_OK;
  if (blocks > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "SpMM grid too large");
  const unsigned grid = (unsigned)blocks;
#define CG_CASE(V, CH)                                                              \
  if (vec == V && chunks == CH) {                                                   \
    spmm_stream_wide_kernel<V, CH><<<grid, kSpmmThreads, 0, stream>>>(a);           \
    CG_LAUNCH_CHECK();                                                              \
    return CG_OK;                                                                   \
  }
#define CG_CASES(V)                                                                                     \
  CG_CASE(V, 1) CG_CASE(V, 2) CG_CASE(V, 3) CG_CASE(V, 4) CG_CASE(V, 5) CG_CASE(V, 6) CG_CASE(V, 7)     \
  CG_CASE(V, 8) CG_CASE(V, 9) CG_CASE(V, 10)
  CG_CASES(1) CG_CASES(2) CG_CASES(4)
#undef CG_CASES
#undef CG_CASE
  CG_FAIL(CG_ERR_UNSUPPORTED, "no streaming SpMM kernel for vec=%d chunks=%d", vec, chunks);
}

// Teams of LPR < 64 lanes (f <= 64 * VEC floats): the window's entries and task table are staged
// in LDS.  Long tasks (>= kLongFactor * G entries) are worked on by all G teams together (entries
// dealt round robin, partial sums combined by the xor butterfly); the short ones are dealt to the
// teams whole, G at a time, so rows of a few entries cost neither a butterfly nor an idle wave.
constexpr int kNarrowLds = 1024;  // entries a window may hold (window length S plus one task, both <= 512)
constexpr int kLongFactor = 4;

template <int VEC, int LPR>
__global__ __launch_bounds__(kSpmmThreads) void spmm_stream_narrow_kernel(const StreamArgs a) {
  constexpr int G = kWave / LPR;
  __shared__ int32_t s_col[kWavesPerBlock][kNarrowLds];
  __shared__ float s_val[kWavesPerBlock][kNarrowLds];
  __shared__ int32_t s_beg[kWavesPerBlock][kWave], s_end[kWavesPerBlock][kWave], s_dst[kWavesPerBlock][kWave];
  __shared__ int32_t s_short[kWavesPerBlock][kWave];

  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x / kWave;
  const int x = blockIdx.x & 7;
  const int per = 8 / a.groups;
  const int grp = x % a.groups;
  const int64_t lblock = (int64_t)(blockIdx.x >> 3) * per + x / a.groups;
  const int64_t wl = lblock * kWavesPerBlock + wv;
  if (wl >= a.win_first[grp + 1] - a.win_first[grp]) return;
  const int32_t w = __builtin_amdgcn_readfirstlane((int32_t)(a.win_first[grp] + wl));
  const int32_t t0 = a.wstart[w], t1 = a.wstart[w + 1];
  const int ntask = t1 - t0;  // 1..64
  const bool valid = lane < ntask;
  int32_t m_beg = 0, m_end = 0, m_dst = 0;
  if (valid) {
    m_beg = a.task_start[t0 + lane];
    m_end = a.task_start[t0 + lane + 1];
    m_dst = a.task_dst[t0 + lane];
  }
  const int32_t e_begin = __builtin_amdgcn_readlane(m_beg, 0);
  const int32_t e_end = __builtin_amdgcn_readlane(m_end, ntask - 1);
  const int32_t nent = e_end - e_begin;
  if (nent > kNarrowLds) return;  // excluded by the schedule (S + seg <= kNarrowLds); keeps LDS writes in bounds

  for (int32_t k = lane; k < nent; k += kWave) {
    s_col[wv][k] = a.colind[e_begin + k];
    s_val[wv][k] = a.val[e_begin + k];
  }
  const int32_t r_beg = m_beg - e_begin, r_end = m_end - e_begin;  // relative to the window
  s_beg[wv][lane] = r_beg;
  s_end[wv][lane] = r_end;
  s_dst[wv][lane] = m_dst;
  const int32_t len = r_end - r_beg;
  const bool is_long = valid && len >= kLongFactor * G;
  // an empty row that goes straight to C needs no work when beta == 1
  const bool is_short = valid && !is_long && !(len == 0 && m_dst >= 0 && a.beta == 1.0f);

  const int g = lane / LPR, j = lane % LPR;
  const bool active = j * VEC < a.f;
  const int64_t boff = active ? (int64_t)j * VEC : 0;
  const int32_t *cw = s_col[wv];
  const float *vw = s_val[wv];

  const uint64_t short_mask = __ballot(is_short);
  if (is_short) s_short[wv][__popcll(short_mask & ((1ull << lane) - 1ull))] = lane;
  const int nshort = __popcll(short_mask);
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();  // the staged window and tables are visible to every lane of the wave

  // ---- long tasks: all teams together
  uint64_t long_mask = __ballot(is_long);
  while (long_mask) {
    const int k = __builtin_ctzll(long_mask);
    long_mask &= long_mask - 1;
    const int32_t s = __builtin_amdgcn_readlane(r_beg, k);
    const int32_t e = __builtin_amdgcn_readlane(r_end, k);
    const int32_t d = __builtin_amdgcn_readlane(m_dst, k);
    float acc[VEC];
#pragma unroll
    for (int q = 0; q < VEC; ++q) acc[q] = 0.f;
    int32_t i = s + g;
    for (; i + 3 * G < e; i += 4 * G) {
      float b[4][VEC], vv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int32_t cc = cw[i + u * G];
        vv[u] = vw[i + u * G];
        load_vec<VEC>(a.B + (int64_t)cc * a.ldb + boff, b[u]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int q = 0; q < VEC; ++q) acc[q] = fmaf(vv[u], b[u][q], acc[q]);
    }
    for (; i < e; i += G) {
      float b[VEC];
      const float vv = vw[i];
      load_vec<VEC>(a.B + (int64_t)cw[i] * a.ldb + boff, b);
#pragma unroll
      for (int q = 0; q < VEC; ++q) acc[q] = fmaf(vv, b[q], acc[q]);
    }
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1)
#pragma unroll
      for (int q = 0; q < VEC; ++q) acc[q] += __shfl_xor(acc[q], off, kWave);
    if (g == 0 && active) {
      if (d >= 0) {
        float *crow = a.C + (int64_t)d * a.ldc + boff;
        float out[VEC];
        if (a.beta != 0.f) {
          float old[VEC];
          load_vec<VEC>(crow, old);
#pragma unroll
          for (int q = 0; q < VEC; ++q) out[q] = fmaf(a.beta, old[q], acc[q]);
        } else {
#pragma unroll
          for (int q = 0; q < VEC; ++q) out[q] = acc[q];
        }
        store_vec<VEC>(crow, out);
      } else {
        store_vec<VEC>(a.P + (int64_t)(-(d + 1)) * a.f + boff, acc);
      }
    }
  }

  // ---- short tasks: one team each, G per round
  for (int q0 = 0; q0 < nshort; q0 += G) {
    const int my = q0 + g;
    const bool has = my < nshort;
    const int k = has ? s_short[wv][my] : 0;
    const int32_t s = s_beg[wv][k];
    const int32_t e = has ? s_end[wv][k] : s;
    const int32_t d = s_dst[wv][k];
    float acc[VEC];
#pragma unroll
    for (int q = 0; q < VEC; ++q) acc[q] = 0.f;
    int32_t i = s;
    for (; i + 3 < e; i += 4) {
      float b[4][VEC], vv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int32_t cc = cw[i + u];
        vv[u] = vw[i + u];
        load_vec<VEC>(a.B + (int64_t)cc * a.ldb + boff, b[u]);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int q = 0; q < VEC; ++q) acc[q] = fmaf(vv[u], b[u][q], acc[q]);
    }
    for (; i < e; ++i) {
      float b[VEC];
      const float vv = vw[i];
      load_vec<VEC>(a.B + (int64_t)cw[i] * a.ldb + boff, b);
#pragma unroll
      for (int q = 0; q < VEC; ++q) acc[q] = fmaf(vv, b[q], acc[q]);
    }
    if (has && active) {
      if (d >= 0) {
        float *crow = a.C + (int64_t)d * a.ldc + boff;
        float out[VEC];
        if (a.beta != 0.f) {
          float old[VEC];
          load_vec<VEC>(crow, old);
#pragma unroll
          for (int q = 0; q < VEC; ++q) out[q] = fmaf(a.beta, old[q], acc[q]);
        } else {
#pragma unroll
          for (int q = 0; q < VEC; ++q) out[q] = acc[q];
        }
        store_vec<VEC>(crow, out);
      } else {
        store_vec<VEC>(a.P + (int64_t)(-(d + 1)) * a.f + boff, acc);
      }
    }
  }
}

static int64_t stream_grid(const StreamArgs &a) {
  int64_t longest = 0;
  for (int g = 0; g < a.groups; ++g) {
    const int64_t len = a.win_first[g + 1] - a.win_first[g];
    longest = longest > len ? longest : len;
  }
  return ceil_div64(ceil_div64(longest, kWavesPerBlock), 8 / a.groups) * 8;
}

static int launch_stream_narrow(int vec, int lpr, const StreamArgs &a, hipStream_t stream) {
  const int64_t blocks = stream_grid(a);
  if (blocks == 0) return CG_OK;
  if (blocks > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "SpMM grid too large");
  const unsigned grid = (unsigned)blocks;
#define CG_CASE(V, L)                                                               \
  if (vec == V && lpr == L) {                                                       \
    spmm_stream_narrow_kernel<V, L><<<grid, kSpmmThreads, 0, stream>>>(a);          \
    CG_LAUNCH_CHECK();                                                              \
    return CG_OK;                                                                   \
  }
#define CG_CASES(V) CG_CASE(V, 4) CG_CASE(V, 8) CG_CASE(V, 16) CG_CASE(V, 32)
  CG_CASES(1) CG_CASES(2) CG_CASES(4)
#undef CG_CASES
#undef CG_CASE
  CG_FAIL(CG_ERR_UNSUPPORTED, "no narrow streaming SpMM kernel for vec=%d lpr=%d", vec, lpr);
}

// A small cache of schedules keyed by segment length.
struct SchedCache {
  static constexpr int kMax = 4;
  Sched sched[kMax];
  StreamTab tab[kMax];  // window tables of sched[i], built on first use
  int count = 0;
  void release() {
    for (int i = 0; i < count; ++i) {
      sched[i].release();
      tab[i].release();
    }
    count = 0;
  }
  StreamTab &tab_of(const Sched *s) { return tab[s - sched]; }
  int get(const int32_t *rowptr, int32_t n, int32_t seg, Sched **out, hipStream_t stream) {
    for (int i = 0; i < count; ++i)
      if (sched[i].seg == seg) {
        *out = &sched[i];
        return CG_OK;
      }
    if (count == kMax) {  // recycle the oldest
      CG_HIP(hipStreamSynchronize(stream));
      sched[0].release();
      tab[0].release();
      for (int i = 1; i < count; ++i) {
        sched[i - 1] = sched[i];
        tab[i - 1] = tab[i];
      }
      sched[--count] = Sched();
      tab[count] = StreamTab();
    }
    CG_TRY(make_sched(rowptr, n, seg, 0, sched[count], stream));
    *out = &sched[count++];
    return CG_OK;
  }
};

// Hub plan: the stored entries regrouped by column class.  Columns (= rows of B) are ranked by
// descending reference count; the first `hot` ranks form tier 0, the next `hot` tier 1, ...; inside
// a tier the columns are dealt round robin to `groups` groups, and every column behind the last
// tier is cold.  Class = tier * groups + group.  A tier is one launch in which XCD x only reads the
// B rows of group x % groups, sized to stay resident in that XCD's L2.  Entries are kept as one CSR
// over (classes + 1) * rows virtual rows, virtual row c * rows + r holding the entries of row r whose
// column has class c (cold = class `classes`).
struct HubPlan {
  int32_t hot = 0, groups = 0, tiers = 0, seg = 0;
  int32_t classes() const { return groups * tiers; }
  int32_t *vrowptr = nullptr, *colind = nullptr;
  float *val = nullptr;
  Sched hot_sched;        // over the virtual rows of the hot classes, empty rows skipped
  StreamTab hot_tab;      // its windows, one class per group
  SchedCache cold_sched;  // over the cold class
  int64_t tstart[18] = {0};
  bool valid = false;
  void release() {
    hot_sched.release();
    hot_tab.release();
    cold_sched.release();
    if (vrowptr) (void)hipFree(vrowptr);
    if (colind) (void)hipFree(colind);
    if (val) (void)hipFree(val);
    vrowptr = colind = nullptr;
    val = nullptr;
    valid = false;
  }
};

struct CsrSide {
  int32_t rows = 0, cols = 0;
  int64_t nnz = 0;
  int32_t *rowptr = nullptr, *colind = nullptr;
  float *val = nullptr;
  int32_t max_degree = 0;
  SchedCache sched;
  HubPlan hub;
  void release() {
    sched.release();
    hub.release();
    if (rowptr) (void)hipFree(rowptr);
    if (colind) (void)hipFree(colind);
    if (val) (void)hipFree(val);
    rowptr = colind = nullptr;
    val = nullptr;
  }
};

// Entries per task.  A team step consumes G entries per wave instruction, so narrow outputs get
// longer segments for the same number of steps.
static int32_t pick_seg(const SpmmShape &s) {
  const int t = g_tune_seg.load(std::memory_order_relaxed);
  if (t >= 64) return t;
  const int g = kWave / s.lpr;
  if (g == 1) return 1024;
  if (g_tune_stream.load(std::memory_order_relaxed) >= 0) return 512;  // a window and one task fit the LDS stage
  if (g == 2) return 2048;
  return 4096;
}

// ---------------------------------------------------------------------------------------------
// hub plan construction
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kSpmmThreads) void col_count_kernel(const int32_t *__restrict__ colind, int64_t nnz,
                                                                 uint32_t *__restrict__ count) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < nnz) atomicAdd(&count[colind[k]], 1u);  // integer count: independent of arrival order
}

// sort key that orders columns by descending count (ties: ascending column, by stability)
__global__ __launch_bounds__(kSpmmThreads) void col_key_kernel(const uint32_t *__restrict__ count, int32_t m,
                                                               uint32_t maxcount, int32_t *__restrict__ key,
                                                               int32_t *__restrict__ id) {
  const int64_t j = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (j < m) {
    key[j] = (int32_t)(maxcount - count[j]);
    id[j] = (int32_t)j;
  }
}

// class of every column from its rank: `hot` ranks per tier, dealt round robin to the groups
__global__ __launch_bounds__(kSpmmThreads) void col_class_kernel(const int32_t *__restrict__ ranked_col, int32_t m,
                                                                 int32_t hot, int32_t groups, int32_t tiers,
                                                                 int32_t *__restrict__ cls) {
  const int64_t rank = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (rank >= m) return;
  const int64_t tier = rank / hot;
  cls[ranked_col[rank]] = tier < tiers ? (int32_t)(tier * groups + (rank % hot) % groups) : groups * tiers;
}

__global__ __launch_bounds__(kSpmmThreads) void entry_class_kernel(const int32_t *__restrict__ colind, int64_t nnz,
                                                                   const int32_t *__restrict__ cls,
                                                                   int32_t *__restrict__ out) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < nnz) out[k] = cls[colind[k]];
}

__global__ __launch_bounds__(kSpmmThreads) void entry_finish_kernel(const int32_t *__restrict__ cls_sorted,
                                                                    const int32_t *__restrict__ row_sorted,
                                                                    const int32_t *__restrict__ pos, int64_t nnz,
                                                                    int32_t rows, const int32_t *__restrict__ colind,
                                                                    const float *__restrict__ val,
                                                                    int32_t *__restrict__ vrow,
                                                                    int32_t *__restrict__ colind2,
                                                                    float *__restrict__ val2) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < nnz) {
    const int32_t p = pos[k];
    vrow[k] = cls_sorted[k] * rows + row_sorted[k];
    colind2[k] = colind[p];
    val2[k] = val[p];
  }
}

__global__ __launch_bounds__(kSpmmThreads) void hub_iota_kernel(int32_t *__restrict__ out, int64_t count) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < count) out[k] = (int32_t)k;
}

__global__ __launch_bounds__(kSpmmThreads) void csr_rows_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                int32_t *__restrict__ row_out) {
  const int64_t wave = ((int64_t)blockIdx.x * kSpmmThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (wave >= n) return;
  const int32_t s = rowptr[wave], e = rowptr[wave + 1];
  for (int32_t k = s + lane; k < e; k += kWave) row_out[k] = (int32_t)wave;
}

static int build_hub(CsrSide &s, int32_t hot, int32_t groups, int32_t tiers, int32_t seg, hipStream_t stream) {
  HubPlan &h = s.hub;
  CG_HIP(hipStreamSynchronize(stream));
  h.release();
  const int64_t nnz = s.nnz;
  const int32_t n = s.rows, m = s.cols;
  const int32_t nclass = groups * tiers;
  const int64_t vrows = (int64_t)(nclass + 1) * n;
  if (hot < 1) hot = 1;
  if (vrows + 1 > 0x7fffffffLL) CG_FAIL(CG_ERR_OVERFLOW, "hub plan: %lld virtual rows exceed int32", (long long)vrows);
  TempFree tmp;
  const unsigned gm = (unsigned)ceil_div64(m, kSpmmThreads), ge = (unsigned)ceil_div64(nnz, kSpmmThreads);

  // 1. reference count of every column, and the columns ranked by it
  uint32_t *count = nullptr;
  int32_t *cls = nullptr;
  CG_TRY(tmp.alloc((void **)&count, (size_t)m * 4));
  CG_TRY(tmp.alloc((void **)&cls, (size_t)m * 4));
  CG_HIP(hipMemsetAsync(count, 0, (size_t)m * 4, stream));
  col_count_kernel<<<ge, kSpmmThreads, 0, stream>>>(s.colind, nnz, count);
  CG_LAUNCH_CHECK();
  {
    SortBuffers buf;
    for (int i = 0; i < 2; ++i) {
      CG_TRY(tmp.alloc((void **)&buf.key_a[i], (size_t)m * 4));
      CG_TRY(tmp.alloc((void **)&buf.payload[i], (size_t)m * 4));
      CG_TRY(tmp.alloc((void **)&buf.key_b[i], (size_t)m * 4));  // no minor key: carried, never sorted on
    }
    // the largest possible count is the number of rows (duplicate-free) or nnz in general
    const uint32_t maxcount = (uint32_t)(nnz < 0x7fffffffLL ? nnz : 0x7fffffffLL);
    col_key_kernel<<<gm, kSpmmThreads, 0, stream>>>(count, m, maxcount, buf.key_a[0], buf.payload[0]);
    CG_LAUNCH_CHECK();
    CG_HIP(hipMemsetAsync(buf.key_b[0], 0, (size_t)m * 4, stream));
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, m, bits_for((int32_t)(maxcount < 0x7ffffffeu ? maxcount + 1 : 0x7fffffff)), 0, &set,
                            stream));
    col_class_kernel<<<gm, kSpmmThreads, 0, stream>>>(buf.payload[set], m, hot, groups, tiers, cls);
    CG_LAUNCH_CHECK();
  }

  // 2. stable regrouping of the entries by class: (row, col) order is kept inside a class
  CG_TRY(dev_alloc((void **)&h.colind, (size_t)nnz * 4));
  CG_TRY(dev_alloc((void **)&h.val, (size_t)nnz * 4));
  CG_TRY(dev_alloc((void **)&h.vrowptr, (size_t)(vrows + 1) * 4));
  int32_t *vrow = nullptr;
  CG_TRY(tmp.alloc((void **)&vrow, (size_t)nnz * 4));
  {
    TempFree tmp2;
    SortBuffers buf;
    for (int i = 0; i < 2; ++i) {
      CG_TRY(tmp2.alloc((void **)&buf.key_a[i], (size_t)nnz * 4));
      CG_TRY(tmp2.alloc((void **)&buf.key_b[i], (size_t)nnz * 4));
      CG_TRY(tmp2.alloc((void **)&buf.payload[i], (size_t)nnz * 4));
    }
    entry_class_kernel<<<ge, kSpmmThreads, 0, stream>>>(s.colind, nnz, cls, buf.key_a[0]);
    CG_LAUNCH_CHECK();
    if (n > 0) {
      csr_rows_kernel<<<(unsigned)ceil_div64((int64_t)n * kWave, kSpmmThreads), kSpmmThreads, 0, stream>>>(
          s.rowptr, n, buf.key_b[0]);
      CG_LAUNCH_CHECK();
    }
    hub_iota_kernel<<<ge, kSpmmThreads, 0, stream>>>(buf.payload[0], nnz);  // position in the original CSR
    CG_LAUNCH_CHECK();
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, nnz, bits_for(nclass + 1), 0, &set, stream));
    entry_finish_kernel<<<ge, kSpmmThreads, 0, stream>>>(buf.key_a[set], buf.key_b[set], buf.payload[set], nnz, n,
                                                         s.colind, s.val, vrow, h.colind, h.val);
    CG_LAUNCH_CHECK();
    CG_HIP(hipStreamSynchronize(stream));
  }
  CG_TRY(launch_rowptr(vrow, nnz, (int32_t)vrows, h.vrowptr, stream));

  // 3. tasks of the hot classes (empty virtual rows get none); the cold class is scheduled on demand
  CG_TRY(make_sched(h.vrowptr, nclass * n, seg, 1, h.hot_sched, stream));
  {
    int32_t t[18];
    for (int g = 0; g <= nclass; ++g)
      CG_HIP(hipMemcpyAsync(&t[g], h.hot_sched.tbase + (int64_t)g * n, 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipStreamSynchronize(stream));
    for (int g = 0; g <= nclass; ++g) h.tstart[g] = t[g];
  }
  h.hot = hot;
  h.groups = groups;
  h.tiers = tiers;
  h.seg = seg;
  h.valid = true;
  return CG_OK;
}

// C[r, :] += sum of the partial rows of r's hot tasks, in (group, segment) order.  One wavefront
// per row: lane g fetches the task range of group g, then the lanes sweep the row's columns with
// the partial rows of all tasks in flight together.
template <int NC>  // classes the unrolled loops cover (nclass <= NC)
__global__ __launch_bounds__(kSpmmThreads) void hub_reduce_kernel(const int32_t *__restrict__ tbase, int32_t n,
                                                                  int32_t nclass, const float *__restrict__ P,
                                                                  float *__restrict__ C, int64_t ldc, int32_t f) {
  const int64_t r = ((int64_t)blockIdx.x * kSpmmThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (r >= n) return;
  int32_t t0 = 0, t1 = 0;
  if (lane < nclass) {
    const int64_t v = (int64_t)lane * n + r;
    t0 = tbase[v];
    t1 = tbase[v + 1];
  }
  int32_t first[NC], count[NC];
  int32_t total = 0;
#pragma unroll
  for (int g = 0; g < NC; ++g) {
    first[g] = __builtin_amdgcn_readlane(t0, g);
    count[g] = __builtin_amdgcn_readlane(t1, g) - first[g];
    total += count[g];
  }
  if (total == 0) return;
  float *crow = C + r * ldc;
  for (int32_t c0 = 0; c0 < f; c0 += kWave) {
    const int32_t col = c0 + lane;
    if (col < f) {
      float s = 0.f;
#pragma unroll
      for (int g = 0; g < NC; ++g) {
        const float *p = P + (int64_t)first[g] * f + col;
        if (count[g] == 1) {
          s += p[0];
        } else {
          for (int32_t t = 0; t < count[g]; ++t) s += p[(int64_t)t * f];
        }
      }
      crow[col] += s;
    }
  }
}

std::atomic<int> g_tune_hub{0}, g_tune_hub_kb{0}, g_tune_hub_groups{0}, g_tune_hub_tiers{0};

// stored entries after which a new window starts
static int32_t window_entries() {
  const int w = g_tune_win.load(std::memory_order_relaxed);
  return w >= 64 ? w : 512;
}

static void fill_args(SpmmArgs &a, const int32_t *rowptr, const int32_t *colind, const float *val, const Sched *sc,
                      int32_t cols, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta,
                      const SpmmPlan &plan) {
  a.rowptr = rowptr;
  a.colind = colind;
  a.val = val;
  a.task_row = sc->task_row;
  a.tbase = sc->tbase;
  a.pbase = sc->pbase;
  a.ntasks = sc->ntasks;
  a.seg = sc->seg;
  a.m = cols;
  a.B = B;
  a.ldb = ldb;
  a.C = C;
  a.ldc = ldc;
  a.f = f;
  a.beta = beta;
  a.tiles = plan.tiles;
  a.tile_slots = plan.tile_slots;
  a.groups = 1;
  a.P = nullptr;
}

// Plain handle path for one column range: row-segment tasks over (rowptr, colind, val).
static int spmm_plain(const int32_t *rowptr, const int32_t *colind, const float *val, int32_t rows, int32_t cols,
                      SchedCache &cache, int vec, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f,
                      float beta, int prof_tag, hipStream_t stream) {
  SpmmPlan plan = plan_range(vec, f);
  if (plan.shape.chunks > kMaxChunks) {  // tiling was tuned down: fall back to 8 tiles
    plan.tiles = 8;
    plan.tile_slots = (f / vec + 7) / 8;
    plan.shape = pick_shape(vec, plan.tile_slots);
  }
  Sched *sc = nullptr;
  CG_TRY(cache.get(rowptr, rows, pick_seg(plan.shape), &sc, stream));
  SpmmArgs a{};
  fill_args(a, rowptr, colind, val, sc, cols, B, ldb, C, ldc, f, beta, plan);
  if (sc->nslots > 0) {
    void *p = nullptr;
    CG_TRY(scratch_get(stream, kSlotA, (size_t)sc->nslots * f * sizeof(float), &p));
    a.P = (float *)p;
  }
  const bool narrow = plan.shape.lpr < kWave;
  if (plan.tiles == 1 && g_tune_stream.load(std::memory_order_relaxed) >= 0 &&
      (!narrow || (sc->seg <= 512 && window_entries() <= 512))) {
    // stream windows of consecutive tasks
    StreamTab &tab = cache.tab_of(sc);
    const int32_t S = window_entries();
    if (tab.S != S) {
      const int64_t first[2] = {0, sc->ntasks};
      CG_TRY(build_stream(*sc, rowptr, rows, false, 1, first, S, tab, stream));
    }
    StreamArgs sa{};
    sa.task_start = tab.task_start;
    sa.task_dst = tab.task_dst;
    sa.wstart = tab.wstart;
    sa.colind = colind;
    sa.val = val;
    sa.win_first[0] = 0;
    sa.win_first[1] = tab.nwin;
    sa.groups = 1;
    sa.B = B;
    sa.ldb = ldb;
    sa.C = C;
    sa.ldc = ldc;
    sa.P = a.P;
    sa.f = f;
    sa.beta = beta;
    ProfScope prof("spmm_rowseg", prof_tag, stream);
    if (narrow) CG_TRY(launch_stream_narrow(vec, plan.shape.lpr, sa, stream));
    else CG_TRY(launch_stream_wide(vec, plan.shape.chunks, sa, stream));
  } else {
    ProfScope prof("spmm_rowseg", prof_tag, stream);
    CG_TRY((launch_shape<kModeTable>(plan.shape, a, stream)));
  }
  if (sc->nmulti > 0) {
    ProfScope prof("spmm_reduce", prof_tag, stream);
    const int64_t threads = sc->nmulti * (int64_t)f;
    spmm_reduce_kernel<<<(unsigned)ceil_div64(threads, kSpmmThreads), kSpmmThreads, 0, stream>>>(
        sc->multi_rows, sc->nmulti, rowptr, sc->pbase, sc->seg, a.P, C, ldc, f, beta);
    CG_LAUNCH_CHECK();
  }
  return CG_OK;
}

// Should a product of this width over this matrix go through a hub plan?  It pays when a row of B
// is many cache lines (the gather dominates) and rows hold enough hot entries per group that the
// partial rows they cost are small against the gathers they turn into L2 hits.
static bool want_hub(const CsrSide &s, int32_t f) {
  const int t = g_tune_hub.load(std::memory_order_relaxed);
  if (t < 0) return false;
  if (s.rows == 0 || s.nnz == 0) return false;
  if (t > 0) return true;
  return f >= 128 && s.nnz / s.rows >= 128;
}

static int spmm_hub(CsrSide &s, int vec, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta,
                    hipStream_t stream) {
  int groups = g_tune_hub_groups.load(std::memory_order_relaxed);
  if (groups != 1 && groups != 2 && groups != 4 && groups != 8) groups = 8;
  int tiers = g_tune_hub_tiers.load(std::memory_order_relaxed);
  if (tiers < 1 || tiers * groups > 16) tiers = 1;
  int kb = g_tune_hub_kb.load(std::memory_order_relaxed);
  // one tier: twice the 4 MB L2 of an XCD is the measured optimum (LRU keeps the hottest half);
  // several tiers: each is sized to stay resident
  if (kb <= 0) kb = tiers == 1 ? 8192 : 3584;
  int64_t per_group = (int64_t)kb * 1024 / ((int64_t)f * 4);
  if (per_group < 1) per_group = 1;
  int64_t hot = per_group * groups;  // columns per tier
  if (hot > s.cols) hot = s.cols;
  // hot tasks use full-wave teams on the whole width with one dword per lane and chunk when the rows
  // are not 16-byte aligned: that is the fastest gather of L2-resident rows
  const int hot_vec = (vec == 4 || f / vec <= kWave) ? vec : 1;
  SpmmPlan hplan;
  hplan.tiles = 1;
  hplan.tile_slots = f / hot_vec;
  hplan.shape = pick_shape(hot_vec, hplan.tile_slots);
  const int32_t seg = pick_seg(hplan.shape);
  if (!s.hub.valid || s.hub.hot != (int32_t)hot || s.hub.groups != groups || s.hub.tiers != tiers || s.hub.seg != seg)
    CG_TRY(build_hub(s, (int32_t)hot, groups, tiers, seg, stream));
  HubPlan &h = s.hub;
  const int32_t n = s.rows;
  const int32_t nclass = h.classes();
  // 1. cold class straight into C
  CG_TRY(spmm_plain(h.vrowptr + (int64_t)nclass * n, h.colind, h.val, n, s.cols, h.cold_sched, vec, B, ldb, C, ldc, f,
                    beta, f, stream));
  // 2. hot classes, one launch per tier: every task writes a partial row
  const int64_t hot_tasks = h.hot_sched.ntasks;
  if (hot_tasks == 0) return CG_OK;
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotC, (size_t)hot_tasks * f * sizeof(float), &p));
  const bool hnarrow = hplan.shape.lpr < kWave;
  const bool streaming =
      g_tune_stream.load(std::memory_order_relaxed) >= 0 && (!hnarrow || (seg <= 512 && window_entries() <= 512));
  if (streaming) {
    const int32_t S = window_entries();
    if (h.hot_tab.S != S || h.hot_tab.groups != nclass)
      CG_TRY(build_stream(h.hot_sched, h.vrowptr, nclass * n, true, nclass, h.tstart, S, h.hot_tab, stream));
  }
  for (int t = 0; t < tiers; ++t) {
    ProfScope prof("spmm_hub_hot", f, stream);
    if (streaming) {
      StreamArgs sa{};
      sa.task_start = h.hot_tab.task_start;
      sa.task_dst = h.hot_tab.task_dst;
      sa.wstart = h.hot_tab.wstart;
      sa.colind = h.colind;
      sa.val = h.val;
      for (int g = 0; g <= groups; ++g) sa.win_first[g] = h.hot_tab.win_first[t * groups + g];
      sa.groups = groups;
      sa.B = B;
      sa.ldb = ldb;
      sa.C = C;
      sa.ldc = ldc;
      sa.P = (float *)p;
      sa.f = f;
      sa.beta = 0.f;
      if (hnarrow) CG_TRY(launch_stream_narrow(hot_vec, hplan.shape.lpr, sa, stream));
      else CG_TRY(launch_stream_wide(hot_vec, hplan.shape.chunks, sa, stream));
    } else {
      SpmmArgs a{};
      fill_args(a, h.vrowptr, h.colind, h.val, &h.hot_sched, s.cols, B, ldb, C, ldc, f, 0.f, hplan);
      a.P = (float *)p;
      a.groups = groups;
      for (int g = 0; g <= groups; ++g) a.tstart[g] = h.tstart[t * groups + g];
      CG_TRY((launch_shape<kModeHub>(hplan.shape, a, stream)));
    }
  }
  // 3. fold the partial rows into C
  {
    ProfScope prof("spmm_hub_reduce", f, stream);
    const unsigned rgrid = (unsigned)ceil_div64((int64_t)n * kWave, kSpmmThreads);
    if (nclass <= 8)
      hub_reduce_kernel<8><<<rgrid, kSpmmThreads, 0, stream>>>(h.hot_sched.tbase, n, nclass, (const float *)p, C, ldc, f);
    else
      hub_reduce_kernel<16><<<rgrid, kSpmmThreads, 0, stream>>>(h.hot_sched.tbase, n, nclass, (const float *)p, C, ldc, f);
    CG_LAUNCH_CHECK();
  }
  return CG_OK;
}

static int spmm_side(CsrSide &s, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta,
                     hipStream_t stream) {
  if (s.rows == 0) return CG_OK;
  const int vec = pick_vec(f, B, ldb, C, ldc);
  const int32_t cap = range_cap(vec) * 8;  // 8 tiles of kMaxChunks chunks
  if (f <= range_cap(vec == 4 ? 4 : 1) && want_hub(s, f)) return spmm_hub(s, vec, B, ldb, C, ldc, f, beta, stream);
  for (int32_t f0 = 0; f0 < f; f0 += cap) {
    const int32_t ft = f - f0 < cap ? f - f0 : cap;
    CG_TRY(spmm_plain(s.rowptr, s.colind, s.val, s.rows, s.cols, s.sched, vec, B + f0, ldb, C + f0, ldc, ft, beta, f,
                      stream));
  }
  return CG_OK;
}

}  // namespace cg

namespace cg {
extern std::atomic<int> g_tune_dense_mfma;  // dense.hip
}

struct cg_csr {
  int device = 0;
  int32_t n = 0, m = 0;
  int64_t nnz = 0;
  bool has_t = false;
  cg::CsrSide fwd, tr;
};

namespace cg {
static int side_alloc(CsrSide &s, int32_t rows, int32_t cols, int64_t nnz) {
  s.rows = rows;
  s.cols = cols;
  s.nnz = nnz;
  CG_TRY(dev_alloc((void **)&s.rowptr, (size_t)(rows + 1) * sizeof(int32_t)));
  CG_TRY(dev_alloc((void **)&s.colind, (size_t)nnz * sizeof(int32_t)));
  CG_TRY(dev_alloc((void **)&s.val, (size_t)nnz * sizeof(float)));
  return CG_OK;
}

static int side_max_degree(CsrSide &s, hipStream_t stream) {
  void *d = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, sizeof(int), &d));
  CG_HIP(hipMemsetAsync(d, 0, sizeof(int), stream));
  if (s.rows > 0) {
    max_degree_kernel<<<(unsigned)ceil_div64(s.rows, kSpmmThreads), kSpmmThreads, 0, stream>>>(s.rowptr, s.rows,
                                                                                              (int *)d);
    CG_LAUNCH_CHECK();
  }
  int v = 0;
  CG_HIP(hipMemcpyAsync(&v, d, sizeof(int), hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  s.max_degree = v;
  return CG_OK;
}

static int csr_create(cg_csr *h, const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz,
                      int32_t n, int32_t m, uint32_t flags, hipStream_t stream) {
  h->n = n;
  h->m = m;
  h->nnz = nnz;
  CG_HIP(hipGetDevice(&h->device));
  // index ranges are always checked here: the SpMM kernels of a handle trust them
  CG_TRY(coo_check(d_row, d_col, nnz, n, m, (flags & CG_CSR_SORTED) ? ((flags & CG_CSR_VALIDATE) ? 2 : 1) : 0, stream));
  CG_TRY(side_alloc(h->fwd, n, m, nnz));
  if (flags & CG_CSR_SORTED) {
    CG_TRY(launch_rowptr(d_row, nnz, n, h->fwd.rowptr, stream));
    if (nnz > 0) {
      CG_HIP(hipMemcpyAsync(h->fwd.colind, d_col, (size_t)nnz * sizeof(int32_t), hipMemcpyDeviceToDevice, stream));
      CG_HIP(hipMemcpyAsync(h->fwd.val, d_val, (size_t)nnz * sizeof(float), hipMemcpyDeviceToDevice, stream));
    }
  } else {
    CG_TRY(coo2csr_general(d_row, d_col, d_val, nnz, n, m, h->fwd.rowptr, h->fwd.colind, h->fwd.val, nullptr, stream));
  }
  CG_TRY(side_max_degree(h->fwd, stream));
  if (flags & CG_CSR_TRANSPOSE) {
    CG_TRY(side_alloc(h->tr, m, n, nnz));
    CG_TRY(csr_transpose(h->fwd.rowptr, h->fwd.colind, h->fwd.val, nnz, n, m, h->tr.rowptr, h->tr.colind, h->tr.val,
                         nullptr, stream));
    CG_TRY(side_max_degree(h->tr, stream));
    h->has_t = true;
  }
  CG_HIP(hipStreamSynchronize(stream));
  return CG_OK;
}
}  // namespace cg

extern "C" {

int cg_spmm_coo(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n, int32_t m,
                const float *d_B, int64_t ldb, float *d_C, int64_t ldc, int32_t f, float beta, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  if (nnz < 0 || n < 0 || m < 0) CG_FAIL(CG_ERR_SIZE, "cg_spmm_coo: negative size");
  if (nnz > 0x7fffffffLL - 1 || n == 0x7fffffff) CG_FAIL(CG_ERR_OVERFLOW, "cg_spmm_coo: nnz=%lld n=%d exceed int32", (long long)nnz, n);
  if (nnz > 0 && (!d_row || !d_col || !d_val)) CG_FAIL(CG_ERR_NULL, "cg_spmm_coo: null sparse operand");
  CG_TRY(check_dense("cg_spmm_coo", d_B, ldb, d_C, ldc, f, m, n));
  if (n == 0) return CG_OK;
  if (nnz > 0 && m == 0) CG_FAIL(CG_ERR_SIZE, "cg_spmm_coo: nnz > 0 with m == 0");
  void *d_rowptr = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, (size_t)(n + 1) * sizeof(int32_t), &d_rowptr));
  // rows the compression never reaches (only possible for unsorted input) stay 0 -> empty or
  // in-range spans, never an out-of-bounds read
  CG_HIP(hipMemsetAsync(d_rowptr, 0, (size_t)(n + 1) * sizeof(int32_t), stream));
  CG_TRY(launch_rowptr(d_row, nnz, n, (int32_t *)d_rowptr, stream));
  const int vec = pick_vec(f, d_B, ldb, d_C, ldc);
  const int32_t cap = range_cap(vec);
  for (int32_t f0 = 0; f0 < f; f0 += cap) {
    const int32_t ft = f - f0 < cap ? f - f0 : cap;
    SpmmArgs a{};
    a.rowptr = (const int32_t *)d_rowptr;
    a.colind = d_col;
    a.val = d_val;
    a.ntasks = n;
    a.seg = 0;
    a.m = m;
    a.B = d_B + f0;
    a.ldb = ldb;
    a.C = d_C + f0;
    a.ldc = ldc;
    a.f = ft;
    a.beta = beta;
    a.tiles = 1;
    a.tile_slots = ft / vec;
    CG_TRY((launch_shape<kModeRows>(pick_shape(vec, ft / vec), a, stream)));
  }
  return CG_OK;
}

int cg_csr_create(cg_csr_t **out, const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz,
                  int32_t n, int32_t m, uint32_t flags, cg_stream_t stream) {
  using namespace cg;
  if (!out) CG_FAIL(CG_ERR_NULL, "cg_csr_create: out is NULL");
  *out = nullptr;
  if (nnz < 0 || n < 0 || m < 0) CG_FAIL(CG_ERR_SIZE, "cg_csr_create: negative size");
  if (nnz > 0x7fffffffLL - 1 || n == 0x7fffffff || m == 0x7fffffff)
    CG_FAIL(CG_ERR_OVERFLOW, "cg_csr_create: nnz=%lld n=%d m=%d exceed the int32 index contract", (long long)nnz, n, m);
  if (nnz > 0 && (!d_row || !d_col || !d_val)) CG_FAIL(CG_ERR_NULL, "cg_csr_create: null sparse operand");
  if (nnz > 0 && (n == 0 || m == 0)) CG_FAIL(CG_ERR_SIZE, "cg_csr_create: nnz > 0 in an empty matrix");
  cg_csr *h = new (std::nothrow) cg_csr();
  if (!h) CG_FAIL(CG_ERR_ALLOC, "cg_csr_create: host allocation failed");
  int st = csr_create(h, d_row, d_col, d_val, nnz, n, m, flags, (hipStream_t)stream);
  if (st != CG_OK) {
    h->fwd.release();
    h->tr.release();
    delete h;
    return st;
  }
  *out = h;
  return CG_OK;
}

int cg_csr_destroy(cg_csr_t *h) {
  if (!h) return CG_OK;
  (void)hipDeviceSynchronize();
  h->fwd.release();
  h->tr.release();
  delete h;
  return CG_OK;
}

int cg_csr_spmm(cg_csr_t *h, int transpose, const float *d_B, int64_t ldb, float *d_C, int64_t ldc, int32_t f,
                float beta, cg_stream_t stream) {
  using namespace cg;
  if (!h) CG_FAIL(CG_ERR_NULL, "cg_csr_spmm: handle is NULL");
  if (transpose && !h->has_t) CG_FAIL(CG_ERR_NO_TRANSPOSE, "cg_csr_spmm: handle was built without CG_CSR_TRANSPOSE");
  CsrSide &s = transpose ? h->tr : h->fwd;
  CG_TRY(check_dense("cg_csr_spmm", d_B, ldb, d_C, ldc, f, s.cols, s.rows));
  return spmm_side(s, d_B, ldb, d_C, ldc, f, beta, (hipStream_t)stream);
}

int cg_tune_set(const char *key, int value) {
  if (!key) CG_FAIL(CG_ERR_NULL, "cg_tune_set: key is NULL");
  if (!strcmp(key, "spmm_seg")) cg::g_tune_seg.store(value);
  else if (!strcmp(key, "spmm_tiles")) cg::g_tune_tiles.store(value);
  else if (!strcmp(key, "spmm_vec")) cg::g_tune_vec.store(value);
  else if (!strcmp(key, "spmm_hub")) cg::g_tune_hub.store(value);
  else if (!strcmp(key, "spmm_stream")) cg::g_tune_stream.store(value);
  else if (!strcmp(key, "dense_mfma")) cg::g_tune_dense_mfma.store(value);
  else if (!strcmp(key, "spmm_win")) cg::g_tune_win.store(value);
  else if (!strcmp(key, "spmm_hub_kb")) cg::g_tune_hub_kb.store(value);
  else if (!strcmp(key, "spmm_hub_groups")) cg::g_tune_hub_groups.store(value);
  else if (!strcmp(key, "spmm_hub_tiers")) cg::g_tune_hub_tiers.store(value);
  else CG_FAIL(CG_ERR_UNSUPPORTED, "cg_tune_set: unknown key %s", key);
  return CG_OK;
}

int cg_csr_info(const cg_csr_t *h, int64_t info[8]) {
  if (!h || !info) CG_FAIL(CG_ERR_NULL, "cg_csr_info: null pointer");
  info[0] = h->n;
  info[1] = h->m;
  info[2] = h->nnz;
  info[3] = h->has_t ? 1 : 0;
  info[4] = h->fwd.max_degree;
  info[5] = h->has_t ? h->tr.max_degree : -1;
  info[6] = 0;
  info[7] = 0;
  return CG_OK;
}

int cg_csr_arrays(const cg_csr_t *h, int transpose, const int32_t **d_rowptr, const int32_t **d_colind,
                  const float **d_values) {
  if (!h) CG_FAIL(CG_ERR_NULL, "cg_csr_arrays: handle is NULL");
  if (transpose && !h->has_t) CG_FAIL(CG_ERR_NO_TRANSPOSE, "cg_csr_arrays: handle was built without CG_CSR_TRANSPOSE");
  const cg::CsrSide &s = transpose ? h->tr : h->fwd;
  if (d_rowptr) *d_rowptr = s.rowptr;
  if (d_colind) *d_colind = s.colind;
  if (d_values) *d_values = s.val;
  return CG_OK;
}

}  // extern "C"
