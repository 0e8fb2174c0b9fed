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
};

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

template <int VEC, int LPR, int CHUNKS, bool TABLE, bool CLAMP>
__global__ __launch_bounds__(kSpmmThreads) void spmm_rowseg_kernel(const SpmmArgs a) {
  static_assert(LPR == 64 || CHUNKS == 1, "several chunks only with a full-wave team");
  constexpr int G = kWave / LPR;
  const int lane = threadIdx.x & (kWave - 1);
  // Workgroups are dealt to the 8 XCDs round robin (workgroup w runs on XCD w % 8), and every XCD
  // has its own L2.  With T feature tiles, XCD x only ever touches tile x % T of B, so its L2 holds
  // a T times narrower slice of B's hot rows: the 8 L2s cache different data instead of 8 copies.
  int tile = 0;
  int64_t tb = blockIdx.x;
  if (a.tiles > 1) {
    const int x = blockIdx.x & 7;
    const int per = 8 / a.tiles;  // XCDs that share a tile
    tile = x % a.tiles;
    tb = (int64_t)(blockIdx.x >> 3) * per + x / a.tiles;
  }
  const int64_t task = __builtin_amdgcn_readfirstlane((int)(tb * kWavesPerBlock + threadIdx.x / kWave));
  if (task >= a.ntasks) return;

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
  const bool single = TABLE ? (re - rs <= a.seg) : true;
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
    float *prow = a.P + ((int64_t)a.pbase[row] + sidx) * a.f;
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

constexpr int kMaxChunks = 5;

// Widest vector the operands allow.
static int pick_vec(int32_t f, const float *B, int64_t ldb, const float *C, int64_t ldc) {
  const uintptr_t bits = (uintptr_t)B | (uintptr_t)C;
  if (f % 4 == 0 && ldb % 4 == 0 && ldc % 4 == 0 && bits % 16 == 0) return 4;
  if (f % 2 == 0 && ldb % 2 == 0 && ldc % 2 == 0 && bits % 8 == 0) return 2;
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

// Tuning knobs (cg_tune_set): 0 = built-in choice.
std::atomic<int> g_tune_seg{0}, g_tune_tiles{0};

// Feature tiles per launch.  Wide outputs are split over the XCDs so that each L2 caches its own
// column slice of B; narrow ones (a row of B is a cache line or two) stay whole.
static int pick_tiles(int vec, int slots) {
  const int t = g_tune_tiles.load(std::memory_order_relaxed);
  if (t == 1 || t == 2 || t == 4 || t == 8) return slots >= t ? t : 1;
  (void)vec;
  return slots >= 256 ? 8 : 1;
}

template <bool TABLE, bool CLAMP>
static int launch_shape(const SpmmShape &s, const SpmmArgs &a, hipStream_t stream) {
  int64_t blocks = ceil_div64(a.ntasks, kWavesPerBlock);
  if (a.tiles > 1) blocks = ceil_div64(blocks, 8 / a.tiles) * 8;
  if (blocks > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "SpMM grid too large");
  const unsigned grid = (unsigned)blocks;
  if (grid == 0) return CG_OK;
#define CG_CASE(V, L, CH)                                                                          \
  if (s.vec == V && s.lpr == L && s.chunks == CH) {                                                \
    spmm_rowseg_kernel<V, L, CH, TABLE, CLAMP><<<grid, kSpmmThreads, 0, stream>>>(a);              \
    CG_LAUNCH_CHECK();                                                                             \
    return CG_OK;                                                                                  \
  }
#define CG_CASES(V)                                                                                \
  CG_CASE(V, 4, 1) CG_CASE(V, 8, 1) CG_CASE(V, 16, 1) CG_CASE(V, 32, 1) CG_CASE(V, 64, 1)           \
  CG_CASE(V, 64, 2) CG_CASE(V, 64, 3) CG_CASE(V, 64, 4) CG_CASE(V, 64, 5)
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
__global__ __launch_bounds__(kSpmmThreads) void sched_count_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                   int32_t seg, uint32_t *__restrict__ ntask,
                                                                   uint32_t *__restrict__ nslot,
                                                                   uint32_t *__restrict__ nmulti) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r >= n) return;
  const int32_t deg = rowptr[r + 1] - rowptr[r];
  const uint32_t t = deg <= seg ? 1u : (uint32_t)((deg + seg - 1) / seg);
  ntask[r] = t;
  nslot[r] = t > 1 ? t : 0u;
  nmulti[r] = t > 1 ? 1u : 0u;
}

__global__ __launch_bounds__(kSpmmThreads) void sched_fill_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                  int32_t seg, const uint32_t *__restrict__ tbase,
                                                                  const uint32_t *__restrict__ mbase,
                                                                  int32_t *__restrict__ task_row,
                                                                  int32_t *__restrict__ multi_rows) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r >= n) return;
  const int32_t deg = rowptr[r + 1] - rowptr[r];
  const uint32_t t = deg <= seg ? 1u : (uint32_t)((deg + seg - 1) / seg);
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

struct CsrSide {
  int32_t rows = 0, cols = 0;
  int32_t *rowptr = nullptr, *colind = nullptr;
  float *val = nullptr;
  int32_t max_degree = 0;
  static constexpr int kMaxSched = 4;
  Sched sched[kMaxSched];
  int nsched = 0;
  void release() {
    for (int i = 0; i < nsched; ++i) sched[i].release();
    nsched = 0;
    if (rowptr) (void)hipFree(rowptr);
    if (colind) (void)hipFree(colind);
    if (val) (void)hipFree(val);
    rowptr = colind = nullptr;
    val = nullptr;
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

static int build_sched(CsrSide &s, int32_t seg, Sched **out, hipStream_t stream) {
  for (int i = 0; i < s.nsched; ++i)
    if (s.sched[i].seg == seg) {
      *out = &s.sched[i];
      return CG_OK;
    }
  if (s.nsched == CsrSide::kMaxSched) {  // recycle the oldest
    CG_HIP(hipStreamSynchronize(stream));
    s.sched[0].release();
    for (int i = 1; i < s.nsched; ++i) s.sched[i - 1] = s.sched[i];
    s.sched[--s.nsched] = Sched();
  }
  Sched sc;
  sc.seg = seg;
  const int32_t n = s.rows;
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
      sched_count_kernel<<<grid, kSpmmThreads, 0, stream>>>(s.rowptr, n, seg, (uint32_t *)sc.tbase,
                                                            (uint32_t *)sc.pbase, d_mbase);
      if (hipGetLastError() != hipSuccess) { st = CG_ERR_HIP; set_error("sched_count launch failed"); break; }
      if ((st = exclusive_scan_u32((uint32_t *)sc.tbase, (uint32_t *)sc.tbase, n, d_totals + 0, stream)) != CG_OK) break;
      if ((st = exclusive_scan_u32((uint32_t *)sc.pbase, (uint32_t *)sc.pbase, n, d_totals + 1, stream)) != CG_OK) break;
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
      sched_fill_kernel<<<grid, kSpmmThreads, 0, stream>>>(s.rowptr, n, seg, (const uint32_t *)sc.tbase, d_mbase,
                                                           sc.task_row, sc.multi_rows);
      if (hipGetLastError() != hipSuccess) { st = CG_ERR_HIP; set_error("sched_fill launch failed"); break; }
      if (hipStreamSynchronize(stream) != hipSuccess) { st = CG_ERR_HIP; set_error("sched_fill failed"); break; }
    }
  } while (0);
  if (d_mbase) (void)hipFree(d_mbase);
  if (st != CG_OK) {
    sc.release();
    return st;
  }
  s.sched[s.nsched] = sc;
  *out = &s.sched[s.nsched++];
  return CG_OK;
}

// Entries per task.  A team step consumes G entries per wave instruction, so narrow outputs get
// longer segments for the same number of steps.
static int32_t pick_seg(const SpmmShape &s) {
  const int t = g_tune_seg.load(std::memory_order_relaxed);
  if (t >= 64) return t;
  const int g = kWave / s.lpr;
  if (g == 1) return 1024;
  if (g == 2) return 2048;
  return 4096;
}

static int spmm_side(CsrSide &s, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta,
                     hipStream_t stream) {
  if (s.rows == 0) return CG_OK;
  const int vec = pick_vec(f, B, ldb, C, ldc);
  const int32_t cap = range_cap(vec) * 8;  // 8 tiles of kMaxChunks chunks
  for (int32_t f0 = 0; f0 < f; f0 += cap) {
    const int32_t ft = f - f0 < cap ? f - f0 : cap;
    const float *Bt = B + f0;
    float *Ct = C + f0;
    SpmmPlan plan = plan_range(vec, ft);
    if (plan.shape.chunks > kMaxChunks) {  // tiling was tuned down: fall back to 8 tiles
      plan.tiles = 8;
      plan.tile_slots = (ft / vec + 7) / 8;
      plan.shape = pick_shape(vec, plan.tile_slots);
    }
    const SpmmShape shape = plan.shape;
    Sched *sc = nullptr;
    CG_TRY(build_sched(s, pick_seg(shape), &sc, stream));
    SpmmArgs a{};
    a.rowptr = s.rowptr;
    a.colind = s.colind;
    a.val = s.val;
    a.task_row = sc->task_row;
    a.tbase = sc->tbase;
    a.pbase = sc->pbase;
    a.ntasks = sc->ntasks;
    a.seg = sc->seg;
    a.m = s.cols;
    a.B = Bt;
    a.ldb = ldb;
    a.C = Ct;
    a.ldc = ldc;
    a.f = ft;
    a.beta = beta;
    a.tiles = plan.tiles;
    a.tile_slots = plan.tile_slots;
    a.P = nullptr;
    if (sc->nslots > 0) {
      void *p = nullptr;
      CG_TRY(scratch_get(stream, kSlotA, (size_t)sc->nslots * ft * sizeof(float), &p));
      a.P = (float *)p;
    }
    {
      ProfScope prof("spmm_rowseg", f, stream);
      CG_TRY((launch_shape<true, false>(shape, a, stream)));
    }
    if (sc->nmulti > 0) {
      ProfScope prof("spmm_reduce", f, stream);
      const int64_t threads = sc->nmulti * (int64_t)ft;
      spmm_reduce_kernel<<<(unsigned)ceil_div64(threads, kSpmmThreads), kSpmmThreads, 0, stream>>>(
          sc->multi_rows, sc->nmulti, s.rowptr, sc->pbase, sc->seg, a.P, Ct, ldc, ft, beta);
      CG_LAUNCH_CHECK();
    }
  }
  return CG_OK;
}

}  // namespace cg

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
    CG_TRY((launch_shape<false, true>(pick_shape(vec, ft / vec), a, stream)));
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
