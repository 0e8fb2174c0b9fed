// Host side of the CSR SpMM: schedules, window tables, hub plans, the cached handle and the C ABI
// entry points.  The device kernels are in spmm_kernels.h.
//
// Replaces everything the reference wraps around cusparseSpMM on every call
// (sparse-extension/sparse_coo_tensor.cu:136-231): B and C stay row-major, nothing is transposed,
// and the CSR, its transpose, the schedules and the hub plan live in a handle.
#include "spmm_kernels.h"
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <memory>
#include <mutex>
#include <new>
#include <vector>

namespace cg {

extern std::atomic<int> g_tune_dense_mfma;  // dense.hip

// Tuning knobs (cg_tune_set): 0 = built-in choice.
static std::atomic<int> g_tune_seg{0}, g_tune_vec{0}, g_tune_win{0};
static std::atomic<int> g_tune_hub{0}, g_tune_hub_kb{0}, g_tune_hub_groups{0}, g_tune_hub_tiers{0}, g_tune_hub_row{0};
static std::atomic<int> g_tune_coo_cache{0};  // blocks cg_spmm_coo_cached keeps: 0 = 8, negative = none

// ---------------------------------------------------------------------------------------------
// kernel shape selection
// ---------------------------------------------------------------------------------------------
struct SpmmShape {
  int vec, lpr, chunks;
};

constexpr int kMaxHubClasses = 64;  // column classes of a hub plan (XCD groups x tiers)
constexpr int kHubAutoTiers = 6;    // most tiers the automatic choice takes
constexpr double kHubTierEntriesPerPair = 2.4;  // entries per (class, row) pair below which a tier no longer pays
constexpr double kHubMinHotFraction = 0.35;     // share of the entries the first tier must hold for a plan to pay
constexpr int kMaxChunks = 10;  // full-wave teams cover up to 64 * kMaxChunks * VEC columns per launch

// Widest vector the operands allow.
static int pick_vec(int32_t f, const float *B, int64_t ldb, const float *C, int64_t ldc) {
  const uintptr_t bits = (uintptr_t)B | (uintptr_t)C;
  const int cap = g_tune_vec.load(std::memory_order_relaxed);
  const int lim = (cap == 1 || cap == 2) ? cap : 4;
  if (lim >= 4 && f % 4 == 0 && ldb % 4 == 0 && ldc % 4 == 0 && bits % 16 == 0) return 4;
  if (lim >= 2 && f % 2 == 0 && ldb % 2 == 0 && ldc % 2 == 0 && bits % 8 == 0) return 2;
  return 1;
}

// Smallest team that covers `slots` vector slots.
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

static int32_t range_cap(int vec) { return kWave * kMaxChunks * vec; }

// Entries per task.  Narrow teams stage a window plus one task in LDS, so their tasks are shorter.
static int32_t pick_seg(const SpmmShape &s) {
  const int t = g_tune_seg.load(std::memory_order_relaxed);
  if (s.lpr == kWave) return t >= 64 ? t : 1024;
  return (t >= 64 && t <= 512) ? t : 512;
}

// Stored entries after which a new window starts.
static int32_t window_entries() {
  const int w = g_tune_win.load(std::memory_order_relaxed);
  return (w >= 64 && w <= 512) ? w : 512;
}

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
// device memory for tables: owned allocations (handles) or a bump arena over a scratch buffer
// (the one-shot entry point, which builds its tables anew on every call)
// ---------------------------------------------------------------------------------------------
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

struct Alloc {
  char *base = nullptr;  // arena mode when set
  size_t cap = 0, off = 0;
  bool arena() const { return base != nullptr; }
  int get(void **p, size_t bytes) {
    if (!base) return dev_alloc(p, bytes);
    const size_t need = (bytes + 255) & ~(size_t)255;
    if (off + need > cap) CG_FAIL(CG_ERR_ALLOC, "table arena too small (%zu + %zu > %zu)", off, need, cap);
    *p = base + off;
    off += need;
    return CG_OK;
  }
};

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

__global__ __launch_bounds__(kSpmmThreads) void fill_u32_kernel(uint32_t *__restrict__ p, int64_t count, uint32_t v) {
  const int64_t i = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (i < count) p[i] = v;
}

static int fill_u32(uint32_t *p, int64_t count, uint32_t v, hipStream_t stream) {
  if (count <= 0) return CG_OK;
  fill_u32_kernel<<<(unsigned)ceil_div64(count, kSpmmThreads), kSpmmThreads, 0, stream>>>(p, count, v);
  CG_LAUNCH_CHECK();
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
  if (r > n) return;
  if (r == n) {  // the scans run over n + 1 entries so that entry n receives the total
    ntask[r] = nslot[r] = nmulti[r] = 0u;
    return;
  }
  const uint32_t t = tasks_of(rowptr[r + 1] - rowptr[r], seg, skip_empty);
  ntask[r] = t;
  nslot[r] = t > 1 ? t : 0u;
  nmulti[r] = t > 1 ? 1u : 0u;
}

// max_tasks / max_multi: capacities of the output tables (a malformed, unsorted row array could
// otherwise describe more tasks than the arena of the one-shot entry point holds)
__global__ __launch_bounds__(kSpmmThreads) void sched_fill_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                  int32_t seg, int skip_empty,
                                                                  const uint32_t *__restrict__ tbase,
                                                                  const uint32_t *__restrict__ mbase,
                                                                  int32_t *__restrict__ task_row, int64_t max_tasks,
                                                                  int32_t *__restrict__ multi_rows,
                                                                  int64_t max_multi) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r >= n) return;
  const uint32_t t = tasks_of(rowptr[r + 1] - rowptr[r], seg, skip_empty);
  const uint32_t b = tbase[r];
  for (uint32_t i = 0; i < t; ++i)
    if ((int64_t)b + i < max_tasks) task_row[b + i] = (int32_t)r;
  if (t > 1 && (int64_t)mbase[r] < max_multi) multi_rows[mbase[r]] = (int32_t)r;
}

__global__ __launch_bounds__(kSpmmThreads) void max_degree_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                  int *__restrict__ out) {
  int32_t deg = 0;  // grid-stride: a few thousand atomics on the one word, not one per 64 rows
  for (int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x; r < n; r += (int64_t)gridDim.x * kSpmmThreads) {
    const int32_t d = rowptr[r + 1] - rowptr[r];
    deg = d > deg ? d : deg;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    int32_t o = __shfl_xor(deg, off, kWave);
    deg = o > deg ? o : deg;
  }
  if ((threadIdx.x & (kWave - 1)) == 0 && deg > 0) atomicMax(out, deg);  // integer max: order independent
}

struct Sched {
  int32_t seg = 0;
  bool owned = true;  // false: tables live in an arena
  // exact when built synchronously; upper bounds (table capacities) when built without a host
  // round trip, in which case the exact values are only on the device (d_counts)
  int64_t ntasks = 0, nmulti = 0, nslots = 0;
  int32_t *task_row = nullptr, *tbase = nullptr, *pbase = nullptr, *multi_rows = nullptr;
  uint32_t *d_counts = nullptr;  // {ntasks, nslots, nmulti} on the device (asynchronous builds only)
  void release() {
    if (owned) {
      if (task_row) (void)hipFree(task_row);
      if (tbase) (void)hipFree(tbase);
      if (pbase) (void)hipFree(pbase);
      if (multi_rows) (void)hipFree(multi_rows);
    }
    task_row = tbase = pbase = multi_rows = nullptr;
    d_counts = nullptr;
  }
};

// Task tables for the rows [0, n) described by rowptr.
//   synchronous (async == false): exact table sizes, synchronises `stream`;
//   asynchronous: tables sized by the bounds max_tasks / max_multi, nothing is read back.
static int make_sched(const int32_t *rowptr, int32_t n, int32_t seg, int skip_empty, Sched &out, Alloc &mem,
                      bool async, int64_t max_tasks, int64_t max_multi, hipStream_t stream) {
  Sched sc;
  sc.seg = seg;
  sc.owned = !mem.arena();
  const size_t nb = (size_t)(n + 1) * sizeof(uint32_t);
  uint32_t *d_mbase = nullptr, *d_totals = nullptr;
  TempFree tmp;
  int st = CG_OK;
  do {
    if ((st = mem.get((void **)&sc.tbase, nb)) != CG_OK) break;
    if ((st = mem.get((void **)&sc.pbase, nb)) != CG_OK) break;
    if (mem.arena()) {
      if ((st = mem.get((void **)&d_mbase, nb)) != CG_OK) break;
      if ((st = mem.get((void **)&d_totals, 3 * sizeof(uint32_t))) != CG_OK) break;
    } else {
      if ((st = tmp.alloc((void **)&d_mbase, nb)) != CG_OK) break;
      void *v = nullptr;
      if ((st = scratch_get(stream, kSlotB, 3 * sizeof(uint32_t), &v)) != CG_OK) break;
      d_totals = (uint32_t *)v;
    }
    const unsigned grid = (unsigned)ceil_div64((int64_t)n + 1, kSpmmThreads);
    sched_count_kernel<<<grid, kSpmmThreads, 0, stream>>>(rowptr, n, seg, skip_empty, (uint32_t *)sc.tbase,
                                                          (uint32_t *)sc.pbase, d_mbase);
    if (hipGetLastError() != hipSuccess) {
      st = CG_ERR_HIP;
      set_error("sched_count launch failed");
      break;
    }
    // scanning n + 1 entries leaves the grand total behind the last row: tbase[n] == ntasks
    if ((st = exclusive_scan_u32((uint32_t *)sc.tbase, (uint32_t *)sc.tbase, (int64_t)n + 1, d_totals + 0, stream)) !=
        CG_OK)
      break;
    if ((st = exclusive_scan_u32((uint32_t *)sc.pbase, (uint32_t *)sc.pbase, (int64_t)n + 1, d_totals + 1, stream)) !=
        CG_OK)
      break;
    if ((st = exclusive_scan_u32(d_mbase, d_mbase, (int64_t)n + 1, d_totals + 2, stream)) != CG_OK) break;
    if (async) {
      sc.ntasks = max_tasks;
      sc.nmulti = max_multi;
      sc.nslots = 2 * max_multi;  // bound used for sizing only
      sc.d_counts = d_totals;
    } else {
      uint32_t totals[3] = {0, 0, 0};
      if (hipMemcpyAsync(totals, d_totals, sizeof(totals), hipMemcpyDeviceToHost, stream) != hipSuccess ||
          hipStreamSynchronize(stream) != hipSuccess) {
        st = CG_ERR_HIP;
        set_error("schedule totals copy failed");
        break;
      }
      sc.ntasks = totals[0];
      sc.nslots = totals[1];
      sc.nmulti = totals[2];
    }
    if ((st = mem.get((void **)&sc.task_row, (size_t)(sc.ntasks > 0 ? sc.ntasks : 1) * sizeof(int32_t))) != CG_OK)
      break;
    if ((st = mem.get((void **)&sc.multi_rows, (size_t)(sc.nmulti > 0 ? sc.nmulti : 1) * sizeof(int32_t))) != CG_OK)
      break;
    if (n > 0) {
      sched_fill_kernel<<<(unsigned)ceil_div64(n, kSpmmThreads), kSpmmThreads, 0, stream>>>(
          rowptr, n, seg, skip_empty, (const uint32_t *)sc.tbase, d_mbase, sc.task_row, sc.ntasks, sc.multi_rows,
          sc.nmulti);
      if (hipGetLastError() != hipSuccess) {
        st = CG_ERR_HIP;
        set_error("sched_fill launch failed");
        break;
      }
    }
    if (!async && hipStreamSynchronize(stream) != hipSuccess) {
      st = CG_ERR_HIP;
      set_error("sched_fill failed");
      break;
    }
  } while (0);
  if (st != CG_OK) {
    sc.release();
    return st;
  }
  out = sc;
  return CG_OK;
}

// ---------------------------------------------------------------------------------------------
// window tables
// ---------------------------------------------------------------------------------------------
struct StreamTab {
  int32_t S = 0, groups = 0;
  bool hub = false, owned = true;
  int32_t *task_start = nullptr, *task_dst = nullptr, *wstart = nullptr;
  int64_t nwin = 0;            // exact, or the grid bound of an asynchronous build
  uint32_t *d_nwin = nullptr;  // exact count on the device (asynchronous builds only)
  int64_t win_first[kMaxHubClasses + 2] = {0};
  void release() {
    if (owned) {
      if (task_start) (void)hipFree(task_start);
      if (task_dst) (void)hipFree(task_dst);
      if (wstart) (void)hipFree(wstart);
    }
    task_start = task_dst = wstart = nullptr;
    d_nwin = nullptr;
    S = 0;
  }
};

__device__ __forceinline__ int64_t count_of(int64_t host, const uint32_t *dev) { return dev ? (int64_t)*dev : host; }

// task_dst: row index (>= 0) when the task is the whole row and goes straight to C, else
// -(partial slot + 1).  In a hub plan every task is partial and its slot is its own index.
__global__ __launch_bounds__(kSpmmThreads) void stream_tasks_kernel(
    const int32_t *__restrict__ rowptr, int32_t nrows, const int32_t *__restrict__ task_row,
    const int32_t *__restrict__ tbase, const int32_t *__restrict__ pbase, int32_t seg, int64_t ntasks_host,
    const uint32_t *__restrict__ d_ntasks, int64_t cap, int hub, int32_t *__restrict__ task_start,
    int32_t *__restrict__ task_dst) {
  int64_t ntasks = count_of(ntasks_host, d_ntasks);
  if (ntasks > cap) ntasks = cap;
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
__global__ __launch_bounds__(kSpmmThreads) void window_flag_tasks_kernel(int64_t t0, int64_t t1_host,
                                                                         const uint32_t *__restrict__ d_t1,
                                                                         uint32_t *__restrict__ flags) {
  int64_t t1 = count_of(t1_host, d_t1);
  if (t1 > t1_host) t1 = t1_host;
  const int64_t t = t0 + (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (t < t1) flags[t] = ((t - t0) & 63) == 0 ? 1u : 0u;
}

// ... and the first task that starts at or after every multiple of S entries of the class.
__global__ __launch_bounds__(kSpmmThreads) void window_flag_entries_kernel(const int32_t *__restrict__ task_start,
                                                                           int64_t t0, int64_t t1_host,
                                                                           const uint32_t *__restrict__ d_t1,
                                                                           int32_t S, int64_t nbounds,
                                                                           uint32_t *__restrict__ flags) {
  int64_t t1 = count_of(t1_host, d_t1);
  if (t1 > t1_host) t1 = t1_host;
  const int64_t j = 1 + (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (j > nbounds || t1 <= t0) return;
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
                                                                      int64_t ntasks_host,
                                                                      const uint32_t *__restrict__ d_ntasks,
                                                                      int32_t *__restrict__ wstart,
                                                                      uint32_t *__restrict__ d_nwin, int64_t wcap) {
  int64_t ntasks = count_of(ntasks_host, d_ntasks);
  if (ntasks > ntasks_host) ntasks = ntasks_host;
  const int64_t t = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (t < ntasks && flags[t] && (int64_t)index[t] < wcap) wstart[index[t]] = (int32_t)t;
  if (t == ntasks) {
    const int64_t nwin = (int64_t)index[ntasks] < wcap ? (int64_t)index[ntasks] : wcap;
    wstart[nwin] = (int32_t)ntasks;
    if (d_nwin) *d_nwin = (uint32_t)nwin;
  }
}

// class_first[g] .. class_first[g+1]: tasks of class g (nclass == 1 for a plain schedule).
// nnz: stored entries the tasks cover (bounds the window count of an asynchronous build).
static int build_stream(const Sched &sc, const int32_t *rowptr, int32_t nrows, bool hub, int nclass,
                        const int64_t *class_first, int32_t S, int64_t nnz, StreamTab &out, Alloc &mem, bool async,
                        hipStream_t stream) {
  out.release();
  out.owned = !mem.arena();
  const int64_t nt = sc.ntasks;  // exact, or the capacity bound when async
  const uint32_t *d_nt = async ? sc.d_counts + 0 : nullptr;
  CG_TRY(mem.get((void **)&out.task_start, (size_t)(nt + 1) * 4));
  CG_TRY(mem.get((void **)&out.task_dst, (size_t)(nt + 1) * 4));
  stream_tasks_kernel<<<(unsigned)ceil_div64(nt + 1, kSpmmThreads), kSpmmThreads, 0, stream>>>(
      rowptr, nrows, sc.task_row, sc.tbase, sc.pbase, sc.seg, nt, d_nt, nt, hub ? 1 : 0, out.task_start, out.task_dst);
  CG_LAUNCH_CHECK();
  out.S = S;
  out.hub = hub;
  out.groups = nclass;
  out.nwin = 0;
  for (int g = 0; g <= nclass; ++g) out.win_first[g] = 0;
  if (nt == 0) {
    CG_TRY(mem.get((void **)&out.wstart, 4));
    CG_TRY(fill_u32((uint32_t *)out.wstart, 1, 0u, stream));
    if (!async) CG_HIP(hipStreamSynchronize(stream));
    return CG_OK;
  }
  uint32_t *flags = nullptr, *index = nullptr, *d_total = nullptr;
  TempFree tmp;
  if (mem.arena()) {
    CG_TRY(mem.get((void **)&flags, (size_t)(nt + 1) * 4));
    CG_TRY(mem.get((void **)&index, (size_t)(nt + 1) * 4));
    CG_TRY(mem.get((void **)&d_total, 4));
  } else {
    CG_TRY(tmp.alloc((void **)&flags, (size_t)(nt + 1) * 4));
    CG_TRY(tmp.alloc((void **)&index, (size_t)(nt + 1) * 4));
    void *v = nullptr;
    CG_TRY(scratch_get(stream, kSlotB, 4, &v));
    d_total = (uint32_t *)v;
  }
  // flags[nt] stays 0, so the scan over nt + 1 flags leaves the window count in index[ntasks]
  CG_TRY(fill_u32(flags, nt + 1, 0u, stream));
  if (async) {
    // one class over all tasks; the exact task count stays on the device
    window_flag_tasks_kernel<<<(unsigned)ceil_div64(nt, kSpmmThreads), kSpmmThreads, 0, stream>>>(0, nt, d_nt, flags);
    CG_LAUNCH_CHECK();
    const int64_t nb = nnz / S;
    if (nb > 0) {
      window_flag_entries_kernel<<<(unsigned)ceil_div64(nb, kSpmmThreads), kSpmmThreads, 0, stream>>>(
          out.task_start, 0, nt, d_nt, S, nb, flags);
      CG_LAUNCH_CHECK();
    }
    CG_TRY(exclusive_scan_u32(flags, index, nt + 1, nullptr, stream));
    const int64_t wcap = ceil_div64(nt, 64) + nnz / S + 2;
    CG_TRY(mem.get((void **)&out.wstart, (size_t)(wcap + 1) * 4));
    window_compact_kernel<<<(unsigned)ceil_div64(nt + 1, kSpmmThreads), kSpmmThreads, 0, stream>>>(
        flags, index, nt, d_nt, out.wstart, d_total, wcap);
    CG_LAUNCH_CHECK();
    out.nwin = wcap;
    out.d_nwin = d_total;
    out.win_first[0] = 0;
    out.win_first[1] = wcap;
    return CG_OK;
  }
  // entry extents of the classes (the host needs them to size the boundary launches)
  int32_t ends[kMaxHubClasses + 2];
  for (int g = 0; g <= nclass; ++g)
    CG_HIP(hipMemcpyAsync(&ends[g], out.task_start + class_first[g], 4, hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  for (int g = 0; g < nclass; ++g) {
    const int64_t t0 = class_first[g], t1 = class_first[g + 1];
    if (t1 <= t0) continue;
    window_flag_tasks_kernel<<<(unsigned)ceil_div64(t1 - t0, kSpmmThreads), kSpmmThreads, 0, stream>>>(t0, t1, nullptr,
                                                                                                     flags);
    CG_LAUNCH_CHECK();
    const int64_t nb = ((int64_t)ends[g + 1] - ends[g]) / S;
    if (nb > 0) {
      window_flag_entries_kernel<<<(unsigned)ceil_div64(nb, kSpmmThreads), kSpmmThreads, 0, stream>>>(
          out.task_start, t0, t1, nullptr, S, nb, flags);
      CG_LAUNCH_CHECK();
    }
  }
  CG_TRY(exclusive_scan_u32(flags, index, nt + 1, d_total, stream));
  uint32_t nwin = 0;
  CG_HIP(hipMemcpyAsync(&nwin, d_total, 4, hipMemcpyDeviceToHost, stream));
  uint32_t firsts[kMaxHubClasses + 2] = {0};
  for (int g = 0; g < nclass; ++g)
    CG_HIP(hipMemcpyAsync(&firsts[g], index + class_first[g], 4, hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  for (int g = 0; g < nclass; ++g) out.win_first[g] = firsts[g];
  out.win_first[nclass] = nwin;
  out.nwin = nwin;
  CG_TRY(mem.get((void **)&out.wstart, (size_t)(nwin + 1) * 4));
  window_compact_kernel<<<(unsigned)ceil_div64(nt + 1, kSpmmThreads), kSpmmThreads, 0, stream>>>(
      flags, index, nt, nullptr, out.wstart, nullptr, (int64_t)nwin);
  CG_LAUNCH_CHECK();
  CG_HIP(hipStreamSynchronize(stream));
  return CG_OK;
}

// ---------------------------------------------------------------------------------------------
// launches
// ---------------------------------------------------------------------------------------------
static int64_t stream_grid(const StreamArgs &a) {
  int64_t longest = 0;
  for (int g = 0; g < a.groups; ++g) {
    const int64_t len = a.win_first[g + 1] - a.win_first[g];
    longest = longest > len ? longest : len;
  }
  return ceil_div64(ceil_div64(longest, kWavesPerBlock), 8 / a.groups) * 8;
}

static int launch_stream(const SpmmShape &s, const StreamArgs &a, hipStream_t stream, size_t wide_lds = 0) {
  const int64_t blocks = stream_grid(a);
  if (blocks == 0) return CG_OK;
  if (blocks > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "SpMM grid too large");
  const unsigned grid = (unsigned)blocks;
#define CG_WIDE(V, CH)                                                    \
  if (s.lpr == kWave && s.vec == V && s.chunks == CH) {                   \
    spmm_stream_wide_kernel<V, CH><<<grid, kSpmmThreads, wide_lds, stream>>>(a); \
    CG_LAUNCH_CHECK();                                                    \
    return CG_OK;                                                         \
  }
#define CG_NARROW(V, L)                                                    \
  if (s.lpr == L && s.vec == V) {                                          \
    spmm_stream_narrow_kernel<V, L><<<grid, kSpmmThreads, 0, stream>>>(a); \
    CG_LAUNCH_CHECK();                                                     \
    return CG_OK;                                                          \
  }
#define CG_CASES(V)                                                                                 \
  CG_NARROW(V, 4) CG_NARROW(V, 8) CG_NARROW(V, 16) CG_NARROW(V, 32)                                 \
  CG_WIDE(V, 1) CG_WIDE(V, 2) CG_WIDE(V, 3) CG_WIDE(V, 4) CG_WIDE(V, 5) CG_WIDE(V, 6) CG_WIDE(V, 7) \
  CG_WIDE(V, 8) CG_WIDE(V, 9) CG_WIDE(V, 10)
  CG_CASES(1) CG_CASES(2) CG_CASES(4)
#undef CG_CASES
#undef CG_NARROW
#undef CG_WIDE
  CG_FAIL(CG_ERR_UNSUPPORTED, "no SpMM kernel for vec=%d lpr=%d chunks=%d", s.vec, s.lpr, s.chunks);
}

// ---------------------------------------------------------------------------------------------
// handle data
// ---------------------------------------------------------------------------------------------
// A small cache of schedules (and their window tables) keyed by segment length.
struct SchedCache {
  static constexpr int kMax = 4;
  Sched sched[kMax];
  StreamTab tab[kMax];
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
    Alloc owned;
    CG_TRY(make_sched(rowptr, n, seg, 0, sched[count], owned, false, 0, 0, stream));
    *out = &sched[count++];
    return CG_OK;
  }
};

// Hub plan: the stored entries regrouped by column class.  Columns (= rows of B) are ranked by
// descending reference count; the first `hot` ranks form tier 0, the next `hot` tier 1, ...; inside
// a tier the columns are dealt round robin to `groups` groups, and every column behind the last
// tier is cold.  Class = tier * groups + group.  A tier is one launch in which XCD x only reads the
// B rows of group x % groups, so each XCD's private L2 keeps its own share of the hot rows.
// Entries are kept as one CSR over (classes + 1) * rows virtual rows, virtual row c * rows + r
// holding the entries of row r whose column has class c (cold = class `classes`).
struct HubPlan {
  int32_t hot = 0, groups = 0, tiers = 0, seg = 0, min_degree = 0;
  int32_t req_hot = 0, req_tiers = 0, req_single = 0;  // what was asked for (tiers 0: chosen from the column counts)
  bool declined = false;  // the column counts said a plan does not pay: the plain schedule is used
  int32_t classes() const { return groups * tiers; }
  int32_t *vrowptr = nullptr, *colind = nullptr;
  float *val = nullptr;
  uint8_t *row_hot = nullptr;  // 1 for rows long enough to have hot entries
  Sched hot_sched;        // over the virtual rows of the hot classes, empty rows skipped
  StreamTab hot_tab;      // its windows, one class per (tier, group)
  SchedCache cold_sched;  // over the cold class
  int64_t tstart[kMaxHubClasses + 2] = {0};
  bool valid = false;
  void release() {
    hot_sched.release();
    hot_tab.release();
    cold_sched.release();
    if (vrowptr) (void)hipFree(vrowptr);
    if (colind) (void)hipFree(colind);
    if (val) (void)hipFree(val);
    if (row_hot) (void)hipFree(row_hot);
    vrowptr = colind = nullptr;
    val = nullptr;
    row_hot = nullptr;
    valid = false;
    declined = false;
  }
};

struct CsrSide {
  int32_t rows = 0, cols = 0;
  int64_t nnz = 0;
  int32_t *rowptr = nullptr, *colind = nullptr;
  float *val = nullptr;
  int32_t max_degree = 0;
  SchedCache sched;
  // Hub plans depend on the product width (through the number of hot columns); a model with two
  // wide layers alternates between two of them, so two are kept and the older one is replaced.
  static constexpr int kHubPlans = 2;
  HubPlan hub[kHubPlans];
  uint64_t hub_used[kHubPlans] = {0, 0};
  uint64_t hub_clock = 0;
  void release() {
    sched.release();
    for (int i = 0; i < kHubPlans; ++i) hub[i].release();
    if (rowptr) (void)hipFree(rowptr);
    if (colind) (void)hipFree(colind);
    if (val) (void)hipFree(val);
    rowptr = colind = nullptr;
    val = nullptr;
  }
};

// ---------------------------------------------------------------------------------------------
// hub plan construction
// ---------------------------------------------------------------------------------------------
// only entries of rows with at least min_degree entries can be hot, so only they are counted
__global__ __launch_bounds__(kSpmmThreads) void col_count_kernel(const int32_t *__restrict__ colind, int64_t nnz,
                                                                 const int32_t *__restrict__ rowptr,
                                                                 const int32_t *__restrict__ erow, int32_t min_degree,
                                                                 uint32_t *__restrict__ count) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k >= nnz) return;
  const int32_t r = erow[k];
  if (rowptr[r + 1] - rowptr[r] >= min_degree) atomicAdd(&count[colind[k]], 1u);  // integer count: order independent
}

__global__ __launch_bounds__(kSpmmThreads) void row_hot_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                               int32_t min_degree, uint8_t *__restrict__ out) {
  const int64_t r = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (r < n) out[r] = rowptr[r + 1] - rowptr[r] >= min_degree ? 1 : 0;
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

// sums[t] = entries whose column has rank [t * hot, (t + 1) * hot): one workgroup per tier.  The keys
// are maxcount - count in ascending order.
__global__ __launch_bounds__(kSpmmThreads) void tier_sum_kernel(const int32_t *__restrict__ sorted_key, int32_t m,
                                                                uint32_t maxcount, int32_t hot,
                                                                unsigned long long *__restrict__ sums) {
  __shared__ unsigned long long part[kSpmmThreads / kWave];
  const int64_t lo = (int64_t)blockIdx.x * hot;
  int64_t hi = lo + hot;
  if (hi > m) hi = m;
  unsigned long long v = 0;
  for (int64_t r = lo + threadIdx.x; r < hi; r += kSpmmThreads) v += (unsigned long long)(maxcount - (uint32_t)sorted_key[r]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long t = 0;
    for (int w = 0; w < kSpmmThreads / kWave; ++w) t += part[w];
    sums[blockIdx.x] = t;
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

// class of an entry: that of its column when its row is long enough, else cold.  A hot entry costs
// its row a partial row per class (written, then read again by the fold), which only pays when
// the row has many entries to spread over the classes.
__global__ __launch_bounds__(kSpmmThreads) void entry_class_kernel(const int32_t *__restrict__ colind, int64_t nnz,
                                                                   const int32_t *__restrict__ cls,
                                                                   const int32_t *__restrict__ rowptr,
                                                                   const int32_t *__restrict__ erow,
                                                                   int32_t min_degree, int32_t cold,
                                                                   int32_t *__restrict__ out,
                                                                   int32_t *__restrict__ pos) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < nnz) {
    const int32_t r = erow[k];
    out[k] = rowptr[r + 1] - rowptr[r] >= min_degree ? cls[colind[k]] : cold;
    pos[k] = (int32_t)k;  // position in the original CSR, carried through the sort
  }
}

__global__ __launch_bounds__(kSpmmThreads) void entry_finish_kernel(
    const int32_t *__restrict__ cls_sorted, const int32_t *__restrict__ row_sorted, const int32_t *__restrict__ pos,
    int64_t nnz, int32_t rows, const int32_t *__restrict__ colind, const float *__restrict__ val,
    int32_t *__restrict__ vrow, int32_t *__restrict__ colind2, float *__restrict__ val2) {
  const int64_t k = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  if (k < nnz) {
    const int32_t p = pos[k];
    vrow[k] = cls_sorted[k] * rows + row_sorted[k];
    colind2[k] = colind[p];
    val2[k] = val[p];
  }
}

__global__ __launch_bounds__(kSpmmThreads) void csr_rows_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                int32_t *__restrict__ row_out) {
  const int64_t wave = ((int64_t)blockIdx.x * kSpmmThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (wave >= n) return;
  const int32_t s = rowptr[wave], e = rowptr[wave + 1];
  for (int32_t k = s + lane; k < e; k += kWave) row_out[k] = (int32_t)wave;
}

// tiers == 0: the number of tiers is chosen from the column counts (tiers of `hot` columns each); if
// one tier comes out, it holds `hot_single` columns.
// may_decline: leave the plan empty (h.declined) when the first tier would hold less than
// kHubMinHotFraction of the entries.
static int build_hub(CsrSide &s, HubPlan &h, int32_t hot, int32_t hot_single, int32_t groups, int32_t tiers,
                     int32_t seg, int32_t min_degree, bool may_decline, hipStream_t stream) {
  CG_HIP(hipStreamSynchronize(stream));
  h.release();
  h.req_hot = hot;
  h.req_tiers = tiers;
  h.req_single = hot_single;
  const int64_t nnz = s.nnz;
  const int32_t n = s.rows, m = s.cols;
  if (hot < 1) hot = 1;
  if (hot_single < 1) hot_single = 1;
  if ((int64_t)(kMaxHubClasses + 1) * n + 1 > 0x7fffffffLL && tiers == 0) tiers = 1;  // keep the virtual rows in int32
  TempFree tmp;
  const unsigned gm = (unsigned)ceil_div64(m, kSpmmThreads), ge = (unsigned)ceil_div64(nnz, kSpmmThreads);

  // 1. reference count of every column (over the rows that may have hot entries), and the columns
  //    ranked by it
  uint32_t *count = nullptr;
  int32_t *cls = nullptr, *erow = nullptr;
  CG_TRY(tmp.alloc((void **)&count, (size_t)m * 4));
  CG_TRY(tmp.alloc((void **)&cls, (size_t)m * 4));
  CG_TRY(tmp.alloc((void **)&erow, (size_t)nnz * 4));
  CG_TRY(fill_u32(count, m, 0u, stream));
  if (n > 0) {
    csr_rows_kernel<<<(unsigned)ceil_div64((int64_t)n * kWave, kSpmmThreads), kSpmmThreads, 0, stream>>>(s.rowptr, n, erow);
    CG_LAUNCH_CHECK();
  }
  col_count_kernel<<<ge, kSpmmThreads, 0, stream>>>(s.colind, nnz, s.rowptr, erow, min_degree, count);
  CG_LAUNCH_CHECK();
  {
    SortBuffers buf;
    for (int i = 0; i < 2; ++i) {
      CG_TRY(tmp.alloc((void **)&buf.key_a[i], (size_t)m * 4));
      CG_TRY(tmp.alloc((void **)&buf.payload[i], (size_t)m * 4));
      CG_TRY(tmp.alloc((void **)&buf.key_b[i], (size_t)m * 4));  // no minor key: carried, never sorted on
    }
    const uint32_t maxcount = (uint32_t)(nnz < 0x7fffffffLL ? nnz : 0x7fffffffLL);
    col_key_kernel<<<gm, kSpmmThreads, 0, stream>>>(count, m, maxcount, buf.key_a[0], buf.payload[0]);
    CG_LAUNCH_CHECK();
    CG_TRY(fill_u32((uint32_t *)buf.key_b[0], m, 0u, stream));
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, m, bits_for((int32_t)(maxcount < 0x7ffffffeu ? maxcount + 1 : 0x7fffffff)), 0, &set,
                            stream));
    if (tiers == 0 || may_decline) {
      const int max_tiers = kMaxHubClasses / groups < kHubAutoTiers ? kMaxHubClasses / groups : kHubAutoTiers;
      unsigned long long *d_sums = nullptr, sums[kHubAutoTiers] = {0};
      CG_TRY(tmp.alloc((void **)&d_sums, sizeof(sums)));
      tier_sum_kernel<<<max_tiers, kSpmmThreads, 0, stream>>>(buf.key_a[set], m, maxcount, hot, d_sums);
      CG_LAUNCH_CHECK();
      CG_HIP(hipMemcpyAsync(sums, d_sums, sizeof(unsigned long long) * max_tiers, hipMemcpyDeviceToHost, stream));
      CG_HIP(hipStreamSynchronize(stream));
      // Measured over R-MAT graphs of 16 to 492 entries per row and blocks of them: with 45 % or more
      // of the entries in the first tier the plan gains 20 to 37 %, with 25 to 29 % it gains 1 to 4 %.
      if (may_decline && (double)sums[0] < kHubMinHotFraction * (double)nnz) {
        h.declined = true;
        h.groups = groups;
        h.seg = seg;
        h.min_degree = min_degree;
        h.valid = true;
        return CG_OK;
      }
      if (tiers == 0) {
        // A further tier serves its entries from L2 instead of HBM but costs every (class, row) pair it
        // touches a partial row, written and read again: it pays while it holds well over two
        // entries per pair it can have (measured break-even 2.4: f = 602 takes 3 tiers, 300 two, 128 one).
        tiers = 1;
        while (tiers < max_tiers && (double)sums[tiers] >= kHubTierEntriesPerPair * (double)groups * (double)n) ++tiers;
        if (tiers == 1) hot = hot_single;
      }
    }
    col_class_kernel<<<gm, kSpmmThreads, 0, stream>>>(buf.payload[set], m, hot, groups, tiers, cls);
    CG_LAUNCH_CHECK();
  }
  const int32_t nclass = groups * tiers;
  const int64_t vrows = (int64_t)(nclass + 1) * n;
  if (vrows + 1 > 0x7fffffffLL) CG_FAIL(CG_ERR_OVERFLOW, "hub plan: %lld virtual rows exceed int32", (long long)vrows);

  // 2. stable regrouping of the entries by class: (row, col) order is kept inside a class
  CG_TRY(dev_alloc((void **)&h.row_hot, (size_t)(n > 0 ? n : 1)));
  if (n > 0) {
    row_hot_kernel<<<(unsigned)ceil_div64(n, kSpmmThreads), kSpmmThreads, 0, stream>>>(s.rowptr, n, min_degree, h.row_hot);
    CG_LAUNCH_CHECK();
  }
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
    entry_class_kernel<<<ge, kSpmmThreads, 0, stream>>>(s.colind, nnz, cls, s.rowptr, erow, min_degree, nclass,
                                                        buf.key_a[0], buf.payload[0]);
    CG_LAUNCH_CHECK();
    CG_HIP(hipMemcpyAsync(buf.key_b[0], erow, (size_t)nnz * 4, hipMemcpyDeviceToDevice, stream));
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, nnz, bits_for(nclass + 1), 0, &set, stream));
    entry_finish_kernel<<<ge, kSpmmThreads, 0, stream>>>(buf.key_a[set], buf.key_b[set], buf.payload[set], nnz, n,
                                                         s.colind, s.val, vrow, h.colind, h.val);
    CG_LAUNCH_CHECK();
    CG_HIP(hipStreamSynchronize(stream));
  }
  CG_TRY(launch_rowptr(vrow, nnz, (int32_t)vrows, h.vrowptr, stream));

  // 3. tasks of the hot classes (empty virtual rows get none); the cold class is scheduled on demand
  Alloc owned;
  CG_TRY(make_sched(h.vrowptr, nclass * n, seg, 1, h.hot_sched, owned, false, 0, 0, stream));
  {
    int32_t t[kMaxHubClasses + 2];
    for (int g = 0; g <= nclass; ++g)
      CG_HIP(hipMemcpyAsync(&t[g], h.hot_sched.tbase + (int64_t)g * n, 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipStreamSynchronize(stream));
    for (int g = 0; g <= nclass; ++g) h.tstart[g] = t[g];
  }
  h.hot = hot;
  h.groups = groups;
  h.tiers = tiers;
  h.seg = seg;
  h.min_degree = min_degree;
  h.valid = true;
  return CG_OK;
}

// ---------------------------------------------------------------------------------------------
// products
// ---------------------------------------------------------------------------------------------
struct DenseOps {
  const float *B;
  int64_t ldb;
  float *C;
  int64_t ldc;
  int32_t f;
  float beta;
  // optional fold of another launch's partial rows into the rows written here (see StreamArgs)
  const int32_t *fold_tbase = nullptr;
  const float *fold_P = nullptr;
  const uint8_t *fold_any = nullptr;
  int32_t fold_classes = 0, fold_rows = 0;
  // optional epilogue: finished rows are multiplied by W (f x fo) into Z instead of being stored
  // (see StreamArgs); C is then only read, and only when beta != 0
  const float *epi_W = nullptr;
  int64_t epi_ldw = 0;
  float *epi_Z = nullptr;
  int64_t epi_ldz = 0;
  int32_t epi_fo = 0, epi_relu = 0;
};

constexpr size_t kEpiLdsBytes = 64 * 1024;
static int32_t epi_pad(int32_t fo) { return fo <= 16 ? 16 : (fo <= 32 ? 32 : 64); }
static size_t epi_lds_bytes(int32_t f, int32_t fo) {  // W^T rows and one row buffer per wave, each fpad floats
  const size_t fpad = (size_t)(f + 15) / 16 * 16 + 4;
  return ((size_t)epi_pad(fo) + kWavesPerBlock) * fpad * sizeof(float);
}

// Row-segment tasks over (rowptr, colind, val), for a column range one launch can cover.
static int spmm_plain(const int32_t *rowptr, const int32_t *colind, const float *val, int32_t rows, int64_t nnz,
                      SchedCache &cache, int vec, const DenseOps &d, int prof_tag, hipStream_t stream) {
  const SpmmShape shape = pick_shape(vec, d.f / vec);
  Sched *sc = nullptr;
  CG_TRY(cache.get(rowptr, rows, pick_seg(shape), &sc, stream));
  StreamTab &tab = cache.tab_of(sc);
  const int32_t S = window_entries();
  if (tab.S != S) {
    const int64_t first[2] = {0, sc->ntasks};
    Alloc owned;
    CG_TRY(build_stream(*sc, rowptr, rows, false, 1, first, S, nnz, tab, owned, false, stream));
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
  sa.B = d.B;
  sa.ldb = d.ldb;
  sa.C = d.C;
  sa.ldc = d.ldc;
  sa.f = d.f;
  sa.beta = d.beta;
  sa.fold_tbase = d.fold_tbase;
  sa.fold_P = d.fold_P;
  sa.fold_any = d.fold_any;
  sa.fold_classes = d.fold_classes;
  sa.fold_rows = d.fold_rows;
  if (d.fold_tbase && shape.lpr != kWave) CG_FAIL(CG_ERR_UNSUPPORTED, "fold needs full-wave teams");
  size_t lds = 0;
  if (d.epi_W) {
    if (shape.lpr != kWave) CG_FAIL(CG_ERR_UNSUPPORTED, "epilogue needs full-wave teams");
    sa.epi_W = d.epi_W;
    sa.epi_ldw = d.epi_ldw;
    sa.epi_Z = d.epi_Z;
    sa.epi_ldz = d.epi_ldz;
    sa.epi_fo = d.epi_fo;
    sa.epi_fop = epi_pad(d.epi_fo);
    sa.epi_relu = d.epi_relu;
    lds = epi_lds_bytes(d.f, d.epi_fo);
  }
  if (sc->nslots > 0) {
    void *p = nullptr;
    CG_TRY(scratch_get(stream, kSlotA, (size_t)sc->nslots * d.f * sizeof(float), &p));
    sa.P = (float *)p;
  }
  {
    ProfScope prof("spmm_rowseg", prof_tag, stream);
    CG_TRY(launch_stream(shape, sa, stream, lds));
  }
  if (sc->nmulti > 0 && d.epi_W) {
    ProfScope prof("spmm_reduce", prof_tag, stream);
    ReduceEpiArgs ra{};
    ra.multi_rows = sc->multi_rows;
    ra.nmulti = sc->nmulti;
    ra.rowptr = rowptr;
    ra.pbase = sc->pbase;
    ra.seg = sc->seg;
    ra.P = sa.P;
    ra.C = d.C;
    ra.ldc = d.ldc;
    ra.f = d.f;
    ra.beta = d.beta;
    ra.fold_tbase = d.fold_tbase;
    ra.fold_P = d.fold_P;
    ra.fold_classes = d.fold_classes;
    ra.fold_rows = d.fold_rows;
    ra.epi_W = sa.epi_W;
    ra.epi_ldw = sa.epi_ldw;
    ra.epi_Z = sa.epi_Z;
    ra.epi_ldz = sa.epi_ldz;
    ra.epi_fo = sa.epi_fo;
    ra.epi_fop = sa.epi_fop;
    ra.epi_relu = sa.epi_relu;
    spmm_reduce_epi_kernel<<<(unsigned)ceil_div64(sc->nmulti, kWavesPerBlock), kSpmmThreads, lds, stream>>>(ra);
    CG_LAUNCH_CHECK();
  } else if (sc->nmulti > 0) {
    ProfScope prof("spmm_reduce", prof_tag, stream);
    const int64_t threads = sc->nmulti * (int64_t)d.f;
    spmm_reduce_kernel<<<(unsigned)ceil_div64(threads, kSpmmThreads), kSpmmThreads, 0, stream>>>(
        sc->multi_rows, sc->nmulti, nullptr, rowptr, sc->pbase, sc->seg, sa.P, d.C, d.ldc, d.f, d.beta, 0, d.fold_tbase,
        d.fold_P, d.fold_classes, d.fold_rows);
    CG_LAUNCH_CHECK();
  }
  return CG_OK;
}

// Should a product of this width over this matrix go through a hub plan?  It pays when a row of B
// is two cache lines or more (the gather dominates) and rows hold enough hot entries per group that the
// partial rows they cost are small against the gathers they turn into L2 hits.
constexpr int32_t kHubRowDegree = 64;  // rows shorter than this keep all their entries in the cold class

// Cheap test before any plan is built: wide rows of B, enough work for the extra launches to
// disappear in it (products under about 3e9 multiply-adds measured slower with a plan), and not
// a matrix of near-empty rows.  Whether the hot columns carry enough of the entries is decided
// from the column counts when the plan is built (build_hub may decline).
static bool want_hub(int32_t rows, int64_t nnz, int32_t f) {
  const int t = g_tune_hub.load(std::memory_order_relaxed);
  if (t < 0) return false;
  if (rows == 0 || nnz == 0) return false;
  if (t > 0) return true;
  return f >= 64 && nnz / rows >= 8 && (double)nnz * f >= 3e9;
}
static bool want_hub(const CsrSide &s, int32_t f) { return want_hub(s.rows, s.nnz, f); }

// *declined: the plan was found not to pay for this matrix and width; nothing was computed.
static int spmm_hub(CsrSide &s, int vec, const DenseOps &d, hipStream_t stream, bool *declined) {
  *declined = false;
  const int32_t f = d.f;
  // Aligned rows whose 16-byte pieces would leave a third of the last chunk's lanes idle (f = 300:
  // 75 pieces on 128 lanes) take narrower pieces: with most gathers served from L2 the product is
  // bound by issued loads rather than by bytes (Reddit shape, f = 300: 8.95 -> 8.2 ms).
  if (vec == 4 && f / 4 > kWave) {
    auto lanes_used = [&](int v) {
      const int slots = f / v;
      return (double)slots / (double)((slots + kWave - 1) / kWave * kWave);
    };
    while (vec > 1 && lanes_used(vec) < 0.75 && lanes_used(vec / 2) > lanes_used(vec)) vec /= 2;
  }
  int groups = g_tune_hub_groups.load(std::memory_order_relaxed);
  if (groups != 1 && groups != 2 && groups != 4 && groups != 8) groups = 8;
  // Hot columns per tier = the rows of B that fit `kb` KiB per XCD group.  One tier: twice the 4 MB
  // L2 of an XCD is the measured optimum (LRU keeps the hotter half).  Several tiers: each is sized
  // to stay resident (measured optimum 5 to 6 MiB); how many there are is decided from the column
  // counts when the plan is built, unless a number is forced.
  int tiers = g_tune_hub_tiers.load(std::memory_order_relaxed);
  if (tiers < 0 || tiers * groups > kMaxHubClasses) tiers = 0;
  const int kb_forced = g_tune_hub_kb.load(std::memory_order_relaxed);
  auto columns_for = [&](int kb) {
    int64_t per_group = (int64_t)kb * 1024 / ((int64_t)f * 4);
    if (per_group < 1) per_group = 1;
    const int64_t c = per_group * groups;
    return c > s.cols ? (int64_t)s.cols : c;
  };
  const int64_t hot = columns_for(kb_forced > 0 ? kb_forced : (tiers == 1 ? 8192 : 5632));  // per tier
  const int64_t hot_single = columns_for(kb_forced > 0 ? kb_forced : 8192);
  // hot tasks of a wide product use one dword per lane and chunk when the rows are not 16-byte
  // aligned: that is the fastest gather of L2-resident rows
  const int hot_vec = (vec == 4 || f / vec <= kWave) ? vec : 1;
  const SpmmShape hshape = pick_shape(hot_vec, f / hot_vec);
  const int32_t seg = pick_seg(hshape);
  int32_t min_degree = g_tune_hub_row.load(std::memory_order_relaxed);
  if (min_degree <= 0) min_degree = kHubRowDegree;
  const bool may_decline = g_tune_hub.load(std::memory_order_relaxed) == 0;
  int slot = -1;
  for (int i = 0; i < CsrSide::kHubPlans; ++i)
    if (s.hub[i].valid && s.hub[i].req_hot == (int32_t)hot && s.hub[i].req_single == (int32_t)hot_single &&
        s.hub[i].req_tiers == tiers && s.hub[i].groups == groups && s.hub[i].seg == seg &&
        s.hub[i].min_degree == min_degree && (may_decline || !s.hub[i].declined))
      slot = i;
  if (slot < 0) {
    slot = 0;
    for (int i = 0; i < CsrSide::kHubPlans; ++i) {
      if (!s.hub[i].valid) {
        slot = i;
        break;
      }
      if (s.hub_used[i] < s.hub_used[slot]) slot = i;
    }
    CG_TRY(build_hub(s, s.hub[slot], (int32_t)hot, (int32_t)hot_single, groups, tiers, seg, min_degree, may_decline,
                     stream));
  }
  s.hub_used[slot] = ++s.hub_clock;
  HubPlan &h = s.hub[slot];
  if (h.declined) {
    *declined = true;
    return CG_OK;
  }
  const int32_t n = s.rows;
  const int32_t nclass = h.classes();
  // 1. hot classes, one launch per tier: every task writes a partial row
  const int64_t hot_tasks = h.hot_sched.ntasks;
  void *p = nullptr;
  if (hot_tasks > 0) {
    CG_TRY(scratch_get(stream, kSlotC, (size_t)hot_tasks * f * sizeof(float), &p));
    const int32_t S = window_entries();
    if (h.hot_tab.S != S || h.hot_tab.groups != nclass) {
      Alloc owned;
      CG_TRY(build_stream(h.hot_sched, h.vrowptr, nclass * n, true, nclass, h.tstart, S, s.nnz, h.hot_tab, owned, false,
                          stream));
    }
    ProfScope prof("spmm_hub_hot", f, stream);  // all tiers of a product are timed as one
    for (int t = 0; t < h.tiers; ++t) {
      StreamArgs sa{};
      sa.task_start = h.hot_tab.task_start;
      sa.task_dst = h.hot_tab.task_dst;
      sa.wstart = h.hot_tab.wstart;
      sa.colind = h.colind;
      sa.val = h.val;
      for (int g = 0; g <= groups; ++g) sa.win_first[g] = h.hot_tab.win_first[t * groups + g];
      sa.groups = groups;
      sa.B = d.B;
      sa.ldb = d.ldb;
      sa.C = d.C;
      sa.ldc = d.ldc;
      sa.P = (float *)p;
      sa.f = f;
      sa.beta = 0.f;
      CG_TRY(launch_stream(hshape, sa, stream));
    }
  }
  // 2. cold class straight into C.  Full-wave teams add the hot partial rows of a row in the same
  //    store; narrower teams leave that to a separate fold.
  DenseOps cold = d;
  const bool fused = hot_tasks > 0 && pick_shape(vec, f / vec).lpr == kWave;
  if (fused) {
    cold.fold_tbase = h.hot_sched.tbase;
    cold.fold_P = (const float *)p;
    cold.fold_any = h.row_hot;
    cold.fold_classes = nclass;
    cold.fold_rows = n;
  }
  CG_TRY(spmm_plain(h.vrowptr + (int64_t)nclass * n, h.colind, h.val, n, s.nnz, h.cold_sched, vec, cold, f, stream));
  if (hot_tasks > 0 && !fused) {
    ProfScope prof("spmm_hub_reduce", f, stream);
    const unsigned rgrid = (unsigned)ceil_div64((int64_t)n * kWave, kSpmmThreads);
    if (nclass <= 8)
      hub_reduce_kernel<8><<<rgrid, kSpmmThreads, 0, stream>>>(h.hot_sched.tbase, n, nclass, (const float *)p, d.C,
                                                               d.ldc, f);
    else if (nclass <= 16)
      hub_reduce_kernel<16><<<rgrid, kSpmmThreads, 0, stream>>>(h.hot_sched.tbase, n, nclass, (const float *)p, d.C,
                                                                d.ldc, f);
    else if (nclass <= 32)
      hub_reduce_kernel<32><<<rgrid, kSpmmThreads, 0, stream>>>(h.hot_sched.tbase, n, nclass, (const float *)p, d.C,
                                                                d.ldc, f);
    else
      hub_reduce_kernel<64><<<rgrid, kSpmmThreads, 0, stream>>>(h.hot_sched.tbase, n, nclass, (const float *)p, d.C,
                                                                d.ldc, f);
    CG_LAUNCH_CHECK();
  }
  return CG_OK;
}

// epi (nullable): only its epilogue fields are read; the product then ends in Z = act(row * W)
// instead of C, which needs full-wave teams, one column range and room for W in LDS.
static bool epi_supported(int32_t f, int32_t fo, int vec) {
  return fo >= 1 && fo <= 64 && f <= range_cap(vec) && pick_shape(vec, f / vec).lpr == kWave &&
         epi_lds_bytes(f, fo) <= kEpiLdsBytes;
}

static int spmm_side(CsrSide &s, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta,
                     hipStream_t stream, const DenseOps *epi = nullptr) {
  if (s.rows == 0) return CG_OK;
  const int vec = pick_vec(f, B, ldb, C ? C : B, C ? ldc : ldb);
  const int32_t cap = range_cap(vec);
  DenseOps d{B, ldb, C, ldc, f, beta};
  if (epi) {
    if (!epi_supported(f, epi->epi_fo, vec))
      CG_FAIL(CG_ERR_UNSUPPORTED, "fused product: f=%d fo=%d has no fused form", f, epi->epi_fo);
    d.epi_W = epi->epi_W;
    d.epi_ldw = epi->epi_ldw;
    d.epi_Z = epi->epi_Z;
    d.epi_ldz = epi->epi_ldz;
    d.epi_fo = epi->epi_fo;
    d.epi_relu = epi->epi_relu;
  }
  if (f <= range_cap(vec == 4 ? 4 : 1) && want_hub(s, f)) {
    bool declined = false;
    CG_TRY(spmm_hub(s, vec, d, stream, &declined));
    if (!declined) return CG_OK;
  }
  if (epi) return spmm_plain(s.rowptr, s.colind, s.val, s.rows, s.nnz, s.sched, vec, d, f, stream);
  for (int32_t f0 = 0; f0 < f; f0 += cap) {  // wider outputs take several launches over column ranges
    const int32_t ft = f - f0 < cap ? f - f0 : cap;
    const DenseOps dr{B + f0, ldb, C + f0, ldc, ft, beta};
    CG_TRY(spmm_plain(s.rowptr, s.colind, s.val, s.rows, s.nnz, s.sched, vec, dr, f, stream));
  }
  return CG_OK;
}

// One-shot product from row-sorted COO: rowptr, schedule and window tables are rebuilt in a
// scratch arena on every call, as device work on `stream` only (no allocation once the scratch
// has grown, no host round trip: table sizes are bounds, the exact counts stay on the device).
static int spmm_coo_oneshot(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n,
                            int32_t m, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta,
                            hipStream_t stream) {
  const int vec = pick_vec(f, B, ldb, C, ldc);
  const int32_t cap = range_cap(vec);
  const int32_t fmax = f < cap ? f : cap;
  // every column range uses the tables of the first (widest) one; a narrower last range only
  // means shorter teams over the same tasks, which is valid as long as the segment length fits
  const SpmmShape shape0 = pick_shape(vec, fmax / vec);
  int32_t seg = pick_seg(shape0);
  if (f > cap && (f % cap) / vec <= kWave && seg > 512) seg = 512;  // the tail range runs narrow teams
  const int32_t S = window_entries();
  const int64_t max_multi = nnz / seg + 1;
  const int64_t max_tasks = (int64_t)n + nnz / seg + 1;
  const int64_t wcap = ceil_div64(max_tasks, 64) + nnz / S + 2;
  // arena: rowptr, tbase/pbase/mbase, task_row, multi_rows, task_start/dst, flags/index, wstart
  const size_t words = 4 * (size_t)(n + 1) + (size_t)max_tasks + (size_t)max_multi + 4 * (size_t)(max_tasks + 1) +
                       (size_t)(wcap + 1) + 16;
  const size_t arena_bytes = words * 4 + 32 * 256;
  void *abase = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, arena_bytes, &abase));
  Alloc mem;
  mem.base = (char *)abase;
  mem.cap = arena_bytes;
  int32_t *rowptr = nullptr;
  CG_TRY(mem.get((void **)&rowptr, (size_t)(n + 1) * 4));
  // rows the compression never reaches (only possible for unsorted input) stay 0
  CG_TRY(fill_u32((uint32_t *)rowptr, (int64_t)n + 1, 0u, stream));
  CG_TRY(launch_rowptr(d_row, nnz, n, rowptr, stream));
  Sched sc;
  CG_TRY(make_sched(rowptr, n, seg, 0, sc, mem, true, max_tasks, max_multi, stream));
  StreamTab tab;
  const int64_t first[2] = {0, max_tasks};
  CG_TRY(build_stream(sc, rowptr, n, false, 1, first, S, nnz, tab, mem, true, stream));
  const int64_t pslots = 2 * max_multi;
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotA, (size_t)pslots * fmax * sizeof(float), &p));
  for (int32_t f0 = 0; f0 < f; f0 += cap) {
    const int32_t ft = f - f0 < cap ? f - f0 : cap;
    const SpmmShape shape = pick_shape(vec, ft / vec);
    StreamArgs sa{};
    sa.task_start = tab.task_start;
    sa.task_dst = tab.task_dst;
    sa.wstart = tab.wstart;
    sa.colind = d_col;
    sa.val = d_val;
    sa.win_first[0] = 0;
    sa.win_first[1] = tab.nwin;
    sa.groups = 1;
    sa.clamp_m = m;
    sa.p_cap = pslots;
    sa.d_nwin = tab.d_nwin;
    sa.B = B + f0;
    sa.ldb = ldb;
    sa.C = C + f0;
    sa.ldc = ldc;
    sa.P = (float *)p;
    sa.f = ft;
    sa.beta = beta;
    {
      ProfScope prof("spmm_rowseg", f, stream);
      CG_TRY(launch_stream(shape, sa, stream));
    }
    ProfScope prof("spmm_reduce", f, stream);
    const int64_t threads = max_multi * (int64_t)ft;
    spmm_reduce_kernel<<<(unsigned)ceil_div64(threads, kSpmmThreads), kSpmmThreads, 0, stream>>>(
        sc.multi_rows, max_multi, sc.d_counts + 2, rowptr, sc.pbase, seg, (const float *)p, C + f0, ldc, ft, beta,
        pslots, nullptr, nullptr, 0, 0);
    CG_LAUNCH_CHECK();
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
  s.nnz = nnz;
  CG_TRY(dev_alloc((void **)&s.rowptr, (size_t)(rows + 1) * sizeof(int32_t)));
  CG_TRY(dev_alloc((void **)&s.colind, (size_t)nnz * sizeof(int32_t)));
  CG_TRY(dev_alloc((void **)&s.val, (size_t)nnz * sizeof(float)));
  return CG_OK;
}

static int side_max_degree(CsrSide &s, hipStream_t stream) {
  void *d = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, sizeof(int), &d));
  CG_TRY(fill_u32((uint32_t *)d, 1, 0u, stream));
  if (s.rows > 0) {
    int64_t blocks = ceil_div64(s.rows, kSpmmThreads);
    if (blocks > 2048) blocks = 2048;
    max_degree_kernel<<<(unsigned)blocks, kSpmmThreads, 0, stream>>>(s.rowptr, s.rows, (int *)d);
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

// ---------------------------------------------------------------------------------------------
// Blocks recognised by content (cg_spmm_coo_cached).  The reference's callers hand the same COO
// arrays to spmm_gpu at every stage of every epoch (gcn_distr.py:238-240), through fresh `.int()`
// temporaries, so neither addresses nor tensor identities say whether a block was seen before.
// A 128-bit digest of (row, col, val) computed on the device does; blocks seen before reuse the
// handle (CSR copy, schedules, hub plans) built at their first sighting.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned long long mix64(unsigned long long x) {  // splitmix64 finaliser
  x ^= x >> 30;
  x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 27;
  x *= 0x94D049BB133111EBull;
  x ^= x >> 31;
  return x;
}

// out[0..1] += two independent 64-bit sums over the entries; the position of an entry is part of
// what is mixed, so the digest depends on the order, and integer addition makes it independent of
// how the partial sums are combined.
__device__ __forceinline__ void digest_entry(int32_t r, int32_t c, float v, int64_t i, unsigned long long &h1,
                                             unsigned long long &h2) {
  const unsigned long long a = (unsigned long long)(uint32_t)r | ((unsigned long long)(uint32_t)c << 32);
  const unsigned long long b = (unsigned long long)__float_as_uint(v) | ((unsigned long long)i << 32);
  h1 += mix64(a ^ mix64(b + 0x9E3779B97F4A7C15ull));
  h2 += mix64((a + 0xD6E8FEB86659FD93ull) * 0xFF51AFD7ED558CCDull ^ mix64(b ^ 0xC2B2AE3D27D4EB4Full));
}

// VEC 4: the three arrays are 16-byte aligned and a thread reads 4 entries per access.
template <int VEC>
__global__ __launch_bounds__(kSpmmThreads) void coo_digest_kernel(const int32_t *__restrict__ row,
                                                                  const int32_t *__restrict__ col,
                                                                  const float *__restrict__ val, int64_t nnz,
                                                                  unsigned long long *__restrict__ out) {
  unsigned long long h1 = 0, h2 = 0;
  const int64_t tid = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x, nthreads = (int64_t)gridDim.x * kSpmmThreads;
  if (VEC == 4) {
    const int64_t groups = nnz / 4;
    for (int64_t g = tid; g < groups; g += nthreads) {
      const int4 r = reinterpret_cast<const int4 *>(row)[g];
      const int4 c = reinterpret_cast<const int4 *>(col)[g];
      const float4 v = reinterpret_cast<const float4 *>(val)[g];
      digest_entry(r.x, c.x, v.x, 4 * g, h1, h2);
      digest_entry(r.y, c.y, v.y, 4 * g + 1, h1, h2);
      digest_entry(r.z, c.z, v.z, 4 * g + 2, h1, h2);
      digest_entry(r.w, c.w, v.w, 4 * g + 3, h1, h2);
    }
    for (int64_t i = groups * 4 + tid; i < nnz; i += nthreads) digest_entry(row[i], col[i], val[i], i, h1, h2);
  } else {
    for (int64_t i = tid; i < nnz; i += nthreads) digest_entry(row[i], col[i], val[i], i, h1, h2);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    h1 += __shfl_xor(h1, off, kWave);
    h2 += __shfl_xor(h2, off, kWave);
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    atomicAdd(out, h1);
    atomicAdd(out + 1, h2);
  }
}

struct CooCacheEntry {
  unsigned long long d0 = 0, d1 = 0;
  int64_t nnz = 0;
  int32_t n = 0, m = 0;
  int device = 0;
  uint64_t tick = 0;
  std::shared_ptr<cg_csr> h;
  std::mutex use;  // one product at a time per block: a handle's schedule caches are not re-entrant
};

static std::mutex g_coo_cache_mu;
// Never destroyed: at process exit the kept blocks are left to the driver, like the scratch buffers;
// freeing device memory from a static destructor would race the teardown of the HIP runtime.
static std::vector<std::shared_ptr<CooCacheEntry>> &g_coo_cache = *new std::vector<std::shared_ptr<CooCacheEntry>>();
static uint64_t g_coo_cache_tick = 0;
static int64_t g_coo_cache_hits = 0, g_coo_cache_misses = 0, g_coo_cache_evictions = 0;

static int coo_cache_capacity() {
  const int v = g_tune_coo_cache.load(std::memory_order_relaxed);
  return v == 0 ? 8 : (v < 0 ? 0 : v);
}

static int coo_digest(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz,
                      unsigned long long digest[2], hipStream_t stream) {
  void *d = nullptr;
  CG_TRY(scratch_get(stream, kSlotD, 2 * sizeof(unsigned long long), &d));
  CG_TRY(fill_u32((uint32_t *)d, 4, 0u, stream));
  int64_t blocks = ceil_div64(nnz, kSpmmThreads * 8);
  if (blocks > 4096) blocks = 4096;
  const bool aligned = (((uintptr_t)d_row | (uintptr_t)d_col | (uintptr_t)d_val) & 15) == 0;
  if (aligned)
    coo_digest_kernel<4><<<(unsigned)blocks, kSpmmThreads, 0, stream>>>(d_row, d_col, d_val, nnz, (unsigned long long *)d);
  else
    coo_digest_kernel<1><<<(unsigned)blocks, kSpmmThreads, 0, stream>>>(d_row, d_col, d_val, nnz, (unsigned long long *)d);
  CG_LAUNCH_CHECK();
  CG_HIP(hipMemcpyAsync(digest, d, 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost, stream));
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
  if (nnz > 0x7fffffffLL - 1 || n == 0x7fffffff)
    CG_FAIL(CG_ERR_OVERFLOW, "cg_spmm_coo: nnz=%lld n=%d exceed int32", (long long)nnz, n);
  if (nnz > 0 && (!d_row || !d_col || !d_val)) CG_FAIL(CG_ERR_NULL, "cg_spmm_coo: null sparse operand");
  CG_TRY(check_dense("cg_spmm_coo", d_B, ldb, d_C, ldc, f, m, n));
  if (n == 0) return CG_OK;
  if (nnz > 0 && m == 0) CG_FAIL(CG_ERR_SIZE, "cg_spmm_coo: nnz > 0 with m == 0");
  return spmm_coo_oneshot(d_row, d_col, d_val, nnz, n, m, d_B, ldb, d_C, ldc, f, beta, stream);
}

int cg_spmm_coo_cached(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n,
                       int32_t m, const float *d_B, int64_t ldb, float *d_C, int64_t ldc, int32_t f, float beta,
                       cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  const int capacity = coo_cache_capacity();
  // Keeping a block pays through the column-popularity plan, which is too costly to build per call;
  // the plain schedule is rebuilt on the device for less than the digest costs (measured on 114.6 M
  // entries: rebuild + 0.26 ms, digest and read-back + 0.57 ms; with a plan 34.4 -> 18.6 ms).
  if (nnz <= 0 || n <= 0 || m <= 0 || capacity == 0 || !want_hub(n, nnz, f))
    return cg_spmm_coo(d_row, d_col, d_val, nnz, n, m, d_B, ldb, d_C, ldc, f, beta, stream_);
  if (nnz > 0x7fffffffLL - 1 || n == 0x7fffffff || m == 0x7fffffff)
    CG_FAIL(CG_ERR_OVERFLOW, "cg_spmm_coo_cached: nnz=%lld n=%d m=%d exceed int32", (long long)nnz, n, m);
  if (!d_row || !d_col || !d_val) CG_FAIL(CG_ERR_NULL, "cg_spmm_coo_cached: null sparse operand");
  CG_TRY(check_dense("cg_spmm_coo_cached", d_B, ldb, d_C, ldc, f, m, n));
  int device = 0;
  CG_HIP(hipGetDevice(&device));
  unsigned long long dg[2] = {0, 0};
  CG_TRY(coo_digest(d_row, d_col, d_val, nnz, dg, stream));

  std::shared_ptr<CooCacheEntry> entry;
  {
    std::lock_guard<std::mutex> lock(g_coo_cache_mu);
    for (auto &e : g_coo_cache)
      if (e->d0 == dg[0] && e->d1 == dg[1] && e->nnz == nnz && e->n == n && e->m == m && e->device == device) {
        entry = e;
        e->tick = ++g_coo_cache_tick;
        ++g_coo_cache_hits;
        break;
      }
  }
  if (!entry) {
    // first sighting: the same build as cg_csr_create(CG_CSR_SORTED), which checks the index ranges
    // and the row order the kernels rely on
    std::shared_ptr<cg_csr> h(new (std::nothrow) cg_csr(), [](cg_csr *p) {
      if (!p) return;
      (void)hipDeviceSynchronize();  // products queued on any stream may still read the arrays
      p->fwd.release();
      p->tr.release();
      delete p;
    });
    if (!h) CG_FAIL(CG_ERR_ALLOC, "cg_spmm_coo_cached: host allocation failed");
    CG_TRY(csr_create(h.get(), d_row, d_col, d_val, nnz, n, m, CG_CSR_SORTED, stream));
    entry = std::make_shared<CooCacheEntry>();
    entry->d0 = dg[0];
    entry->d1 = dg[1];
    entry->nnz = nnz;
    entry->n = n;
    entry->m = m;
    entry->device = device;
    entry->h = h;
    std::vector<std::shared_ptr<CooCacheEntry>> evicted;  // released after the lock is dropped
    {
      std::lock_guard<std::mutex> lock(g_coo_cache_mu);
      ++g_coo_cache_misses;
      entry->tick = ++g_coo_cache_tick;
      g_coo_cache.push_back(entry);
      while ((int)g_coo_cache.size() > capacity) {
        size_t oldest = 0;
        for (size_t i = 1; i < g_coo_cache.size(); ++i)
          if (g_coo_cache[i]->tick < g_coo_cache[oldest]->tick) oldest = i;
        evicted.push_back(g_coo_cache[oldest]);
        g_coo_cache.erase(g_coo_cache.begin() + (long)oldest);
        ++g_coo_cache_evictions;
      }
    }
  }
  std::lock_guard<std::mutex> use(entry->use);
  return spmm_side(entry->h->fwd, d_B, ldb, d_C, ldc, f, beta, stream);
}

int cg_coo_cache_clear(void) {
  std::vector<std::shared_ptr<cg::CooCacheEntry>> dropped;
  {
    std::lock_guard<std::mutex> lock(cg::g_coo_cache_mu);
    dropped.swap(cg::g_coo_cache);
  }
  return CG_OK;  // the handles are freed here, as `dropped` goes out of scope
}

int cg_coo_cache_info(int64_t info[4]) {
  if (!info) CG_FAIL(CG_ERR_NULL, "cg_coo_cache_info: info is NULL");
  std::lock_guard<std::mutex> lock(cg::g_coo_cache_mu);
  info[0] = (int64_t)cg::g_coo_cache.size();
  info[1] = cg::g_coo_cache_hits;
  info[2] = cg::g_coo_cache_misses;
  info[3] = cg::g_coo_cache_evictions;
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

int cg_csr_spmm_xw(cg_csr_t *h, int transpose, const float *d_B, int64_t ldb, const float *d_C, int64_t ldc, float beta,
                   const float *d_W, int64_t ldw, float *d_Z, int64_t ldz, int32_t f, int32_t fo, int relu,
                   cg_stream_t stream) {
  using namespace cg;
  if (!h) CG_FAIL(CG_ERR_NULL, "cg_csr_spmm_xw: handle is NULL");
  if (transpose && !h->has_t) CG_FAIL(CG_ERR_NO_TRANSPOSE, "cg_csr_spmm_xw: handle was built without CG_CSR_TRANSPOSE");
  CsrSide &s = transpose ? h->tr : h->fwd;
  if (f <= 0 || fo <= 0) CG_FAIL(CG_ERR_SIZE, "cg_csr_spmm_xw: f=%d fo=%d must be positive", f, fo);
  if (ldb < f || ldw < fo || ldz < fo) CG_FAIL(CG_ERR_SIZE, "cg_csr_spmm_xw: leading dimension too small");
  if (beta != 0.f && (!d_C || ldc < f)) CG_FAIL(d_C ? CG_ERR_SIZE : CG_ERR_NULL, "cg_csr_spmm_xw: beta != 0 needs C");
  if (!d_W || (!d_B && s.cols > 0) || (!d_Z && s.rows > 0)) CG_FAIL(CG_ERR_NULL, "cg_csr_spmm_xw: null dense operand");
  if ((const float *)d_Z == d_B || (beta != 0.f && (const float *)d_Z == d_C))
    CG_FAIL(CG_ERR_ALIAS, "cg_csr_spmm_xw: Z aliases an input");
  DenseOps epi{};
  epi.epi_W = d_W;
  epi.epi_ldw = ldw;
  epi.epi_Z = d_Z;
  epi.epi_ldz = ldz;
  epi.epi_fo = fo;
  epi.epi_relu = relu ? 1 : 0;
  // C is never written on this path
  return spmm_side(s, d_B, ldb, beta != 0.f ? const_cast<float *>(d_C) : nullptr, ldc, f, beta, (hipStream_t)stream, &epi);
}

int cg_tune_set(const char *key, int value) {
  if (!key) CG_FAIL(CG_ERR_NULL, "cg_tune_set: key is NULL");
  if (!strcmp(key, "spmm_seg")) cg::g_tune_seg.store(value);
  else if (!strcmp(key, "spmm_vec")) cg::g_tune_vec.store(value);
  else if (!strcmp(key, "spmm_win")) cg::g_tune_win.store(value);
  else if (!strcmp(key, "spmm_hub")) cg::g_tune_hub.store(value);
  else if (!strcmp(key, "spmm_hub_kb")) cg::g_tune_hub_kb.store(value);
  else if (!strcmp(key, "spmm_hub_groups")) cg::g_tune_hub_groups.store(value);
  else if (!strcmp(key, "spmm_hub_tiers")) cg::g_tune_hub_tiers.store(value);
  else if (!strcmp(key, "spmm_hub_row")) cg::g_tune_hub_row.store(value);
  else if (!strcmp(key, "dense_mfma")) cg::g_tune_dense_mfma.store(value);
  else if (!strcmp(key, "coo_cache_blocks")) cg::g_tune_coo_cache.store(value);
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
  // the plan the last wide product of a side looked up: tiers taken, -1 declined, 0 none so far
  auto last_plan = [](const cg::CsrSide &s) -> int64_t {
    int best = -1;
    for (int i = 0; i < cg::CsrSide::kHubPlans; ++i)
      if (s.hub[i].valid && (best < 0 || s.hub_used[i] > s.hub_used[best])) best = i;
    if (best < 0) return 0;
    return s.hub[best].declined ? -1 : s.hub[best].tiers;
  };
  info[6] = last_plan(h->fwd);
  info[7] = h->has_t ? last_plan(h->tr) : 0;
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
