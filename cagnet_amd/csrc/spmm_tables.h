// Host-side tables of the CSR SpMM: tuning knobs, kernel shape selection, device memory for
// tables, the row-segment schedule, the window tables and the kernel launch.  Included by spmm.hip
// only (one translation unit; everything here has internal linkage).
#pragma once
#include "spmm_kernels.h"
#include <atomic>

namespace cg {

// Tuning knobs (cg_tune_set): 0 = built-in choice.
static std::atomic<int> g_tune_seg{0}, g_tune_vec{0}, g_tune_win{0};
static std::atomic<int> g_tune_hub{0}, g_tune_hub_kb{0}, g_tune_hub_groups{0}, g_tune_hub_tiers{0}, g_tune_hub_row{0};
static std::atomic<int> g_test_alloc_fail{0};  // test hook: k > 0 makes the k-th table allocation from now fail once
static std::atomic<int> g_tune_coo_cache_mib{0};  // MiB the kept blocks may hold together: 0 = 32768
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
constexpr double kHubMinHotFractionRest = 0.12; // the same for the rest matrix of a panel plan
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
  if (g_test_alloc_fail.load(std::memory_order_relaxed) > 0 && g_test_alloc_fail.fetch_sub(1) == 1) {
    *p = nullptr;
    CG_FAIL(CG_ERR_ALLOC, "hipMalloc of %zu bytes failed: injected by the test_alloc_fail tuning key", bytes);
  }
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
      table_free(task_row);
      table_free(tbase);
      table_free(pbase);
      table_free(multi_rows);
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
      table_free(task_start);
      table_free(task_dst);
      table_free(wstart);
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

}  // namespace cg
