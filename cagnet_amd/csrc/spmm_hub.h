// Per-handle data of the CSR SpMM (the two sides of a matrix, their schedule caches) and the
// construction of hub plans: columns ranked by reference count, dealt to tiers and XCD groups, the
// entries regrouped by class.  Included by spmm.hip only, after spmm_tables.h.
#pragma once
#include "spmm_panel.h"

namespace cg {

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
    CG_TRY(refuse_under_capture(stream, "building a schedule"));
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
  bool failed = false;    // declined because the build ran out of memory or of int32 range
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
    table_free(vrowptr);
    table_free(colind);
    table_free(val);
    table_free(row_hot);
    vrowptr = colind = nullptr;
    val = nullptr;
    row_hot = nullptr;
    valid = false;
    declined = false;
    failed = false;
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
  bool is_rest = false;  // this side is the rest matrix of a panel plan: its dense part is gone already
  PanelPlan panel;  // plan of the wide products that multiply the dense part out of LDS (spmm_panel.h)
  PanelPlan panel_narrow;  // plan of the narrow products: dense tiles only (spmm_panel_narrow.h)
  static constexpr int kTilePlans = 3;
  PanelPlan tile[kTilePlans];  // plans of spmm_tile_kernel: panels of 256, 512 and 1024 rows (spmm_tile.h)
  bool pinned = false;          // a product on this side was captured into a graph (spmm_entry)
  std::vector<void *> parked;   // tables replaced since then: a captured graph may still read them
  int64_t unpin() {  // the caller has made sure that no captured graph will replay any more
    const int64_t count = (int64_t)parked.size();
    for (void *p : parked) (void)hipFree(p);
    parked.clear();
    pinned = false;
    return count;
  }
  void release() {
    for (void *p : parked) table_free(p);  // inside another side's product these move to that side's list
    parked.clear();
    panel.release();
    panel_narrow.release();
    for (int i = 0; i < kTilePlans; ++i) tile[i].release();
    sched.release();
    for (int i = 0; i < kHubPlans; ++i) hub[i].release();
    table_free(rowptr);
    table_free(colind);
    table_free(val);
    rowptr = colind = nullptr;
    val = nullptr;
  }
};

inline void PanelPlan::release() {
  void *owned[] = {unit_tile, unit_order, unit_qstart, unit_block, dwg_unit, dunit_tile, dunit_block, dhdr, dA, hdr, ent, dslot, split, bcount, unit_row0, rank_row, finish_rows};
  for (void *p : owned)
    table_free(p);
  unit_tile = unit_order = unit_qstart = unit_block = dwg_unit = dunit_tile = dunit_block = dhdr = hdr = dslot = split = bcount = unit_row0 = rank_row = finish_rows = nullptr;
  nfinish = 0;
  ent = nullptr;
  dA = nullptr;
  if (rest) {
    rest->release();
    delete rest;
    rest = nullptr;
  }
  valid = declined = failed = false;
  covered = dcovered = nrec = 0;
  ntiles = nunits = nsplit = ndtiles = ndunits = ndwg = nblocks = 0;
}

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
  CG_TRY(refuse_under_capture(stream, "building a hub plan"));
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
      // (the rest matrix of a panel plan has lost its dense tiles to that plan: what its popular columns still
      // hold pays from a smaller share on: Reddit shape, rest of 22.8 M entries, 7.6 -> 7.0 ms with a plan)
      if (may_decline && (double)sums[0] < (s.is_rest ? kHubMinHotFractionRest : kHubMinHotFraction) * (double)nnz) {
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

}  // namespace cg
