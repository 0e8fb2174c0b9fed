// Host side of the panel plan (kernels and the plan's layout: spmm_panel.h): construction on the
// device, and the launch of a product's panel part.  Included by spmm.hip after spmm_hub.h.
#pragma once
#include "spmm_hub.h"

namespace cg {

constexpr int64_t kPanelMaxTiles = (int64_t)1 << 26;  // (panel, column block) pairs whose entries are counted
constexpr double kPanelMinCoverage = 0.5;             // share of the entries the active tiles must hold: measured
                                                      // 0.80 (232,965 vertices, 492 entries per row) 17.1 -> 12.6 ms,
                                                      // 0.42 (R-MAT scale 20, 31 per row) 8.0 -> 9.0 ms at f = 602
constexpr int32_t kPanelDefaultEmin = 64;             // entries a 128 x 32 tile needs to be staged: twice the
                                                      // 32 gathers its staging costs
constexpr int32_t kPanelDefaultCols = 131072;         // ranked columns that can be part of a tile
constexpr int32_t kPanelDefaultUnit = 65536;          // entries after which a panel's tiles start a new unit

struct DevTemps {  // device temporaries of a plan build, freed when the build ends
  std::vector<void *> p;
  ~DevTemps() {
    for (void *q : p)
      if (q) (void)hipFree(q);
  }
  int alloc(void **out, size_t bytes) {
    CG_TRY(dev_alloc(out, bytes));
    p.push_back(*out);
    return CG_OK;
  }
};

static int side_max_degree(CsrSide &s, hipStream_t stream);  // spmm.hip

// Is the panel kernel instantiated for this width, and is the product large enough to consider a plan?
static bool panel_width_ok(int32_t f) { return f >= kPanelMinF && f <= kPanelMaxF && f % 2 == 0; }
static bool want_panel(const CsrSide &s, int32_t f) {
  const int t = g_tune_panel.load(std::memory_order_relaxed);
  if (t < 0 || !panel_width_ok(f) || s.rows == 0 || s.nnz == 0) return false;
  if (t > 0) return true;
  return s.nnz / s.rows >= 8 && (double)s.nnz * f >= 3e9;
}

static int alloc_sort_buffers(DevTemps &tmp, SortBuffers &buf, int64_t count) {
  for (int i = 0; i < 2; ++i) {
    CG_TRY(tmp.alloc((void **)&buf.key_a[i], (size_t)count * 4));
    CG_TRY(tmp.alloc((void **)&buf.key_b[i], (size_t)count * 4));
    CG_TRY(tmp.alloc((void **)&buf.payload[i], (size_t)count * 4));
  }
  return CG_OK;
}

// may_decline: leave the plan empty (pp.declined) when the active tiles hold too few of the entries.
static int build_panel(CsrSide &s, PanelPlan &pp, int32_t emin, int32_t hot_req, int32_t unit_entries, bool may_decline,
                       hipStream_t stream) {
  CG_TRY(refuse_under_capture(stream, "building a panel plan"));
  CG_HIP(hipStreamSynchronize(stream));
  pp.release();
  pp.emin = emin;
  pp.hot_cols = hot_req;
  pp.unit_entries = unit_entries;
  const int64_t nnz = s.nnz;
  const int32_t n = s.rows, m = s.cols;
  auto decline = [&]() {
    pp.release();
    pp.emin = emin;
    pp.hot_cols = hot_req;
    pp.unit_entries = unit_entries;
    pp.declined = true;
    pp.valid = true;
    return CG_OK;
  };
  const int32_t hot = (hot_req < m ? hot_req : m) / kPanelCols * kPanelCols;
  if (hot < kPanelCols || n < 1 || nnz < 1) return decline();
  const int32_t nkb = hot / kPanelCols;
  int64_t npanels = ceil_div64(n, kPanelRows);
  if (npanels > kPanelMaxTiles / nkb) npanels = kPanelMaxTiles / nkb;  // rows are ranked: the panels left out are the sparsest
  if (npanels < 1) return decline();
  const int32_t prows = (int32_t)(npanels * kPanelRows < n ? npanels * kPanelRows : n);
  const int64_t tiles = npanels * nkb;
  const unsigned gn = (unsigned)ceil_div64(n, kSpmmThreads), gm = (unsigned)ceil_div64(m, kSpmmThreads);
  const unsigned ge = (unsigned)ceil_div64(nnz, kSpmmThreads), gt = (unsigned)ceil_div64(tiles + 1, kSpmmThreads);
  DevTemps tmp;

  // 1. rows ranked by descending degree, columns by descending entry count (ties: by index)
  int32_t *row_rank = nullptr, *col_rank = nullptr;
  CG_TRY(tmp.alloc((void **)&row_rank, (size_t)n * 4));
  CG_TRY(tmp.alloc((void **)&col_rank, (size_t)m * 4));
  int32_t *qcol = nullptr;  // row of B of every ranked hot column
  CG_TRY(tmp.alloc((void **)&qcol, (size_t)hot * 4));
  {
    DevTemps t2;
    SortBuffers buf;
    CG_TRY(alloc_sort_buffers(t2, buf, n));
    panel_degree_key_kernel<<<gn, kSpmmThreads, 0, stream>>>(s.rowptr, n, s.max_degree, buf.key_a[0], buf.payload[0]);
    CG_LAUNCH_CHECK();
    CG_TRY(fill_u32((uint32_t *)buf.key_b[0], n, 0u, stream));
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, n, bits_for(s.max_degree + 1), 0, &set, stream));
    panel_invert_kernel<<<gn, kSpmmThreads, 0, stream>>>(buf.payload[set], n, row_rank);
    CG_LAUNCH_CHECK();
    CG_HIP(hipStreamSynchronize(stream));
  }
  {
    DevTemps t2;
    SortBuffers buf;
    uint32_t *count = nullptr;
    CG_TRY(t2.alloc((void **)&count, (size_t)m * 4));
    CG_TRY(alloc_sort_buffers(t2, buf, m));
    CG_TRY(fill_u32(count, m, 0u, stream));
    panel_col_count_kernel<<<ge, kSpmmThreads, 0, stream>>>(s.colind, nnz, count);
    CG_LAUNCH_CHECK();
    const uint32_t maxcount = (uint32_t)(nnz < 0x7ffffffeLL ? nnz : 0x7ffffffeLL);
    panel_count_key_kernel<<<gm, kSpmmThreads, 0, stream>>>(count, m, maxcount, buf.key_a[0], buf.payload[0]);
    CG_LAUNCH_CHECK();
    CG_TRY(fill_u32((uint32_t *)buf.key_b[0], m, 0u, stream));
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, m, bits_for((int32_t)maxcount + 1), 0, &set, stream));
    panel_invert_kernel<<<gm, kSpmmThreads, 0, stream>>>(buf.payload[set], m, col_rank);
    CG_LAUNCH_CHECK();
    CG_HIP(hipMemcpyAsync(qcol, buf.payload[set], (size_t)hot * 4, hipMemcpyDeviceToDevice, stream));
    CG_HIP(hipStreamSynchronize(stream));
  }

  // 2. entries per tile; active tiles = those with at least emin entries
  int32_t *erow = nullptr;
  uint32_t *tcount = nullptr, *tindex = nullptr, *kept = nullptr, *d_tot = nullptr;
  CG_TRY(tmp.alloc((void **)&erow, (size_t)nnz * 4));
  CG_TRY(tmp.alloc((void **)&tcount, (size_t)(tiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&tindex, (size_t)(tiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&kept, (size_t)(tiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&d_tot, 2 * 4));
  panel_expand_rows_kernel<<<(unsigned)ceil_div64((int64_t)n * kWave, kSpmmThreads), kSpmmThreads, 0, stream>>>(s.rowptr, n, erow);
  CG_LAUNCH_CHECK();
  CG_TRY(fill_u32(tcount, tiles + 1, 0u, stream));
  panel_tile_count_kernel<<<ge, kSpmmThreads, 0, stream>>>(erow, s.colind, nnz, row_rank, col_rank, prows, hot, nkb, tcount);
  CG_LAUNCH_CHECK();
  panel_tile_select_kernel<<<gt, kSpmmThreads, 0, stream>>>(tcount, tiles, (uint32_t)emin, tindex, kept);
  CG_LAUNCH_CHECK();
  CG_TRY(exclusive_scan_u32(tindex, tindex, tiles + 1, d_tot + 0, stream));
  CG_TRY(exclusive_scan_u32(kept, kept, tiles + 1, d_tot + 1, stream));
  uint32_t tot[2] = {0, 0};
  CG_HIP(hipMemcpyAsync(tot, d_tot, sizeof(tot), hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  const int64_t ntiles = tot[0], covered = tot[1];
  if (ntiles == 0 || covered == 0 || (may_decline && (double)covered < kPanelMinCoverage * (double)nnz)) return decline();
  if (ntiles * kPanelWaves + 1 > 0x7fffffffLL) return decline();

  // 3. tables of the active tiles
  int32_t *tile_panel = nullptr, *tile_kb = nullptr, *tile_wptr = nullptr;
  CG_TRY(tmp.alloc((void **)&tile_kb, (size_t)ntiles * 4));
  CG_TRY(tmp.alloc((void **)&tile_panel, (size_t)ntiles * 4));
  panel_tile_tables_kernel<<<gt, kSpmmThreads, 0, stream>>>(tcount, tindex, tiles, (uint32_t)emin, nkb, tile_kb, tile_panel);
  CG_LAUNCH_CHECK();

  // 4. one stable sort puts the covered entries first, by (tile, wave, slot), and leaves the others
  //    behind them in (row, col) order: those are the rest matrix
  const int64_t nrest = nnz - covered;
  pp.rest = new (std::nothrow) CsrSide();
  if (!pp.rest) CG_FAIL(CG_ERR_ALLOC, "panel plan: host allocation failed");
  CsrSide &rest = *pp.rest;
  rest.is_rest = true;
  rest.rows = n;
  rest.cols = m;
  rest.nnz = nrest;
  CG_TRY(dev_alloc((void **)&rest.rowptr, (size_t)(n + 1) * 4));
  CG_TRY(dev_alloc((void **)&rest.colind, (size_t)nrest * 4));
  CG_TRY(dev_alloc((void **)&rest.val, (size_t)nrest * 4));
  CG_TRY(dev_alloc((void **)&pp.ent, (size_t)covered * 8));
  CG_TRY(tmp.alloc((void **)&tile_wptr, (size_t)(ntiles * kPanelWaves + 1) * 4));
  CG_TRY(dev_alloc((void **)&pp.hdr, (size_t)ntiles * kPanelWaves * 16));
  {
    DevTemps t2;
    SortBuffers buf;
    int32_t *rest_row = nullptr;
    CG_TRY(alloc_sort_buffers(t2, buf, nnz));
    CG_TRY(t2.alloc((void **)&rest_row, (size_t)(nrest > 0 ? nrest : 1) * 4));
    const int32_t sentinel = (int32_t)(ntiles * kPanelWaves);
    panel_entry_key_kernel<<<ge, kSpmmThreads, 0, stream>>>(erow, s.colind, nnz, row_rank, col_rank, prows, hot, nkb, tcount,
                                                            tindex, (uint32_t)emin, sentinel, buf.key_a[0], buf.key_b[0],
                                                            buf.payload[0]);
    CG_LAUNCH_CHECK();
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, nnz, bits_for(sentinel + 1), bits_for(kPanelSlots), &set, stream));
    panel_entry_finish_kernel<<<ge, kSpmmThreads, 0, stream>>>(buf.key_b[set], buf.payload[set], nnz, covered, erow, s.colind,
                                                               s.val, col_rank, pp.ent, rest_row, rest.colind, rest.val);
    CG_LAUNCH_CHECK();
    CG_TRY(launch_rowptr(buf.key_a[set], covered, sentinel, tile_wptr, stream));
    panel_hdr_kernel<<<(unsigned)ceil_div64(ntiles * kPanelWaves, kSpmmThreads), kSpmmThreads, 0, stream>>>(
        tile_kb, tile_wptr, qcol, ntiles, (int4 *)pp.hdr);
    CG_LAUNCH_CHECK();
    CG_TRY(launch_rowptr(rest_row, nrest, n, rest.rowptr, stream));
    CG_HIP(hipStreamSynchronize(stream));
  }
  CG_TRY(side_max_degree(rest, stream));

  // 5. units: runs of tiles of one panel with about unit_entries entries, heaviest first at launch
  std::vector<int32_t> h_panel((size_t)ntiles), h_base((size_t)ntiles + 1);
  {
    // entries of active tile k = difference of the scanned kept[] at its all-tile index; read them compacted
    // through the (tile, wave) table instead: tile_wptr[16 k] is the first record of tile k
    std::vector<int32_t> h_wptr((size_t)ntiles * kPanelWaves + 1);
    CG_HIP(hipMemcpyAsync(h_wptr.data(), tile_wptr, h_wptr.size() * 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipMemcpyAsync(h_panel.data(), tile_panel, (size_t)ntiles * 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipStreamSynchronize(stream));
    for (int64_t k = 0; k <= ntiles; ++k) h_base[(size_t)k] = h_wptr[(size_t)k * kPanelWaves];
  }
  std::vector<int32_t> unit_tile, split, panel_unit((size_t)npanels, -1);
  std::vector<int64_t> unit_size;
  unit_tile.push_back(0);
  int64_t in_unit = 0;
  for (int64_t k = 0; k < ntiles; ++k) {
    const int64_t e = (int64_t)h_base[(size_t)k + 1] - h_base[(size_t)k];
    const bool new_panel = k > 0 && h_panel[(size_t)k] != h_panel[(size_t)k - 1];
    if (k > unit_tile.back() && (new_panel || in_unit + e > unit_entries)) {
      unit_size.push_back(in_unit);
      unit_tile.push_back((int32_t)k);
      in_unit = 0;
    }
    in_unit += e;
  }
  unit_size.push_back(in_unit);
  unit_tile.push_back((int32_t)ntiles);
  const int32_t nunits = (int32_t)unit_size.size();
  for (int32_t u = 0; u < nunits;) {  // units of one panel are consecutive
    const int32_t panel = h_panel[(size_t)unit_tile[(size_t)u]];
    int32_t v = u + 1;
    while (v < nunits && h_panel[(size_t)unit_tile[(size_t)v]] == panel) ++v;
    panel_unit[(size_t)panel] = u;
    if (v - u > 1) {
      split.push_back(u);
      split.push_back(v - u);
    }
    u = v;
  }
  std::vector<int32_t> order((size_t)nunits);
  for (int32_t u = 0; u < nunits; ++u) order[(size_t)u] = u;
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return unit_size[(size_t)a] > unit_size[(size_t)b]; });
  int32_t *d_panel_unit = nullptr;
  CG_TRY(tmp.alloc((void **)&d_panel_unit, (size_t)npanels * 4));
  CG_TRY(dev_alloc((void **)&pp.unit_tile, (size_t)(nunits + 1) * 4));
  CG_TRY(dev_alloc((void **)&pp.unit_order, (size_t)nunits * 4));
  CG_TRY(dev_alloc((void **)&pp.dslot, (size_t)n * 4));
  CG_HIP(hipMemcpyAsync(pp.unit_tile, unit_tile.data(), (size_t)(nunits + 1) * 4, hipMemcpyHostToDevice, stream));
  CG_HIP(hipMemcpyAsync(pp.unit_order, order.data(), (size_t)nunits * 4, hipMemcpyHostToDevice, stream));
  CG_HIP(hipMemcpyAsync(d_panel_unit, panel_unit.data(), (size_t)npanels * 4, hipMemcpyHostToDevice, stream));
  if (!split.empty()) {
    CG_TRY(dev_alloc((void **)&pp.split, split.size() * 4));
    CG_HIP(hipMemcpyAsync(pp.split, split.data(), split.size() * 4, hipMemcpyHostToDevice, stream));
  }
  panel_dslot_kernel<<<gn, kSpmmThreads, 0, stream>>>(row_rank, n, d_panel_unit, (int32_t)npanels, pp.dslot);
  CG_LAUNCH_CHECK();
  CG_HIP(hipStreamSynchronize(stream));
  pp.covered = covered;
  pp.ntiles = (int32_t)ntiles;
  pp.nunits = nunits;
  pp.nsplit = (int32_t)(split.size() / 2);
  pp.hot_cols = hot_req;
  pp.valid = true;
  return CG_OK;
}

// The panel part of C = A B: partial rows of every row that has entries in active tiles, in *P
// (row r: P + dslot[r] * f).  P is stream scratch and stays valid until the next panel product on `stream`.
static int launch_panel(const PanelPlan &pp, const float *B, int64_t ldb, int32_t f, float **P_out, hipStream_t stream) {
  const int chunks = (f / 2 + kWave - 1) / kWave;
  const size_t rs = ((size_t)f * 4 + 15) & ~(size_t)15;
  const size_t lds = 2 * (size_t)kPanelCols * rs;
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotE, (size_t)pp.nunits * kPanelRows * f * sizeof(float), &p));
  float *P = (float *)p;
  int dev = 0;
  CG_HIP(hipGetDevice(&dev));
  {
    ProfScope prof("spmm_panel", f, stream);
#define CG_PANEL(CH)                                                                                                  \
  case CH: {                                                                                                          \
    static std::atomic<uint64_t> attr_set{0}; /* one bit per device: the LDS size of this kernel has been raised */   \
    if (dev < 64 && !(attr_set.load() >> dev & 1)) {                                                                  \
      CG_HIP(hipFuncSetAttribute((const void *)spmm_panel_kernel<CH>, hipFuncAttributeMaxDynamicSharedMemorySize,     \
                                 (int)(2 * (size_t)kPanelCols * ((kPanelMaxF * 4 + 15) & ~15))));                     \
      attr_set.fetch_or((uint64_t)1 << dev);                                                                          \
    } else if (dev >= 64) {                                                                                           \
      CG_HIP(hipFuncSetAttribute((const void *)spmm_panel_kernel<CH>, hipFuncAttributeMaxDynamicSharedMemorySize,     \
                                 (int)lds));                                                                          \
    }                                                                                                                 \
    spmm_panel_kernel<CH><<<(unsigned)pp.nunits, kPanelThreads, lds, stream>>>(pp.unit_tile, pp.unit_order, pp.hdr, pp.ent, B, \
                                                                               ldb, P, f);                                 \
  } break;
    switch (chunks) {
      CG_PANEL(3)
      CG_PANEL(4)
      CG_PANEL(5)
      default:
        CG_FAIL(CG_ERR_UNSUPPORTED, "panel product: no kernel for f=%d", f);
    }
#undef CG_PANEL
    CG_LAUNCH_CHECK();
    if (pp.nsplit > 0) {
      const dim3 grid((unsigned)ceil_div64((int64_t)kPanelRows * f, kSpmmThreads), (unsigned)pp.nsplit);
      panel_reduce_kernel<<<grid, kSpmmThreads, 0, stream>>>(pp.split, P, f);
      CG_LAUNCH_CHECK();
    }
  }
  *P_out = P;
  return CG_OK;
}

}  // namespace cg
