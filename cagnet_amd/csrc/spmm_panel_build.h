// Host side of the panel plan (kernels and the plan's layout: spmm_panel.h): construction on the
// device, and the launch of a product's panel part.  Included by spmm.hip after spmm_hub.h.
#pragma once
#include "spmm_hub.h"
#include "spmm_tile.h"

namespace cg {

constexpr double kPanelMinReuse = 0.5;                // share of the entries that must sit in (panel, column) pairs of at
                                                      // least two, i.e. use a staged row of B more than once: measured at
                                                      // f = 602: 0.88 (232,965 vertices, 492 entries per row) 17.1 -> 8.9 ms,
                                                      // 0.54 (R-MAT scale 20, 31 per row) 7.80 -> 7.69 ms, 0.27 (14,249,639
                                                      // vertices, 16 per row, f = 300) 42.8 -> 45.5 ms
constexpr int32_t kPanelDefaultEmin = 1;              // entries a 128 x 32 tile needs to be staged: every tile is (a tile of
                                                      // columns with one entry each costs what the row-wise kernels' gathers
                                                      // cost, and nothing is left for them to do): 64 -> 1 10.2 -> 8.9 ms
constexpr int32_t kPanelDefaultCols = 1 << 30;        // column ranks of a panel that can be part of a tile: all of them
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
  if (g_tune_strict.load(std::memory_order_relaxed) > 0) return false;  // its dense tiles multiply zeros, its records are padded
  if (t > 0) return true;
  // Below about 8e8 multiply-adds the plan's fixed costs (a block of partial rows per unit, few units per compute
  // unit) outweigh what it saves: blocks of a 4 x 4 grid over 232,965 vertices at f = 602, plan against row-wise
  // kernels: 0.6 M entries 0.29 / 0.30 ms, 1.6 M 0.41 / 0.54, 1.7 M 0.48 / 0.58, 5.4 M 0.87 / 1.17 and 0.87 / 1.29,
  // 12.5 M 1.28 / 2.02, 29.4 M 2.07 / 4.31 ms.
  return s.nnz / s.rows >= 8 && (double)s.nnz * f >= 8e8;
}

// Tile plans (spmm_tile_kernel): the panel height goes by the width of the product.
//   geometry 0: panels of 256 rows, tiles of 64 columns: widths above 128, in slices of up to 316 columns
//   geometry 1: 512 x 128: widths 65 .. 128          geometry 2: 1024 x 256: widths up to 64
static int tile_geometry(int32_t f) { return f <= 64 ? 2 : f <= 128 ? 1 : 0; }
static bool panel_width_ok(int32_t f);
// Measured, tile plan against the library's other kernels (ms; 232,965 vertices with 492 entries per row | R-MAT
// scale 20 with 31 | 14,249,639 vertices with 16):
//   f = 1000  17.0 / 29.7 | 11.5 / 14.0        f = 700  12.6 / 19.6 | 8.2 / 9.5         f = 602  10.6 / 8.2 | 6.7 / 6.1
//   f = 300   5.4 / 5.8 | 3.3 / 4.1 | 35.8 / 42.9          f = 256  4.3 / 6.4 | 2.7 / 3.4          f = 128  2.5 / 3.3 | 1.4 / 1.8
//   f = 64    2.1 / 1.4 | 0.90 / 1.14 | 7.5 / 10.7         f = 48   2.1 / 1.5         f = 24   - | - | 6.5 / 5.1        f = 16  2.0 / 0.70 | 0.81 / 0.39
// So: every width from 65 on except those where the panel plan with its matrix-core tiles is in use (even 318..636,
// where two column slices visit every record twice), and 48..64 on matrices of under 64 entries per row (denser ones
// have the narrow plan's matrix-core tiles).  Products under 8e8 multiply-adds or 8 entries per row stay row-wise.
static bool want_tile(const CsrSide &s, int32_t f, bool after_panel) {
  const int t = g_tune_tile.load(std::memory_order_relaxed);
  if (t < 0 || s.rows == 0 || s.nnz == 0 || s.is_rest || f < 1) return false;
  if (t > 0) return !after_panel;
  if (s.nnz / s.rows < 8 || (double)s.nnz * f < 8e8) return false;
  const bool panel_first = panel_width_ok(f) && f > 316 && g_tune_panel.load(std::memory_order_relaxed) >= 0 &&
                           g_tune_strict.load(std::memory_order_relaxed) <= 0;
  if (panel_first != after_panel) return false;
  if (after_panel) return s.panel.valid && s.panel.declined;  // the panel plan looked at the matrix and stood back
  if (f >= 65) return true;
  return f >= 48 && s.nnz / s.rows < 64;
}

static int alloc_sort_buffers(DevTemps &tmp, SortBuffers &buf, int64_t count) {
  for (int i = 0; i < 2; ++i) {
    CG_TRY(tmp.alloc((void **)&buf.key_a[i], (size_t)count * 4));
    CG_TRY(tmp.alloc((void **)&buf.key_b[i], (size_t)count * 4));
    CG_TRY(tmp.alloc((void **)&buf.payload[i], (size_t)count * 4));
  }
  return CG_OK;
}

constexpr int32_t kXcdQueues = 8;                       // queues of units, one per XCD (spmm_panel_kernel)
constexpr int32_t kPanelDefaultDmin = 768;             // entries from which a 128 x 32 tile is stored whole and multiplied
                                                       // on the matrix cores (3/16 full; 640 / 768 / 896 / 1024: 8.93 / 8.82 /
                                                       // 9.43 / 8.92 ms at 232,965 vertices, f = 602); negative tuning value: never

// may_decline: leave the plan empty (pp.declined) when the tiles hold too few of the entries.
// *collision: two entries of one (row, column) pair fell into a dense tile; the plan is unusable.
// dwg: workgroups of the dense-tile kernel (each takes an equal share of the dense tiles).
static int build_panel_once(CsrSide &s, PanelPlan &pp, int32_t emin, int32_t hot_req, int32_t unit_entries, int32_t dmin,
                            int32_t dwg, bool share_order, bool may_decline, double min_coverage, double min_reuse,
                            bool *collision, hipStream_t stream, int32_t PR = kPanelRows, int32_t TC = kPanelCols,
                            bool padded = true) {
  *collision = false;
  if (PR % kPanelWaves != 0 || TC % kPanelWaves != 0 || TC > 256 || PR / kPanelWaves > 128)
    CG_FAIL(CG_ERR_UNSUPPORTED, "panel plan: panels of %d rows and tiles of %d columns are not supported", PR, TC);
  if (PR != kPanelRows || TC != kPanelCols) dmin = 0;  // the matrix-core kernels take 128 x 32 tiles only
  const int32_t HS = TC / kPanelWaves + 2;            // ints of a (tile, wave) header
  const int64_t nnz = s.nnz;
  const int32_t n = s.rows, m = s.cols;
  auto decline = [&]() {
    pp.release();
    pp.declined = true;
    pp.valid = true;
    return CG_OK;
  };
  // column ranks of a panel that can be part of a tile: whole blocks; a panel's last block may be partly empty
  const int32_t hot = (int32_t)(ceil_div64(hot_req < m ? hot_req : m, TC) * TC);
  if (hot < TC || n < 1 || nnz < 1) return decline();
  const int64_t npanels = ceil_div64(n, PR);
  const int32_t prows = n;  // every row is in a panel
  int64_t tiles = 0;        // all (panel, block) tiles, numbered panel by panel (tbase)
  const unsigned gn = (unsigned)ceil_div64(n, kSpmmThreads);
  const unsigned ge = (unsigned)ceil_div64(nnz, kSpmmThreads);
  DevTemps tmp;

  // 1. rows ranked by descending degree (ties: by index)
  int32_t *row_rank = nullptr;
  CG_TRY(tmp.alloc((void **)&row_rank, (size_t)n * 4));
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
    CG_TRY(dev_alloc((void **)&pp.rank_row, (size_t)n * 4));
    CG_HIP(hipMemcpyAsync(pp.rank_row, buf.payload[set], (size_t)n * 4, hipMemcpyDeviceToDevice, stream));
    CG_HIP(hipStreamSynchronize(stream));
  }

  const bool share = share_order && m < (1 << 30);
  int32_t *col_rank = nullptr;  // columns ranked by their entries in the whole matrix (step 1a, inside 1b)

  // 1b. columns ranked inside every panel by the entries they have there: the entries sorted by (panel, column),
  //     the runs of that order (= pairs) sorted by (panel, descending length).  ecr[entry] = rank of its column
  //     in its panel; the sorted pairs stay for the tile headers.
  int32_t *erow = nullptr, *ecr = nullptr, *pstart = nullptr, *pair_col = nullptr, *spanel = nullptr, *spair = nullptr;
  uint32_t *tcount = nullptr;  // entries per (panel, block) tile
  int32_t *tbase = nullptr;    // [npanels + 1] first tile of a panel
  int64_t npairs = 0;
  CG_TRY(tmp.alloc((void **)&tbase, (size_t)(npanels + 1) * 4));
  CG_TRY(tmp.alloc((void **)&erow, (size_t)nnz * 4));
  CG_TRY(tmp.alloc((void **)&ecr, (size_t)nnz * 4));
  CG_TRY(tmp.alloc((void **)&pstart, (size_t)(npanels + 2) * 4));
  panel_expand_rows_kernel<<<(unsigned)ceil_div64((int64_t)n * kWave, kSpmmThreads), kSpmmThreads, 0, stream>>>(s.rowptr, n, erow);
  CG_LAUNCH_CHECK();
  {
    DevTemps t2;
    SortBuffers buf;
    uint32_t *start = nullptr, *runs_before = nullptr, *pair_first = nullptr, *d_np = nullptr;
    int32_t *pair_lr = nullptr;
    CG_TRY(alloc_sort_buffers(t2, buf, nnz));
    CG_TRY(t2.alloc((void **)&start, (size_t)(nnz + 1) * 4));
    CG_TRY(t2.alloc((void **)&runs_before, (size_t)(nnz + 1) * 4));
    CG_TRY(t2.alloc((void **)&d_np, 4));
    panel_pair_key_kernel<<<ge, kSpmmThreads, 0, stream>>>(erow, s.colind, nnz, row_rank, prows, (int32_t)npanels, PR, buf.key_a[0],
                                                           buf.key_b[0], buf.payload[0]);
    CG_LAUNCH_CHECK();
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, nnz, bits_for((int32_t)npanels + 1), bits_for(m), &set, stream));
    const unsigned ge1 = (unsigned)ceil_div64(nnz + 1, kSpmmThreads);
    panel_run_start_kernel<<<ge1, kSpmmThreads, 0, stream>>>(buf.key_a[set], buf.key_b[set], nnz, start);
    CG_LAUNCH_CHECK();
    CG_TRY(exclusive_scan_u32(start, runs_before, nnz + 1, d_np, stream));
    uint32_t h_np = 0;
    CG_HIP(hipMemcpyAsync(&h_np, d_np, 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipStreamSynchronize(stream));
    npairs = h_np;
    CG_TRY(t2.alloc((void **)&pair_first, (size_t)(npairs + 1) * 4));
    CG_TRY(t2.alloc((void **)&pair_lr, (size_t)npairs * 4));
    CG_TRY(tmp.alloc((void **)&pair_col, (size_t)npairs * 4));
    CG_TRY(tmp.alloc((void **)&spanel, (size_t)npairs * 4));
    CG_TRY(tmp.alloc((void **)&spair, (size_t)npairs * 4));
    panel_run_first_kernel<<<ge1, kSpmmThreads, 0, stream>>>(start, runs_before, nnz, pair_first);
    CG_LAUNCH_CHECK();
    CG_TRY(fill_u32(pair_first + npairs, 1, (uint32_t)nnz, stream));
    if (may_decline && min_reuse > 0.0) {
      // A staged row of B pays where it is used more than once: the share of the entries that sit in (panel, column)
      // pairs of at least two decides about the plan before the rest of it is built.
      unsigned long long *d_reuse = nullptr, h_reuse = 0;
      CG_TRY(t2.alloc((void **)&d_reuse, 8));
      CG_HIP(hipMemsetAsync(d_reuse, 0, 8, stream));
      const int64_t want = ceil_div64(npairs, kSpmmThreads);
      panel_pair_reuse_kernel<<<(unsigned)(want < 2048 ? want : 2048), kSpmmThreads, 0, stream>>>(pair_first, npairs, d_reuse);
      CG_LAUNCH_CHECK();
      CG_HIP(hipMemcpyAsync(&h_reuse, d_reuse, 8, hipMemcpyDeviceToHost, stream));
      CG_HIP(hipStreamSynchronize(stream));
      if ((double)h_reuse < min_reuse * (double)nnz) return decline();
    }
    const unsigned gp = (unsigned)ceil_div64(npairs, kSpmmThreads);
    // 1a. columns ranked by their entries in the whole matrix (ties: by index): the order of a panel's columns that
    //     are worth staging
    if (share) {
      DevTemps t3;
      SortBuffers cb;
      uint32_t *count = nullptr;
      CG_TRY(tmp.alloc((void **)&col_rank, (size_t)m * 4));
      CG_TRY(t3.alloc((void **)&count, (size_t)m * 4));
      CG_TRY(alloc_sort_buffers(t3, cb, m));
      CG_TRY(fill_u32(count, m, 0u, stream));
      if (npairs > 0) {
        panel_col_count_kernel<<<gp, kSpmmThreads, 0, stream>>>(pair_first, npairs, buf.key_b[set], count);
        CG_LAUNCH_CHECK();
      }
      const uint32_t maxcount = (uint32_t)(nnz < 0x7ffffffeLL ? nnz : 0x7ffffffeLL);
      const unsigned gm = (unsigned)ceil_div64(m, kSpmmThreads);
      panel_count_key_kernel<<<gm, kSpmmThreads, 0, stream>>>(count, m, maxcount, cb.key_a[0], cb.payload[0]);
      CG_LAUNCH_CHECK();
      CG_TRY(fill_u32((uint32_t *)cb.key_b[0], m, 0u, stream));
      int cset = 0;
      CG_TRY(radix_sort_pairs(cb, m, bits_for((int32_t)maxcount + 1), 0, &cset, stream));
      panel_invert_kernel<<<gm, kSpmmThreads, 0, stream>>>(cb.payload[cset], m, col_rank);
      CG_LAUNCH_CHECK();
      CG_HIP(hipStreamSynchronize(stream));
    }
    {
      DevTemps t3;
      SortBuffers pb;
      CG_TRY(alloc_sort_buffers(t3, pb, npairs));
      const uint32_t cmin = (uint32_t)((emin + TC - 1) / TC);  // a block of such columns reaches emin
      panel_pair_count_key_kernel<<<gp, kSpmmThreads, 0, stream>>>(pair_first, npairs, buf.key_a[set], buf.key_b[set], col_rank, cmin,
                                                                   m, pb.key_a[0], pb.key_b[0], pb.payload[0], pair_col);
      CG_LAUNCH_CHECK();
      int pset = 0;
      CG_TRY(radix_sort_pairs(pb, npairs, bits_for((int32_t)npanels + 1), share ? bits_for(2 * m) : 8, &pset, stream));
      CG_TRY(launch_rowptr(pb.key_a[pset], npairs, (int32_t)npanels + 1, pstart, stream));
      {
        uint32_t *d_tiles = nullptr, h_tiles = 0;
        CG_TRY(t3.alloc((void **)&d_tiles, 4));
        panel_tile_base_kernel<<<(unsigned)ceil_div64(npanels + 1, kSpmmThreads), kSpmmThreads, 0, stream>>>(
            pstart, (int32_t)npanels, hot, TC, (uint32_t *)tbase);
        CG_LAUNCH_CHECK();
        CG_TRY(exclusive_scan_u32((uint32_t *)tbase, (uint32_t *)tbase, npanels + 1, d_tiles, stream));
        CG_HIP(hipMemcpyAsync(&h_tiles, d_tiles, 4, hipMemcpyDeviceToHost, stream));
        CG_HIP(hipStreamSynchronize(stream));
        tiles = h_tiles;
      }
      CG_TRY(tmp.alloc((void **)&tcount, (size_t)(tiles + 1) * 4));
      CG_TRY(fill_u32(tcount, tiles + 1, 0u, stream));
      panel_pair_rank_kernel<<<gp, kSpmmThreads, 0, stream>>>(pb.key_a[pset], pb.payload[pset], npairs, pstart, (int32_t)npanels,
                                                              hot, TC, tbase, pair_first, pair_lr, tcount);
      CG_LAUNCH_CHECK();
      CG_HIP(hipMemcpyAsync(spanel, pb.key_a[pset], (size_t)npairs * 4, hipMemcpyDeviceToDevice, stream));
      CG_HIP(hipMemcpyAsync(spair, pb.payload[pset], (size_t)npairs * 4, hipMemcpyDeviceToDevice, stream));
      CG_HIP(hipStreamSynchronize(stream));
    }
    panel_entry_rank_kernel<<<ge, kSpmmThreads, 0, stream>>>(start, runs_before, buf.payload[set], nnz, pair_lr, ecr);
    CG_LAUNCH_CHECK();
    CG_HIP(hipStreamSynchronize(stream));
  }

  // 2. active tiles = those with emin .. dmin - 1 entries, dense tiles = those with more
  const unsigned gt = (unsigned)ceil_div64(tiles + 1, kSpmmThreads);
  uint32_t *tindex = nullptr, *kept = nullptr, *dindex = nullptr, *dkept = nullptr, *d_tot = nullptr;
  CG_TRY(tmp.alloc((void **)&tindex, (size_t)(tiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&kept, (size_t)(tiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&dindex, (size_t)(tiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&dkept, (size_t)(tiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&d_tot, 5 * 4));
  CG_TRY(fill_u32(d_tot, 5, 0u, stream));
  panel_tile_select_kernel<<<gt, kSpmmThreads, 0, stream>>>(tcount, tiles, (uint32_t)emin, (uint32_t)dmin, tindex, kept, dindex,
                                                           dkept);
  CG_LAUNCH_CHECK();
  CG_TRY(exclusive_scan_u32(tindex, tindex, tiles + 1, d_tot + 0, stream));
  CG_TRY(exclusive_scan_u32(kept, kept, tiles + 1, d_tot + 1, stream));
  CG_TRY(exclusive_scan_u32(dindex, dindex, tiles + 1, d_tot + 2, stream));
  CG_TRY(exclusive_scan_u32(dkept, dkept, tiles + 1, d_tot + 3, stream));
  uint32_t tot[5] = {0, 0, 0, 0, 0};
  CG_HIP(hipMemcpyAsync(tot, d_tot, 4 * 4, hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  const int64_t ntiles = tot[0], covered = tot[1], ndtiles = tot[2], dcovered = tot[3];
  if (ntiles + ndtiles == 0 || covered + dcovered == 0 ||
      (may_decline && (double)(covered + dcovered) < min_coverage * (double)nnz))
    return decline();
  if (ntiles * kPanelWaves * HS + 2 > 0x7fffffffLL || ndtiles * kDenseTileFloats > 0x7fffffffLL * 4) return decline();

  // 3. tables of the active and of the dense tiles; the columns of their places
  int32_t *tile_panel = nullptr, *tile_kb = nullptr, *tile_wptr = nullptr, *dtile_panel = nullptr;
  CG_TRY(tmp.alloc((void **)&tile_panel, (size_t)(ntiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&tile_kb, (size_t)(ntiles + 1) * 4));
  CG_TRY(tmp.alloc((void **)&dtile_panel, (size_t)(ndtiles + 1) * 4));
  panel_tile_tables_kernel<<<gt, kSpmmThreads, 0, stream>>>(tcount, tindex, tiles, (uint32_t)emin, (uint32_t)dmin, 1, tbase,
                                                           (int32_t)npanels, tile_panel, tile_kb);
  CG_LAUNCH_CHECK();
  // (two tiles' worth of zero headers behind the last: spmm_tile_kernel reads headers two tiles ahead without looking)
  CG_TRY(dev_alloc((void **)&pp.hdr, (size_t)(ntiles + 2) * kPanelWaves * HS * 4));
  CG_TRY(fill_u32((uint32_t *)pp.hdr, ntiles * kPanelWaves * HS, 0xffffffffu, stream));
  CG_TRY(fill_u32((uint32_t *)pp.hdr + ntiles * kPanelWaves * HS, 2 * kPanelWaves * HS, 0u, stream));
  if (ndtiles > 0) {
    panel_tile_tables_kernel<<<gt, kSpmmThreads, 0, stream>>>(tcount, dindex, tiles, (uint32_t)emin, (uint32_t)dmin, 2, tbase,
                                                             (int32_t)npanels, dtile_panel, nullptr);
    CG_LAUNCH_CHECK();
    CG_TRY(dev_alloc((void **)&pp.dA, (size_t)ndtiles * kDenseTileFloats * 4));
    CG_TRY(dev_alloc((void **)&pp.dhdr, (size_t)ndtiles * kPanelCols * 4));
    CG_HIP(hipMemsetAsync(pp.dA, 0, (size_t)ndtiles * kDenseTileFloats * 4, stream));
    CG_TRY(fill_u32((uint32_t *)pp.dhdr, ndtiles * kPanelCols, 0xffffffffu, stream));
  }
  panel_pair_hdr_kernel<<<(unsigned)ceil_div64(npairs, kSpmmThreads), kSpmmThreads, 0, stream>>>(
      spanel, spair, npairs, pstart, (int32_t)npanels, hot, tbase, pair_col, tcount, tindex, dindex, (uint32_t)emin, (uint32_t)dmin,
      TC, pp.hdr, pp.dhdr);
  CG_LAUNCH_CHECK();
  if (ndtiles > 0) {
    panel_dense_hdr_fill_kernel<<<(unsigned)ceil_div64(ndtiles * kPanelCols, kSpmmThreads), kSpmmThreads, 0, stream>>>(pp.dhdr,
                                                                                                                     ndtiles);
    CG_LAUNCH_CHECK();
  }

  // 4. one stable sort puts the entries of active tiles first, by (tile, wave, slot), leaves those of no tile
  //    behind them in (row, col) order (the rest matrix) and those of dense tiles, already stored, last
  const int64_t nrest = nnz - covered - dcovered;
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
  CG_TRY(tmp.alloc((void **)&tile_wptr, (size_t)(ntiles * kPanelWaves + 1) * 4));
  {
    DevTemps t2;
    SortBuffers buf;
    int32_t *rest_row = nullptr;
    CG_TRY(alloc_sort_buffers(t2, buf, nnz));
    CG_TRY(t2.alloc((void **)&rest_row, (size_t)(nrest > 0 ? nrest : 1) * 4));
    const int32_t sentinel = (int32_t)(ntiles * kPanelWaves);
    panel_entry_key_kernel<<<ge, kSpmmThreads, 0, stream>>>(erow, ecr, s.val, nnz, row_rank, hot, tbase, tcount,
                                                            tindex, dindex, (uint32_t)emin, (uint32_t)dmin, sentinel, PR, TC,
                                                            buf.key_a[0], buf.key_b[0], buf.payload[0], (uint32_t *)pp.dA,
                                                            d_tot + 4);
    CG_LAUNCH_CHECK();
    int set = 0;
    CG_TRY(radix_sort_pairs(buf, nnz, bits_for(sentinel + 2), bits_for(PR / kPanelWaves), &set, stream));
    uint2 *ent_raw = nullptr;  // the records before padding
    CG_TRY(t2.alloc((void **)&ent_raw, (size_t)(covered > 0 ? covered : 1) * 8));
    if (covered + nrest > 0) {
      panel_entry_finish_kernel<<<(unsigned)ceil_div64(covered + nrest, kSpmmThreads), kSpmmThreads, 0, stream>>>(
          buf.key_b[set], buf.payload[set], covered + nrest, covered, erow, s.colind, s.val, ecr, TC, ent_raw, rest_row,
          rest.colind, rest.val);
      CG_LAUNCH_CHECK();
    }
    CG_TRY(launch_rowptr(buf.key_a[set], covered, sentinel, tile_wptr, stream));
    // runs of odd length get a padding record (spmm_panel_kernel takes the records of a run two at a time)
    if (!padded) {
      if (covered > 0x7fffffffLL) CG_FAIL(CG_ERR_OVERFLOW, "panel plan: records exceed the int32 range");
      pp.nrec = covered;
      CG_TRY(dev_alloc((void **)&pp.ent, (size_t)(covered + kWave) * 8));  // (the tile kernels load 64 records from any start)
      if (covered > 0) CG_HIP(hipMemcpyAsync(pp.ent, ent_raw, (size_t)covered * 8, hipMemcpyDeviceToDevice, stream));
    } else {
      uint32_t *start = nullptr, *runs_before = nullptr, *run_first = nullptr, *padf = nullptr, *shift = nullptr;
      CG_TRY(t2.alloc((void **)&start, (size_t)(covered + 1) * 4));
      CG_TRY(t2.alloc((void **)&runs_before, (size_t)(covered + 1) * 4));
      CG_TRY(t2.alloc((void **)&run_first, (size_t)(covered + 1) * 4));
      CG_TRY(t2.alloc((void **)&padf, (size_t)(covered + 1) * 4));
      CG_TRY(t2.alloc((void **)&shift, (size_t)(covered + 1) * 4));
      const unsigned gc = (unsigned)ceil_div64(covered + 1, kSpmmThreads);
      panel_run_start_kernel<<<gc, kSpmmThreads, 0, stream>>>(buf.key_a[set], buf.key_b[set], covered, start);
      CG_LAUNCH_CHECK();
      CG_TRY(exclusive_scan_u32(start, runs_before, covered + 1, nullptr, stream));
      panel_run_first_kernel<<<gc, kSpmmThreads, 0, stream>>>(start, runs_before, covered, run_first);
      CG_LAUNCH_CHECK();
      panel_run_pad_kernel<<<gc, kSpmmThreads, 0, stream>>>(start, runs_before, run_first, covered, padf);
      CG_LAUNCH_CHECK();
      CG_TRY(exclusive_scan_u32(padf, shift, covered + 1, d_tot + 0, stream));
      uint32_t npad = 0;
      CG_HIP(hipMemcpyAsync(&npad, d_tot + 0, 4, hipMemcpyDeviceToHost, stream));
      CG_HIP(hipStreamSynchronize(stream));
      if (covered + (int64_t)npad > 0x7fffffffLL) CG_FAIL(CG_ERR_OVERFLOW, "panel plan: records exceed the int32 range");
      pp.nrec = covered + npad;
      CG_TRY(dev_alloc((void **)&pp.ent, (size_t)(pp.nrec + kWave) * 8));
      if (covered > 0) {
        panel_pad_write_kernel<<<gc, kSpmmThreads, 0, stream>>>(ent_raw, padf, shift, covered, pp.ent);
        CG_LAUNCH_CHECK();
      }
      panel_pad_wptr_kernel<<<(unsigned)ceil_div64(ntiles * kPanelWaves + 1, kSpmmThreads), kSpmmThreads, 0, stream>>>(
          tile_wptr, ntiles * kPanelWaves + 1, shift);
      CG_LAUNCH_CHECK();
    }
    if (ntiles > 0) {
      panel_hdr_kernel<<<(unsigned)ceil_div64(ntiles * kPanelWaves, kSpmmThreads), kSpmmThreads, 0, stream>>>(tile_wptr, ntiles,
                                                                                                              TC, pp.hdr);
      CG_LAUNCH_CHECK();
    }
    CG_TRY(launch_rowptr(rest_row, nrest, n, rest.rowptr, stream));
    CG_HIP(hipMemcpyAsync(tot + 4, d_tot + 4, 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipStreamSynchronize(stream));
  }
  if (tot[4] != 0) {
    *collision = true;
    return CG_OK;
  }
  CG_TRY(side_max_degree(rest, stream));

  // 5. units: runs of tiles of one panel and one kind, with about unit_entries entries (active tiles) or inside one
  //    workgroup's share (dense tiles); each unit writes one block of 128 partial rows, the blocks of a panel are
  //    consecutive
  std::vector<int32_t> h_panel((size_t)ntiles), h_kb((size_t)ntiles), h_base((size_t)ntiles + 1, 0), h_dpanel((size_t)ndtiles);
  {
    // entries of active tile k: tile_wptr[16 k] is its first record (picked out on the device: a sixteenth to copy)
    int32_t *d_base = nullptr;
    CG_TRY(tmp.alloc((void **)&d_base, (size_t)(ntiles + 1) * 4));
    panel_tile_first_kernel<<<(unsigned)ceil_div64(ntiles + 1, kSpmmThreads), kSpmmThreads, 0, stream>>>(tile_wptr, ntiles + 1, d_base);
    CG_LAUNCH_CHECK();
    CG_HIP(hipMemcpyAsync(h_base.data(), d_base, (size_t)(ntiles + 1) * 4, hipMemcpyDeviceToHost, stream));
    if (ntiles > 0) CG_HIP(hipMemcpyAsync(h_panel.data(), tile_panel, (size_t)ntiles * 4, hipMemcpyDeviceToHost, stream));
    if (ntiles > 0) CG_HIP(hipMemcpyAsync(h_kb.data(), tile_kb, (size_t)ntiles * 4, hipMemcpyDeviceToHost, stream));
    if (ndtiles > 0) CG_HIP(hipMemcpyAsync(h_dpanel.data(), dtile_panel, (size_t)ndtiles * 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipStreamSynchronize(stream));
  }
  struct Unit {
    int32_t panel, t0, t1;
    int64_t weight;
  };
  std::vector<Unit> su, du;  // units of active tiles, of dense tiles; both in panel order
  // with shared column order a unit starts where a panel's block number passes a multiple of this: every 1024 column ranks
  const int32_t kUnitGrid = TC >= 1024 ? 1 : 1024 / TC;
  constexpr int32_t kXcds = kXcdQueues;  // XCDs of the device
  // What a run of tiles costs, in microseconds: a tile with e records 1.50 + 0.0034 e + 8.7e-6 e^2 (fitted to the
  // durations of the 3744 units of the matrix with 232,965 vertices and 492 entries per row at f = 602: 3.4 % off
  // in the median; a tile costs its copies and its barrier whatever it holds, and the waves' records run the more
  // unevenly the more of them a tile has).  Only ratios matter.  A unit is also cut when its cost reaches a cap
  // (below), so that a small matrix still gets balanced work.
  // (Tiles of other shapes go to spmm_tile_kernel, whose waves take a record in about 60 cycles whatever the tile
  // holds: a fixed part per tile and a linear one.)
  const bool legacy_shape = PR == kPanelRows && TC == kPanelCols;
  auto tile_cost = [&](int64_t t) {
    const double e = (double)(h_base[(size_t)t + 1] - h_base[(size_t)t]);
    return legacy_shape ? 1.50 + 0.0034 * e + 8.7e-6 * e * e : 1.50 + 0.0016 * e;
  };
  // A unit is cut at the latest when its cost reaches `cost_cap`: an eighth of a compute unit's share of the whole cost,
  // and at least a third of it within 100 .. 200 us (300 for the tile plans' shapes).  The lower bounds keep the
  // number of blocks of partial rows down on small matrices, which the pass that sums them pays for: a block row of
  // a 4 x 4 grid over 232,965 vertices at f = 602 (9.4 M entries) takes 1.54 / 1.47 / 1.39 / 1.50 / 1.54 ms with units of
  // at most 100 / 150 / 200 / 300 / 400 us; R-MAT scale 20 at f = 64, 128, 256 with 100 us 0.94 / 1.41 / 2.50 ms, with
  // 300 us 0.87 / 1.30 / 2.40 ms.
  double cost_cap = 100.0;
  {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus < 1) {
      (void)hipGetLastError();
      cus = 256;
    }
    double total = 0.0;
    for (int64_t t = 0; t < ntiles; ++t) total += tile_cost(t);
    const int tuned = g_tune_panel_costcap.load(std::memory_order_relaxed);
    const double hi = legacy_shape ? 200.0 : 300.0;
    cost_cap = tuned > 0 ? (double)tuned : std::min(hi, std::max(100.0, total / (3.0 * cus)));
    if (total / (8.0 * cus) > cost_cap) cost_cap = total / (8.0 * cus);
  }
  for (int64_t k = 0; k < ntiles;) {
    int64_t j = k, in_unit = 0;
    double unit_cost = 0.0;
    // a panel of up to one and a half units' records and cost stays whole: its unit is then its only block and
    // writes C itself
    bool whole = k == 0 || h_panel[(size_t)k - 1] != h_panel[(size_t)k];
    if (whole) {
      int64_t pend = k;
      double pcost = 0.0;
      for (; pend < ntiles && h_panel[(size_t)pend] == h_panel[(size_t)k]; ++pend) pcost += tile_cost(pend);
      whole = (int64_t)h_base[(size_t)pend] - h_base[(size_t)k] <= (int64_t)unit_entries + unit_entries / 2 && pcost <= 1.5 * cost_cap;
    }
    while (j < ntiles && h_panel[(size_t)j] == h_panel[(size_t)k]) {
      const int64_t e = (int64_t)h_base[(size_t)j + 1] - h_base[(size_t)j];
      if (whole) {
      } else if (share) {
        if (j > k && (in_unit >= unit_entries / 2 || unit_cost >= cost_cap) &&
            (h_kb[(size_t)j] / kUnitGrid != h_kb[(size_t)j - 1] / kUnitGrid || in_unit >= 2 * (int64_t)unit_entries))
          break;  // (a stretch of very full tiles is cut inside the grid as well)
      } else if (j > k && (in_unit + e > unit_entries || unit_cost >= cost_cap)) {
        break;
      }
      in_unit += e;
      unit_cost += tile_cost(j);
      ++j;
    }
    su.push_back(Unit{h_panel[(size_t)k], (int32_t)k, (int32_t)j, in_unit});
    k = j;
  }
  const int32_t ndwg = (int32_t)(ndtiles < dwg ? ndtiles : dwg);
  std::vector<int32_t> dwg_unit((size_t)ndwg + 1, 0);
  for (int64_t k = 0, w = 0; k < ndtiles;) {
    while ((int64_t)ndtiles * (w + 1) / ndwg <= k) dwg_unit[(size_t)++w] = (int32_t)du.size();  // share that holds tile k
    const int64_t share_end = (int64_t)ndtiles * (w + 1) / ndwg;
    int64_t j = k;
    while (j < ndtiles && h_dpanel[(size_t)j] == h_dpanel[(size_t)k] && j < share_end) ++j;
    du.push_back(Unit{h_dpanel[(size_t)k], (int32_t)k, (int32_t)j, j - k});
    k = j;
  }
  if (ndwg > 0) dwg_unit[(size_t)ndwg] = (int32_t)du.size();
  const int32_t nunits = (int32_t)su.size(), ndunits = (int32_t)du.size();
  std::vector<int32_t> unit_tile((size_t)nunits + 1, 0), unit_block((size_t)nunits), dunit_tile((size_t)ndunits + 1, 0),
      dunit_block((size_t)ndunits), split, panel_unit((size_t)npanels, -1), bcount, unit_row0((size_t)nunits, -1);
  int32_t nblocks = 0;
  for (size_t a = 0, b = 0; a < su.size() || b < du.size();) {  // merge by panel: dense units first, then the others
    const int32_t pa = a < su.size() ? su[a].panel : 0x7fffffff, pb = b < du.size() ? du[b].panel : 0x7fffffff;
    const int32_t panel = pa < pb ? pa : pb;
    const int32_t first = nblocks;
    for (; b < du.size() && du[b].panel == panel; ++b) dunit_block[b] = nblocks++;
    for (; a < su.size() && su[a].panel == panel; ++a) unit_block[a] = nblocks++;
    panel_unit[(size_t)panel] = first;
    bcount.resize((size_t)nblocks, 0);
    bcount[(size_t)first] = nblocks - first;
    if (nblocks - first == 1 && a > 0 && su[a - 1].panel == panel) {  // one block, and a staged unit's: it can write C itself
      bcount[(size_t)first] = -1;
      unit_row0[a - 1] = panel * PR;
    }
    if (nblocks - first > 1) {
      split.push_back(first);
      split.push_back(nblocks - first);
    }
  }
  for (int32_t u = 0; u < nunits; ++u) unit_tile[(size_t)u + 1] = su[(size_t)u].t1;
  for (int32_t u = 0; u < ndunits; ++u) dunit_tile[(size_t)u + 1] = du[(size_t)u].t1;
  std::vector<int32_t> order((size_t)nunits);
  for (int32_t u = 0; u < nunits; ++u) order[(size_t)u] = u;
  // the launch order goes by the units' costs (a unit's tiles taken as alike)
  auto cost = [&](int32_t u) {
    const double T = (double)(su[(size_t)u].t1 - su[(size_t)u].t0), R = (double)su[(size_t)u].weight;
    if (!legacy_shape) return 1.50 * T + 0.0016 * R;
    return T > 0.0 ? 1.50 * T + 0.0034 * R + 8.7e-6 * R * R / T : 0.0;
  };
  // The units go into eight queues, one per XCD; a workgroup takes the next unit of the queue of the XCD it runs on
  // (spmm_panel_kernel: panel_take_unit).
  std::vector<int32_t> queue[kXcds];
  if (!share) {
    std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return cost(a) > cost(b); });
    for (int32_t i = 0; i < nunits; ++i) queue[i % kXcds].push_back(order[(size_t)i]);
  } else {
    // Units that start at the same block number in neighbouring panels walk nearly the same rows of B: groups of as
    // many of them as an XCD has compute units sit in one queue one behind the other, so that they run on that XCD
    // together and one copy from memory serves the whole group out of its L2.  The groups are dealt out in rounds
    // of one per queue, and within a round the costliest group goes to the queue that has been given the least so far.
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus < kXcds) {
      (void)hipGetLastError();
      cus = 256;
    }
    const int32_t gsize = cus / kXcds;
    std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) {
      const int32_t ka = h_kb[(size_t)su[(size_t)a].t0] / kUnitGrid, kb = h_kb[(size_t)su[(size_t)b].t0] / kUnitGrid;
      return ka != kb ? ka < kb : su[(size_t)a].panel < su[(size_t)b].panel;
    });
    // the units behind the last full group go first, one to a queue in turn
    const int32_t ngroups = nunits / gsize, loose = nunits - ngroups * gsize;
    for (int32_t i = 0; i < loose; ++i) queue[i % kXcds].push_back(order[(size_t)(ngroups * gsize + i)]);
    // a group's place in the order goes by its costliest member (a group that straddles two block numbers holds light
    // and heavy units, and a heavy unit that starts late is what the launch ends on), a queue's load by the sums
    std::vector<double> gcost((size_t)ngroups, 0.0), gmax((size_t)ngroups, 0.0);
    for (int32_t i = 0; i < ngroups * gsize; ++i) {
      const double c = cost(order[(size_t)i]);
      gcost[(size_t)(i / gsize)] += c;
      if (c > gmax[(size_t)(i / gsize)]) gmax[(size_t)(i / gsize)] = c;
    }
    std::vector<int32_t> gorder((size_t)ngroups);
    for (int32_t g = 0; g < ngroups; ++g) gorder[(size_t)g] = g;
    std::stable_sort(gorder.begin(), gorder.end(), [&](int32_t a, int32_t b) {
      return gmax[(size_t)a] != gmax[(size_t)b] ? gmax[(size_t)a] > gmax[(size_t)b] : gcost[(size_t)a] > gcost[(size_t)b];
    });
    double given[kXcds] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int32_t r0 = 0; r0 < ngroups; r0 += kXcds) {
      const int32_t in_round = ngroups - r0 < kXcds ? ngroups - r0 : kXcds;
      int32_t by_load[kXcds];
      for (int32_t x = 0; x < kXcds; ++x) by_load[x] = x;
      std::stable_sort(by_load, by_load + kXcds, [&](int32_t a, int32_t b) { return given[a] < given[b]; });
      for (int32_t k = 0; k < in_round; ++k) {
        const int32_t g = gorder[(size_t)(r0 + k)];
        given[by_load[k]] += gcost[(size_t)g];
        for (int32_t j = 0; j < gsize; ++j) queue[by_load[k]].push_back(order[(size_t)(g * gsize + j)]);
      }
    }
  }
  int32_t qstart[kXcds + 1] = {0};
  for (int32_t x = 0, at = 0; x < kXcds; ++x) {
    for (int32_t u : queue[x]) order[(size_t)at++] = u;
    qstart[x + 1] = at;
  }
  int32_t *d_panel_unit = nullptr;
  CG_TRY(tmp.alloc((void **)&d_panel_unit, (size_t)npanels * 4));
  CG_TRY(dev_alloc((void **)&pp.unit_tile, (size_t)(nunits + 1) * 4));
  CG_TRY(dev_alloc((void **)&pp.unit_order, (size_t)(nunits > 0 ? nunits : 1) * 4));
  CG_TRY(dev_alloc((void **)&pp.unit_qstart, sizeof(qstart)));
  CG_HIP(hipMemcpyAsync(pp.unit_qstart, qstart, sizeof(qstart), hipMemcpyHostToDevice, stream));
  CG_TRY(dev_alloc((void **)&pp.unit_block, (size_t)nunits * 4));
  CG_TRY(dev_alloc((void **)&pp.unit_row0, (size_t)(nunits > 0 ? nunits : 1) * 4));
  CG_TRY(dev_alloc((void **)&pp.dslot, (size_t)n * 4));
  CG_HIP(hipMemcpyAsync(pp.unit_tile, unit_tile.data(), (size_t)(nunits + 1) * 4, hipMemcpyHostToDevice, stream));
  if (nunits > 0) {
    CG_HIP(hipMemcpyAsync(pp.unit_order, order.data(), (size_t)nunits * 4, hipMemcpyHostToDevice, stream));
    CG_HIP(hipMemcpyAsync(pp.unit_block, unit_block.data(), (size_t)nunits * 4, hipMemcpyHostToDevice, stream));
    CG_HIP(hipMemcpyAsync(pp.unit_row0, unit_row0.data(), (size_t)nunits * 4, hipMemcpyHostToDevice, stream));
  }
  if (ndunits > 0) {
    CG_TRY(dev_alloc((void **)&pp.dwg_unit, (size_t)(ndwg + 1) * 4));
    CG_TRY(dev_alloc((void **)&pp.dunit_tile, (size_t)(ndunits + 1) * 4));
    CG_TRY(dev_alloc((void **)&pp.dunit_block, (size_t)ndunits * 4));
    CG_HIP(hipMemcpyAsync(pp.dwg_unit, dwg_unit.data(), (size_t)(ndwg + 1) * 4, hipMemcpyHostToDevice, stream));
    CG_HIP(hipMemcpyAsync(pp.dunit_tile, dunit_tile.data(), (size_t)(ndunits + 1) * 4, hipMemcpyHostToDevice, stream));
    CG_HIP(hipMemcpyAsync(pp.dunit_block, dunit_block.data(), (size_t)ndunits * 4, hipMemcpyHostToDevice, stream));
  }
  CG_HIP(hipMemcpyAsync(d_panel_unit, panel_unit.data(), (size_t)npanels * 4, hipMemcpyHostToDevice, stream));
  if (nblocks > 0) {
    CG_TRY(dev_alloc((void **)&pp.bcount, (size_t)nblocks * 4));
    CG_HIP(hipMemcpyAsync(pp.bcount, bcount.data(), (size_t)nblocks * 4, hipMemcpyHostToDevice, stream));
  }
  if (!split.empty()) {
    CG_TRY(dev_alloc((void **)&pp.split, split.size() * 4));
    CG_HIP(hipMemcpyAsync(pp.split, split.data(), split.size() * 4, hipMemcpyHostToDevice, stream));
  }
  panel_dslot_kernel<<<gn, kSpmmThreads, 0, stream>>>(row_rank, n, d_panel_unit, (int32_t)npanels, PR, pp.dslot);
  CG_LAUNCH_CHECK();
  {  // the rows the pass over the partial rows writes
    uint32_t *flag = nullptr, *pos = nullptr, *d_count = nullptr, h_count = 0;
    CG_TRY(tmp.alloc((void **)&flag, (size_t)(n + 1) * 4));
    CG_TRY(tmp.alloc((void **)&pos, (size_t)(n + 1) * 4));
    CG_TRY(tmp.alloc((void **)&d_count, 4));
    const unsigned gn1 = (unsigned)ceil_div64((int64_t)n + 1, kSpmmThreads);
    panel_finish_flag_kernel<<<gn1, kSpmmThreads, 0, stream>>>(pp.dslot, pp.bcount, n, PR, flag);
    CG_LAUNCH_CHECK();
    CG_TRY(exclusive_scan_u32(flag, pos, (int64_t)n + 1, d_count, stream));
    CG_HIP(hipMemcpyAsync(&h_count, d_count, 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipStreamSynchronize(stream));
    CG_TRY(dev_alloc((void **)&pp.finish_rows, (size_t)(h_count > 0 ? h_count : 1) * 4));
    panel_finish_list_kernel<<<gn1, kSpmmThreads, 0, stream>>>(flag, pos, n, pp.finish_rows);
    CG_LAUNCH_CHECK();
    pp.nfinish = (int32_t)h_count;
  }
  CG_HIP(hipStreamSynchronize(stream));
  pp.covered = covered;
  pp.bcols = m;
  pp.prows = PR;
  pp.tcols = TC;
  pp.padded = padded;
  pp.dcovered = dcovered;
  pp.ntiles = (int32_t)ntiles;
  pp.ndtiles = (int32_t)ndtiles;
  pp.nunits = nunits;
  pp.ndunits = ndunits;
  pp.ndwg = ndwg;
  pp.nblocks = nblocks;
  pp.nsplit = (int32_t)(split.size() / 2);
  pp.valid = true;
  return CG_OK;
}

struct PanelParams {
  int32_t emin, cols, unit, dmin, dwg;
  bool share;  // staged columns in the whole matrix's order, units launched in XCD groups
  int32_t prows = kPanelRows, tcols = kPanelCols;  // rows of a panel, columns of a tile
  bool padded = true;
  bool same(const PanelPlan &pp) const {
    return pp.emin == emin && pp.hot_cols == cols && pp.unit_entries == unit && pp.dmin == dmin && pp.dwg == dwg &&
           pp.share == share && pp.prows == prows && pp.tcols == tcols && pp.padded == padded;
  }
  void stamp(PanelPlan &pp) const {
    pp.emin = emin;
    pp.hot_cols = cols;
    pp.unit_entries = unit;
    pp.dmin = dmin;
    pp.dwg = dwg;
    pp.share = share;
    pp.prows = prows;
    pp.tcols = tcols;
    pp.padded = padded;
  }
};

static PanelParams panel_params() {
  PanelParams p;
  p.emin = g_tune_panel_emin.load(std::memory_order_relaxed);
  if (p.emin <= 0) p.emin = kPanelDefaultEmin;
  p.cols = g_tune_panel_cols.load(std::memory_order_relaxed);
  if (p.cols <= 0) p.cols = kPanelDefaultCols;
  p.unit = g_tune_panel_unit.load(std::memory_order_relaxed);
  if (p.unit <= 0) p.unit = kPanelDefaultUnit;
  p.dmin = g_tune_panel_dmin.load(std::memory_order_relaxed);
  p.dmin = p.dmin < 0 ? 0 : (p.dmin == 0 ? kPanelDefaultDmin : p.dmin);  // 0 from here on: no dense tiles
  if (p.dmin > 0 && p.dmin < p.emin) p.dmin = p.emin;
  p.dwg = g_tune_panel_dwg.load(std::memory_order_relaxed);
  if (p.dwg <= 0) {  // four workgroups per compute unit, one after the other (a workgroup's staging buffers fill a unit's LDS)
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus < 1) {
      (void)hipGetLastError();
      cus = 256;
    }
    p.dwg = 4 * cus;
  }
  p.share = g_tune_panel_share.load(std::memory_order_relaxed) >= 0;
  return p;
}

static PanelParams tile_params(int geom) {
  PanelParams p = panel_params();
  p.prows = geom == 0 ? 256 : geom == 1 ? 512 : 1024;
  p.tcols = geom == 0 ? 64 : geom == 1 ? 128 : 256;
  p.padded = false;
  p.emin = 1;                 // every tile is staged: nothing is left for the row-wise kernels
  p.cols = kPanelDefaultCols;
  p.dmin = 0;                 // no tiles for the matrix cores
  // (units of kPanelDefaultUnit entries whatever the panel height: a unit is what one workgroup does in one go)
  return p;
}

// Builds the plan for the given values; the plan carries them whatever the outcome (in use, declined).
static int build_panel(CsrSide &s, PanelPlan &pp, const PanelParams &par, bool may_decline, hipStream_t stream,
                       double min_coverage = 0.0, double min_reuse = kPanelMinReuse) {
  CG_TRY(refuse_under_capture(stream, "building a panel plan"));
  CG_HIP(hipStreamSynchronize(stream));
  pp.release();
  bool collision = false;
  int st = build_panel_once(s, pp, par.emin, par.cols, par.unit, par.dmin, par.dwg, par.share, may_decline, min_coverage, min_reuse,
                            &collision, stream, par.prows, par.tcols, par.padded);
  if (st == CG_OK && collision) {  // the matrix stores a (row, column) pair twice: every tile goes the record way
    pp.release();
    st = build_panel_once(s, pp, par.emin, par.cols, par.unit, 0, par.dwg, par.share, may_decline, min_coverage, min_reuse, &collision,
                          stream, par.prows, par.tcols, par.padded);
  }
  if (st != CG_OK) pp.release();
  par.stamp(pp);
  return st;
}

// One bit per device and kernel: the dynamic LDS limit of the kernel has been raised there.
template <typename K>
static int panel_lds_attr(K kernel, std::atomic<uint64_t> &done, int dev, size_t lds_max, size_t lds_now) {
  if (dev < 64 && !(done.load() >> dev & 1)) {
    CG_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_max));
    done.fetch_or((uint64_t)1 << dev);
  } else if (dev >= 64) {
    CG_HIP(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_now));
  }
  return CG_OK;
}

// Slices of a product of width f on a plan with panels of `prows` rows: a wave owns prows / 16 rows and has 80
// accumulator registers, so a row of a slice takes at most 80 / (prows / 16) registers (see spmm_tile.h for the
// widths the register layouts cover), and two tiles of the slice's rows of B must fit the LDS.
struct TileShape {
  int32_t nr = 0, nsl = 0, fsw = 0;  // registers per row, slices, columns of a slice (a multiple of 4)
};
static bool tile_shape(int32_t prows, int32_t tcols, int32_t f, TileShape &sh) {
  const int32_t R = prows / kPanelWaves;
  int32_t cap = R <= 8 ? 636 : R <= 16 ? 316 : R <= 32 ? 128 : R <= 64 ? 64 : 0;
  const int32_t lds_cap = (int32_t)((160 * 1024 - 1024 - 256) / (2 * (size_t)tcols) / 16 * 4);  // columns two tiles leave room for
  if (lds_cap < cap) cap = lds_cap;
  if (cap < 4 || f < 1) return false;
  sh.nsl = (f + cap - 1) / cap;
  sh.fsw = ((f + sh.nsl - 1) / sh.nsl + 3) & ~3;
  if (sh.fsw > cap) sh.fsw = cap & ~3;
  sh.nsl = (f + sh.fsw - 1) / sh.fsw;
  if (R <= 8)
    sh.nr = sh.fsw > 512 ? 10 : 8;
  else if (R <= 16)
    sh.nr = sh.fsw > 256 ? 5 : 4;
  else
    sh.nr = R <= 32 ? 2 : 1;
  return true;
}

// Can spmm_tile_kernel read this B?  Its copies move 16 bytes per lane straight into LDS, from addresses that must
// be multiples of 8 (measured: rows 4 bytes off give wrong data); narrow slices address B by 32-bit offsets and copy
// whole 16-byte pieces only.
static bool tile_operands_ok(int32_t prows, int32_t tcols, const float *B, int64_t ldb, int32_t f, int32_t m) {
  TileShape sh;
  if (!tile_shape(prows, tcols, f, sh)) return false;
  if (((uintptr_t)B & 7u) != 0 || (ldb & 1) != 0 || ldb > 0x7fffffffLL) return false;
  if (sh.nr < 4) {
    if (f % 4 != 0) return false;
    if ((int64_t)m * ldb * 4 >= (int64_t)1 << 31) return false;  // (32-bit offsets that are positive as int32 too)
    if (((uintptr_t)B & 15u) != 0 || (ldb & 3) != 0) return false;  // every piece of a narrow row on a 16-byte boundary
  }
  return true;
}

// The staged tiles of a plan through spmm_tile_kernel (any width; panels of 128, 256, 512 or 1024 rows).
static int launch_tile(const PanelPlan &pp, const float *B, int64_t ldb, int32_t f, float *P, int32_t *qhead, float *C_direct,
                       int64_t ldc, int32_t rows, float beta, int dev, int cus, hipStream_t stream) {
  TileShape sh;
  if (!tile_shape(pp.prows, pp.tcols, f, sh)) CG_FAIL(CG_ERR_UNSUPPORTED, "tile product: no kernel for f=%d", f);
  TileArgs ta{};
  ta.unit_tile = pp.unit_tile;
  ta.unit_order = pp.unit_order;
  ta.unit_qstart = pp.unit_qstart;
  ta.qhead = qhead;
  ta.unit_block = pp.unit_block;
  ta.hdr = pp.hdr;
  ta.ent = pp.ent;
  ta.B = B;
  ta.ldb = ldb;
  ta.P = P;
  ta.f = f;
  ta.fsw = sh.fsw;
  ta.nsl = sh.nsl;
  ta.m = pp.bcols;
  ta.unit_row0 = pp.unit_row0;
  ta.rank_row = pp.rank_row;
  ta.C = C_direct;
  ta.ldc = ldc;
  ta.rows = rows;
  ta.beta = beta;
  // two tiles of staged rows (narrow slices: a wave's staging area is a whole number of 1 KiB pieces) and some room
  // behind them: the lanes of a row read beyond the slice's last column
  const size_t tlds_max = 160 * 1024 - 1024;  // the kernel's own LDS word lies in front, the buffers start on a multiple of 1024
  const size_t rs = sh.nr == 1 ? 256 : sh.nr == 2 ? 512 : sh.nr == 4 ? 1024 : (size_t)sh.fsw * 4;  // LROW of the kernel
  const size_t area = (size_t)(pp.tcols / kPanelWaves) * rs;
  size_t tlds = 2 * (size_t)kPanelWaves * area + 256;
  if (tlds > tlds_max) tlds = tlds_max;
  if (2 * (size_t)kPanelWaves * area > tlds_max) CG_FAIL(CG_ERR_UNSUPPORTED, "tile product: f=%d does not fit the LDS", f);
  const int64_t items = (int64_t)pp.nunits * sh.nsl;
  const unsigned grid = (unsigned)(items < cus ? items : cus);
#define CG_TILE(NR, R, TCW)                                                                        \
  {                                                                                                \
    static std::atomic<uint64_t> attr_set{0};                                                      \
    CG_TRY(panel_lds_attr(spmm_tile_kernel<NR, R, TCW>, attr_set, dev, tlds_max, tlds));           \
    spmm_tile_kernel<NR, R, TCW><<<grid, kPanelThreads, tlds, stream>>>(ta);                       \
  }
  const int32_t R = pp.prows / kPanelWaves, TCW = pp.tcols / kPanelWaves;
  if (R == 8 && TCW == 2 && sh.nr == 10) CG_TILE(10, 8, 2)
  else if (R == 8 && TCW == 2 && sh.nr == 8) CG_TILE(8, 8, 2)
  else if (R == 16 && TCW == 4 && sh.nr == 5) CG_TILE(5, 16, 4)
  else if (R == 16 && TCW == 4 && sh.nr == 4) CG_TILE(4, 16, 4)
  else if (R == 32 && TCW == 8 && sh.nr == 2) CG_TILE(2, 32, 8)
  else if (R == 64 && TCW == 16 && sh.nr == 1) CG_TILE(1, 64, 16)
  else CG_FAIL(CG_ERR_UNSUPPORTED, "tile product: no kernel for panels of %d rows and tiles of %d columns", pp.prows, pp.tcols);
#undef CG_TILE
  CG_LAUNCH_CHECK();
  return CG_OK;
}

// The panel part of C = A B: partial rows of every row that has entries in active or dense tiles, in *P
// (row r: P + dslot[r] * f).  P is stream scratch and stays valid until the next panel product on `stream`.
// sum_blocks: add the blocks of a panel into its first one (false: the caller's pass over the partial rows does that)
// C_direct (with ldc, rows, beta): staged units that are their panel's only block write C = beta C + their rows
// themselves; launch_panel_finish(direct_written = true) then leaves those rows alone.
static int launch_panel(const PanelPlan &pp, const float *B, int64_t ldb, int32_t f, float **P_out, hipStream_t stream,
                        bool sum_blocks = true, float *C_direct = nullptr, int64_t ldc = 0, int32_t rows = 0, float beta = 0.f) {
  if (ldb > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "panel product: leading dimension %lld >= 2^31", (long long)ldb);
  const int chunks = (f / 2 + kWave - 1) / kWave;
  const int groups = (f + 63) / 64;
  const size_t rs = ((size_t)f * 4 + 15) & ~(size_t)15;
  const size_t lds = 2 * (size_t)kPanelCols * rs;  // two tiles of staged rows
  const size_t lds_max = 2 * (size_t)kPanelCols * ((kPanelMaxF * 4 + 15) & ~15);
  void *p = nullptr;
  const size_t p_bytes = ((size_t)pp.nblocks * pp.prows * f * sizeof(float) + 15) & ~(size_t)15;
  CG_TRY(scratch_get(stream, kSlotE, p_bytes + kXcdQueues * sizeof(int32_t), &p));
  float *P = (float *)p;
  int32_t *qhead = (int32_t *)((char *)p + p_bytes);  // the queues' counters of this launch (panel_take_unit)
  int dev = 0, cus = 0;
  CG_HIP(hipGetDevice(&dev));
  CG_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));  // a workgroup of the staged-tile kernel fills a compute unit's LDS
  if (cus < 1) cus = 256;
  if (pp.ndunits > 0) {
    ProfScope prof("spmm_panel_dense", f, stream);
#define CG_PANEL_DENSE(NG)                                                                                              \
  case NG: {                                                                                                            \
    static std::atomic<uint64_t> attr_set{0};                                                                           \
    CG_TRY(panel_lds_attr(spmm_panel_dense_kernel<NG>, attr_set, dev, lds_max, lds));                                   \
    spmm_panel_dense_kernel<NG><<<(unsigned)pp.ndwg, kDenseThreads, lds, stream>>>(                                     \
        pp.dwg_unit, pp.dunit_tile, pp.dunit_block, pp.dhdr, pp.dA, B, ldb, P, f);                                      \
  } break;
    switch (groups) {
      CG_PANEL_DENSE(5)
      CG_PANEL_DENSE(6)
      CG_PANEL_DENSE(7)
      CG_PANEL_DENSE(8)
      CG_PANEL_DENSE(9)
      CG_PANEL_DENSE(10)
      default:
        CG_FAIL(CG_ERR_UNSUPPORTED, "panel product: no dense-tile kernel for f=%d", f);
    }
#undef CG_PANEL_DENSE
    CG_LAUNCH_CHECK();
  }
  {
    ProfScope prof("spmm_panel", f, stream);
#define CG_PANEL(CH)                                                                                                   \
  case CH: {                                                                                                           \
    static std::atomic<uint64_t> attr_set{0};                                                                          \
    CG_TRY(panel_lds_attr(spmm_panel_kernel<CH>, attr_set, dev, lds_max, lds));                                        \
    spmm_panel_kernel<CH><<<(unsigned)(pp.nunits < cus ? pp.nunits : cus), kPanelThreads, lds, stream>>>(pp.unit_tile, pp.unit_order, pp.unit_qstart, qhead, pp.unit_block, \
                                                                               pp.hdr, pp.ent, B, ldb, P, f, pp.unit_row0, \
                                                                               pp.rank_row, C_direct, ldc, rows, beta, \
                                                                               g_tune_panel_qcap.load(std::memory_order_relaxed)); \
  } break;
    const bool legacy = pp.padded && pp.prows == kPanelRows && pp.tcols == kPanelCols && panel_width_ok(f);
    if (pp.nunits > 0 && !legacy) {
      CG_TRY(fill_u32((uint32_t *)qhead, kXcdQueues, 0u, stream));
      CG_TRY(launch_tile(pp, B, ldb, f, P, qhead, C_direct, ldc, rows, beta, dev, cus, stream));
    } else if (pp.nunits > 0) {
      const int qskip = g_tune_panel_qskip.load(std::memory_order_relaxed);
      CG_TRY(fill_u32((uint32_t *)qhead, kXcdQueues, (uint32_t)(qskip > 0 ? qskip : 0), stream));
      switch (chunks) {
        CG_PANEL(3)
        CG_PANEL(4)
        CG_PANEL(5)
        default:
          CG_FAIL(CG_ERR_UNSUPPORTED, "panel product: no kernel for f=%d", f);
      }
      CG_LAUNCH_CHECK();
    }
#undef CG_PANEL
    if (sum_blocks && pp.nsplit > 0) {
      const dim3 grid((unsigned)ceil_div64((int64_t)pp.prows * f, kSpmmThreads), (unsigned)pp.nsplit);
      panel_reduce_kernel<<<grid, kSpmmThreads, 0, stream>>>(pp.split, P, f, pp.prows);
      CG_LAUNCH_CHECK();
    }
  }
  *P_out = P;
  return CG_OK;
}

// C = beta C + the partial rows (every block of a row's panel), for a plan without a rest matrix to multiply
static int launch_panel_finish(const PanelPlan &pp, const float *P, float *C, int64_t ldc, int32_t f, float beta,
                               hipStream_t stream) {
  ProfScope prof("spmm_panel_add", f, stream);
  if (pp.nfinish == 0) return CG_OK;
  if (f % 2 == 0)
    panel_finish_kernel<<<(unsigned)ceil_div64((int64_t)pp.nfinish * (f / 2), kSpmmThreads), kSpmmThreads, 0, stream>>>(
        C, ldc, P, pp.dslot, pp.bcount, pp.finish_rows, pp.nfinish, f, beta, pp.prows);
  else
    panel_finish1_kernel<<<(unsigned)ceil_div64((int64_t)pp.nfinish * f, kSpmmThreads), kSpmmThreads, 0, stream>>>(
        C, ldc, P, pp.dslot, pp.bcount, pp.finish_rows, pp.nfinish, f, beta, pp.prows);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

}  // namespace cg
