// Host side of the CSR SpMM: the products (plain schedule, hub plan, one-shot), the cached handle,
// blocks recognised by content and the C ABI entry points.  The device kernels are in
// spmm_kernels.h, schedules and window tables in spmm_tables.h, handle data and hub plan
// construction in spmm_hub.h.
//
// Replaces everything the reference wraps around cusparseSpMM on every call
// (sparse-extension/sparse_coo_tensor.cu:136-231): B and C stay row-major, nothing is transposed,
// and the CSR, its transpose, the schedules and the hub plan live in a handle.
#include "spmm_panel_build.h"
#include "spmm_panel_narrow.h"
#include <stdlib.h>
#include <string.h>
#include <atomic>
#include <memory>
#include <mutex>
#include <new>
#include <vector>

namespace cg {

extern std::atomic<int> g_tune_dense_mfma;  // dense.hip

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
  // optional direct fold: one more partial row per row, fold_D[fold_dslot[row] * f ...] (panel plan)
  const float *fold_D = nullptr;
  const int32_t *fold_dslot = nullptr;
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
    CG_TRY(refuse_under_capture(stream, "building the window table of a schedule"));
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
  sa.fold_D = d.fold_D;
  sa.fold_dslot = d.fold_dslot;
  if ((d.fold_tbase || d.fold_dslot) && shape.lpr != kWave) CG_FAIL(CG_ERR_UNSUPPORTED, "fold needs full-wave teams");
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
        d.fold_P, d.fold_classes, d.fold_rows, d.fold_D, d.fold_dslot);
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
// The rest matrix of a narrow panel plan (its dense tiles are gone: what is left are the entries of the less
// popular columns) takes the plan from 40 columns on: measured on 232,965 vertices with 492 entries per row, f = 44
// (rows of B 192 bytes apart): 1.56 -> 1.37 ms, f = 48: 1.54 -> 1.34 ms; on the whole matrix at those widths the
// plan does not pay (1.85 -> 1.90 ms).
static bool want_hub(const CsrSide &s, int32_t f) {
  if (s.is_rest && f >= 40 && f < 64 && g_tune_hub.load(std::memory_order_relaxed) == 0)
    return s.rows > 0 && s.nnz / s.rows >= 8 && (double)s.nnz * f >= 1.5e9;
  return want_hub(s.rows, s.nnz, f);
}

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
        s.hub[i].min_degree == min_degree && (may_decline || !s.hub[i].declined || s.hub[i].failed))
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
    const int st = build_hub(s, s.hub[slot], (int32_t)hot, (int32_t)hot_single, groups, tiers, seg, min_degree,
                             may_decline, stream);
    if (st == CG_ERR_ALLOC || st == CG_ERR_OVERFLOW) {
      // No memory for the plan (its build needs about 6 x 4 nnz bytes of temporaries and a second copy of
      // the entries) or a matrix its virtual rows cannot index: the product goes through the plain
      // schedule, and the refusal is remembered so that later calls do not try again.
      HubPlan &hp = s.hub[slot];
      hp.release();
      hp.req_hot = (int32_t)hot;
      hp.req_single = (int32_t)hot_single;
      hp.req_tiers = tiers;
      hp.groups = groups;
      hp.seg = seg;
      hp.min_degree = min_degree;
      hp.declined = true;
      hp.failed = true;
      hp.valid = true;
    } else if (st != CG_OK) {
      return st;
    }
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
      CG_TRY(refuse_under_capture(stream, "building the window table of a hub plan"));
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

// fold (nullable): only its direct-fold fields are read (the partial rows of a panel plan, added to the rows
// this product finishes).  allow_panel: false for the rest matrix of a panel plan.
static int spmm_side(CsrSide &s, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta,
                     hipStream_t stream, const DenseOps *epi = nullptr, const DenseOps *fold = nullptr,
                     bool allow_panel = true) {
  if (s.rows == 0) return CG_OK;
  const int vec = pick_vec(f, B, ldb, C ? C : B, C ? ldc : ldb);
  const int32_t cap = range_cap(vec);
  DenseOps d{B, ldb, C, ldc, f, beta};
  if (fold) {
    d.fold_D = fold->fold_D;
    d.fold_dslot = fold->fold_dslot;
  }
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
  // Tile plan: every entry is multiplied out of LDS by spmm_tile_kernel, in panels whose height goes by the width.
  // `after_panel`: the second look, for the widths that the panel plan with its matrix-core tiles is tried for first.
  bool tile_done = false;
  auto try_tile = [&](bool after_panel) -> int {
    if (epi || fold || !allow_panel || !want_tile(s, f, after_panel)) return CG_OK;
    const int geom = tile_geometry(f);
    const PanelParams par = tile_params(geom);
    if (!tile_operands_ok(par.prows, par.tcols, B, ldb, f, s.cols)) return CG_OK;
    PanelPlan &pp = s.tile[geom];
    if (!pp.valid || !par.same(pp)) {
      const int st = build_panel(s, pp, par, false, stream, 0.0, 0.0);
      if (st == CG_ERR_ALLOC || st == CG_ERR_OVERFLOW) {  // no memory for the plan: remembered as declined
        pp.declined = pp.failed = pp.valid = true;
      } else if (st != CG_OK) {
        return st;
      }
    }
    if (pp.declined || pp.rest->nnz != 0) return CG_OK;
    float *P = nullptr;
    CG_TRY(launch_panel(pp, B, ldb, f, &P, stream, false, C, ldc, s.rows, beta));
    tile_done = true;
    return launch_panel_finish(pp, P, C, ldc, f, beta, stream);
  };
  CG_TRY(try_tile(false));
  if (tile_done) return CG_OK;
  // Panel plan: the entries of dense (row panel, column block) tiles are multiplied out of LDS into
  // partial rows; the row-wise kernels then run over the other entries and add those rows in.
  if (!epi && allow_panel && f <= cap && want_panel(s, f)) {
    PanelParams par = panel_params();
    // The staged tiles go through spmm_tile_kernel, which takes the records as they are; the older spmm_panel_kernel
    // (records of a run padded to pairs) serves operands that kernel cannot read and the tuning value.
    // (also for the last widths two of whose tiles the tile kernel's LDS layout has no room for: it would take them in two slices)
    TileShape one;
    par.padded = g_tune_panel_legacy.load(std::memory_order_relaxed) > 0 || !tile_operands_ok(par.prows, par.tcols, B, ldb, f, s.cols) ||
                 !tile_shape(par.prows, par.tcols, f, one) || one.nsl != 1;
    const bool may_decline = g_tune_panel.load(std::memory_order_relaxed) == 0;
    PanelPlan &pp = s.panel;
    if (!pp.valid || !par.same(pp) || (pp.declined && !may_decline && !pp.failed)) {
      const int st = build_panel(s, pp, par, may_decline, stream);
      if (st == CG_ERR_ALLOC || st == CG_ERR_OVERFLOW) {  // no memory for the plan: remembered as declined
        pp.declined = pp.failed = pp.valid = true;
      } else if (st != CG_OK) {
        return st;
      }
    }
    if (!pp.declined) {
      float *P = nullptr;
      const bool direct = pp.rest->nnz == 0 && !fold;  // nothing for the row-wise kernels: one pass sums the blocks into C
      if (direct) {  // units that are their panel's only block write their rows of C, the pass over the others skips them
        CG_TRY(launch_panel(pp, B, ldb, f, &P, stream, false, C, ldc, s.rows, beta));
        return launch_panel_finish(pp, P, C, ldc, f, beta, stream);
      }
      CG_TRY(launch_panel(pp, B, ldb, f, &P, stream, true));
      DenseOps fd{};
      fd.fold_D = P;
      fd.fold_dslot = pp.dslot;
      return spmm_side(*pp.rest, B, ldb, C, ldc, f, beta, stream, nullptr, &fd, false);
    }
  }
  CG_TRY(try_tile(true));  // the panel plan stood back (too few entries share their column inside a panel of 128 rows)
  if (tile_done) return CG_OK;
  // Narrow products: the dense tiles of a panel plan of their own on the matrix cores, the other entries by the
  // row-wise kernels, then the partial rows are added in (a pass over an n x f array, which is small here).
  if (!epi && !fold && allow_panel && want_panel_narrow(s, f)) {
    const PanelParams par = panel_narrow_params();
    const bool may_decline = g_tune_panel_narrow.load(std::memory_order_relaxed) == 0;
    PanelPlan &pp = s.panel_narrow;
    if (!pp.valid || !par.same(pp) || (pp.declined && !may_decline && !pp.failed)) {
      const int st = build_panel(s, pp, par, may_decline, stream, kPanelNarrowMinCoverage, 0.0);
      if (st == CG_ERR_ALLOC || st == CG_ERR_OVERFLOW) {
        pp.declined = pp.failed = pp.valid = true;
      } else if (st != CG_OK) {
        return st;
      }
    }
    if (!pp.declined && pp.ndtiles > 0) {
      float *P = nullptr;
      CG_TRY(launch_panel_narrow(pp, B, ldb, f, &P, stream));
      CG_TRY(spmm_side(*pp.rest, B, ldb, C, ldc, f, beta, stream, nullptr, nullptr, false));
      return launch_panel_add_rows(pp, P, C, ldc, s.rows, f, stream);
    }
  }
  if (f <= range_cap(vec == 4 ? 4 : 1) && want_hub(s, f)) {
    bool declined = false;
    CG_TRY(spmm_hub(s, vec, d, stream, &declined));
    if (!declined) return CG_OK;
  }
  if (epi || f <= cap) return spmm_plain(s.rowptr, s.colind, s.val, s.rows, s.nnz, s.sched, vec, d, f, stream);
  if (d.fold_dslot) CG_FAIL(CG_ERR_UNSUPPORTED, "direct fold needs a width one launch covers");
  for (int32_t f0 = 0; f0 < f; f0 += cap) {  // wider outputs take several launches over column ranges
    const int32_t ft = f - f0 < cap ? f - f0 : cap;
    const DenseOps dr{B + f0, ldb, C + f0, ldc, ft, beta};
    CG_TRY(spmm_plain(s.rowptr, s.colind, s.val, s.rows, s.nnz, s.sched, vec, dr, f, stream));
  }
  return CG_OK;
}

// Entry of every product on a handle's side.  A product issued while its stream is being captured pins
// the side: from then on tables of the side that have to go (an evicted hub plan, a recycled schedule,
// a panel plan rebuilt for other tuning values) are parked on the side instead of freed, because the
// captured graph replays with their addresses.  cg_csr_unpin or the handle's destruction frees them.
static int spmm_entry(CsrSide &s, const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta,
                      hipStream_t stream, const DenseOps *epi = nullptr) {
  if (stream_capturing(stream)) s.pinned = true;
  ParkScope park(s.pinned ? &s.parked : nullptr);
  return spmm_side(s, B, ldb, C, ldc, f, beta, stream, epi);
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
        pslots, nullptr, nullptr, 0, 0, nullptr, nullptr);
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
  int64_t bytes = 0;  // estimate of the device memory the block holds (CSR copy and up to two plan copies of the entries)
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
static int64_t coo_cache_byte_cap() {  // kept blocks may hold this much device memory together (the newest one always stays)
  const int v = g_tune_coo_cache_mib.load(std::memory_order_relaxed);
  return (int64_t)(v <= 0 ? 32768 : v) << 20;
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
  CG_TRY(refuse_under_capture(stream, "cg_spmm_coo_cached (it reads the digest of the block back)"));
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
    entry->bytes = 4 * (nnz * 8) + 4 * ((int64_t)n + 1) * 4;  // the CSR, a panel plan (tiles, records, rest) and the rest's hub plans
    entry->h = h;
    std::vector<std::shared_ptr<CooCacheEntry>> evicted;  // released after the lock is dropped
    {
      std::lock_guard<std::mutex> lock(g_coo_cache_mu);
      ++g_coo_cache_misses;
      entry->tick = ++g_coo_cache_tick;
      g_coo_cache.push_back(entry);
      const int64_t byte_cap = coo_cache_byte_cap();
      auto held = [&]() {
        int64_t total = 0;
        for (auto &e : g_coo_cache) total += e->bytes;
        return total;
      };
      while ((int)g_coo_cache.size() > capacity || (g_coo_cache.size() > 1 && held() > byte_cap)) {
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
  return spmm_entry(entry->h->fwd, d_B, ldb, d_C, ldc, f, beta, stream);
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

int cg_csr_unpin(cg_csr_t *h, int64_t *released) {
  if (!h) CG_FAIL(CG_ERR_NULL, "cg_csr_unpin: handle is NULL");
  (void)hipDeviceSynchronize();
  int64_t count = 0;
  for (cg::CsrSide *s : {&h->fwd, &h->tr}) {
    count += s->unpin();
    if (s->panel.rest) count += s->panel.rest->unpin();
    if (s->panel_narrow.rest) count += s->panel_narrow.rest->unpin();
    for (int i = 0; i < cg::CsrSide::kTilePlans; ++i)
      if (s->tile[i].rest) count += s->tile[i].rest->unpin();
  }
  if (released) *released = count;
  return CG_OK;
}

int cg_csr_spmm(cg_csr_t *h, int transpose, const float *d_B, int64_t ldb, float *d_C, int64_t ldc, int32_t f,
                float beta, cg_stream_t stream) {
  using namespace cg;
  if (!h) CG_FAIL(CG_ERR_NULL, "cg_csr_spmm: handle is NULL");
  if (transpose && !h->has_t) CG_FAIL(CG_ERR_NO_TRANSPOSE, "cg_csr_spmm: handle was built without CG_CSR_TRANSPOSE");
  CsrSide &s = transpose ? h->tr : h->fwd;
  CG_TRY(check_dense("cg_csr_spmm", d_B, ldb, d_C, ldc, f, s.cols, s.rows));
  return spmm_entry(s, d_B, ldb, d_C, ldc, f, beta, (hipStream_t)stream);
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
  return spmm_entry(s, d_B, ldb, beta != 0.f ? const_cast<float *>(d_C) : nullptr, ldc, f, beta, (hipStream_t)stream, &epi);
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
  else if (!strcmp(key, "spmm_panel")) cg::g_tune_panel.store(value);
  else if (!strcmp(key, "spmm_panel_emin")) cg::g_tune_panel_emin.store(value);
  else if (!strcmp(key, "spmm_panel_cols")) cg::g_tune_panel_cols.store(value);
  else if (!strcmp(key, "spmm_panel_unit")) cg::g_tune_panel_unit.store(value);
  else if (!strcmp(key, "spmm_panel_dmin")) cg::g_tune_panel_dmin.store(value);
  else if (!strcmp(key, "spmm_panel_dwg")) cg::g_tune_panel_dwg.store(value);
  else if (!strcmp(key, "spmm_panel_share")) cg::g_tune_panel_share.store(value);
  else if (!strcmp(key, "spmm_tile")) cg::g_tune_tile.store(value);
  else if (!strcmp(key, "spmm_panel_legacy")) cg::g_tune_panel_legacy.store(value);
  else if (!strcmp(key, "spmm_panel_costcap")) cg::g_tune_panel_costcap.store(value);
  else if (!strcmp(key, "spmm_strict_nonfinite")) cg::g_tune_strict.store(value);
  else if (!strcmp(key, "spmm_panel_qskip")) cg::g_tune_panel_qskip.store(value);
  else if (!strcmp(key, "spmm_panel_qcap")) cg::g_tune_panel_qcap.store(value);
  else if (!strcmp(key, "spmm_panel_narrow")) cg::g_tune_panel_narrow.store(value);
  else if (!strcmp(key, "spmm_panel_narrow_dmin")) cg::g_tune_panel_narrow_dmin.store(value);
  else if (!strcmp(key, "dense_mfma")) cg::g_tune_dense_mfma.store(value);
  else if (!strcmp(key, "coo_cache_blocks")) cg::g_tune_coo_cache.store(value);
  else if (!strcmp(key, "coo_cache_mib")) cg::g_tune_coo_cache_mib.store(value);
  else if (!strcmp(key, "test_alloc_fail")) cg::g_test_alloc_fail.store(value);
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
  auto last_plan = [](const cg::CsrSide &side) -> int64_t {
    // with a panel plan in use the row-wise kernels, and so the hub plans, work on its rest matrix
    const cg::CsrSide &s = (side.panel.valid && !side.panel.declined && side.panel.rest) ? *side.panel.rest : side;
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

int cg_csr_panel_info(const cg_csr_t *h, int transpose, int64_t info[12]) {
  if (!h || !info) CG_FAIL(CG_ERR_NULL, "cg_csr_panel_info: null pointer");
  if ((transpose & 1) && !h->has_t) CG_FAIL(CG_ERR_NO_TRANSPOSE, "cg_csr_panel_info: handle was built without CG_CSR_TRANSPOSE");
  const cg::CsrSide &side = (transpose & 1) ? h->tr : h->fwd;
  // bits 2..3: 0 the plan of the wide products, 1 .. 3 the tile plans with panels of 256, 512, 1024 rows
  const int which = (transpose >> 2) & 3;
  const cg::PanelPlan &pp = which ? side.tile[which - 1] : (transpose & 2) ? side.panel_narrow : side.panel;
  const bool used = pp.valid && !pp.declined;
  info[0] = !pp.valid ? 0 : (pp.declined ? -1 : 1);
  info[1] = used ? pp.covered : 0;
  info[2] = used ? pp.ntiles : 0;
  info[3] = used ? pp.nunits : 0;
  info[4] = used ? pp.nsplit : 0;
  info[5] = used && pp.rest ? pp.rest->nnz : 0;
  info[6] = pp.valid ? pp.emin : 0;
  info[7] = pp.valid ? pp.hot_cols : 0;
  info[8] = used ? pp.dcovered : 0;
  info[9] = used ? pp.ndtiles : 0;
  info[10] = used ? pp.ndunits : 0;
  info[11] = pp.valid ? pp.dmin : 0;
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
