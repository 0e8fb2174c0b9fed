// Narrow products (f <= 64) of a matrix with well-filled tiles: the dense tiles of a panel plan on the fp32
// matrix cores, everything else by the row-wise kernels.
//
// A row-wise product at f = 16 gathers a 64-byte row of B per entry and is bound by the rate at which L2
// serves such requests, whatever the entry's tile looks like.  A tile that is stored whole costs its 16 KB
// once, however many of its 4096 places are taken, and eight matrix instructions per wave and 16 result
// columns: from a few hundred entries per tile on that is the cheaper form.  The plan is an ordinary panel
// plan (spmm_panel.h, spmm_panel_build.h) whose staged tiles are switched off (every tile is dense or left to
// the rest matrix); this file holds its product kernel, the launch and the pass that adds the partial rows in.
// Replaces nothing in the reference beyond cusparseSpMM itself (sparse-extension/sparse_coo_tensor.cu:215-226).
#pragma once
#include "spmm_panel_build.h"

namespace cg {

constexpr int32_t kPanelNarrowMaxF = 64;
constexpr int32_t kPanelNarrowDmin = 512;        // entries from which a tile is stored whole for narrow products: measured at
                                                 // 232,965 vertices, 492 entries per row: f = 16 0.88 -> 0.70 ms, f = 44 1.83 -> 1.53,
                                                 // f = 64 1.84 -> 1.42; 384 .. 448 the same within 2.5 %, 192, 256 and 768 slower
constexpr double kPanelNarrowMinCoverage = 0.25;  // share of the entries the dense tiles must hold

static std::atomic<int> g_tune_panel_narrow{0}, g_tune_panel_narrow_dmin{0};

// Wave w of 8 owns rows 16 w .. 16 w + 15 of the panel.  Per tile: 8 reduction steps of 4 columns of A, each one
// v_mfma_f32_16x16x4_f32 per 16 result columns (NB of them); lane (q, c) = (l / 16, l % 16) feeds
// A[16 w + c][4 ks + q] and B[4 ks + q][16 nb + c] and holds D[16 w + 4 q + v][16 nb + c] in register v.
// The 32 rows of B of a tile (32 x f floats) are loaded into registers a tile ahead, like the tile itself, and
// written to the other of two LDS buffers behind the multiplies; one barrier per tile.  Workgroups take equal
// shares of the list of dense tiles; a unit is a run of tiles of one panel inside a share and ends in a block
// of 128 partial rows, as in spmm_panel_dense_kernel.
template <int NB>
__global__ __launch_bounds__(kDenseThreads) void spmm_panel_dense_narrow_kernel(
    const int32_t *__restrict__ wg_unit, const int32_t *__restrict__ unit_tile, const int32_t *__restrict__ unit_block,
    const int32_t *__restrict__ dhdr, const float *__restrict__ dA, const float *__restrict__ B, int64_t ldb,
    float *__restrict__ P, int32_t f) {
  constexpr int LDL = NB * 16 + 4;                                  // floats between staged rows (the 4: fewer bank conflicts)
  constexpr int PER = (kPanelCols * NB * 16) / kDenseThreads;       // staged floats per thread: NB
  static_assert(PER * kDenseThreads == kPanelCols * NB * 16, "the staging grid must divide among the threads");
  __shared__ float lds[2][kPanelCols * LDL];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int c16 = lane & 15, q = lane >> 4;
  const int u0 = wg_unit[blockIdx.x], u1 = wg_unit[blockIdx.x + 1];
  if (u0 >= u1) return;
  const int t_first = unit_tile[u0], t_end = unit_tile[u1];
  // thread -> (row, column) of the staging grid, PER places 512 apart
  auto stage_load = [&](int t, float (&v)[PER]) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = (int)threadIdx.x + i * kDenseThreads;
      const int r = idx / (NB * 16), c = idx % (NB * 16);
      const int64_t brow = dhdr[(int64_t)t * kPanelCols + r];
      v[i] = B[brow * ldb + (c < f ? c : 0)];  // unconditional load from a clamped column; zeroed below
    }
  };
  auto stage_store = [&](int buf, const float (&v)[PER]) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = (int)threadIdx.x + i * kDenseThreads;
      const int r = idx / (NB * 16), c = idx % (NB * 16);
      lds[buf][r * LDL + c] = c < f ? v[i] : 0.f;
    }
  };
  auto a_load = [&](int t, float4 (&a)[2]) {
    const float4 *src = reinterpret_cast<const float4 *>(dA) + ((int64_t)t * kDenseWaves + wave) * 2 * kWave + lane;
    a[0] = src[0];
    a[1] = src[kWave];
  };
  float4 a_cur[2];
  {
    float v[PER];
    stage_load(t_first, v);
    a_load(t_first, a_cur);
    stage_store(0, v);
  }
  __syncthreads();
  int buf = 0;
  for (int u = u0; u < u1; ++u) {
    panel_f4 acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = (panel_f4){0.f, 0.f, 0.f, 0.f};
    const int ut1 = unit_tile[u + 1];
    for (int t = unit_tile[u]; t < ut1; ++t) {
      const int tn = t + 1 < t_end ? t + 1 : t;  // the last tile of the share loads itself once more
      float vn[PER];
      float4 a_nxt[2];
      stage_load(tn, vn);
      a_load(tn, a_nxt);
      const float a8[8] = {a_cur[0].x, a_cur[0].y, a_cur[0].z, a_cur[0].w, a_cur[1].x, a_cur[1].y, a_cur[1].z, a_cur[1].w};
      const float *lb = &lds[buf][q * LDL + c16];
#pragma unroll
      for (int ks = 0; ks < 8; ++ks)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a8[ks], lb[ks * 4 * LDL + nb * 16], acc[nb], 0, 0, 0);
      stage_store(buf ^ 1, vn);  // nobody reads that buffer any more: the barrier of the tile before
      a_cur[0] = a_nxt[0];
      a_cur[1] = a_nxt[1];
      buf ^= 1;
      __syncthreads();
    }
    const int block = unit_block[u];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      float *prow = P + ((int64_t)block * kPanelRows + wave * 16 + 4 * q + v) * f;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int col = nb * 16 + c16;
        if (col < f) prow[col] = acc[nb][v];
      }
    }
  }
}

// C[r, :] += P[dslot[r], :] for the rows that have a partial row (one thread per element)
__global__ __launch_bounds__(kSpmmThreads) void panel_add_rows_kernel(float *__restrict__ C, int64_t ldc,
                                                                       const float *__restrict__ P,
                                                                       const int32_t *__restrict__ dslot, int32_t rows,
                                                                       int32_t f) {
  const int64_t idx = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  const int64_t r = idx / f;
  const int32_t c = (int32_t)(idx - r * f);
  if (r >= rows) return;
  const int32_t d = dslot[r];
  if (d >= 0) C[r * ldc + c] += P[(int64_t)d * f + c];
}

static bool want_panel_narrow(const CsrSide &s, int32_t f) {
  const int t = g_tune_panel_narrow.load(std::memory_order_relaxed);
  if (t < 0 || f < 1 || f > kPanelNarrowMaxF || s.rows == 0 || s.nnz == 0 || s.is_rest) return false;
  if (g_tune_strict.load(std::memory_order_relaxed) > 0) return false;  // dense tiles multiply their zeros
  if (t > 0) return true;
  return s.nnz / s.rows >= 64 && (double)s.nnz * f >= 1e9;
}

static PanelParams panel_narrow_params() {
  PanelParams p = panel_params();
  int d = g_tune_panel_narrow_dmin.load(std::memory_order_relaxed);
  p.dmin = d > 0 ? d : kPanelNarrowDmin;
  p.emin = p.dmin;  // no staged tiles: a tile is dense or its entries stay in the rest matrix
  return p;
}

// The dense part of C = A B for a narrow B: partial rows in *P (row r: P + dslot[r] * f), stream scratch.
static int launch_panel_narrow(const PanelPlan &pp, const float *B, int64_t ldb, int32_t f, float **P_out, hipStream_t stream) {
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotE, (size_t)pp.nblocks * kPanelRows * f * sizeof(float), &p));
  float *P = (float *)p;
  {
    ProfScope prof("spmm_panel_dense", f, stream);
#define CG_PANEL_NARROW(NB)                                                                                            \
  case NB:                                                                                                             \
    spmm_panel_dense_narrow_kernel<NB><<<(unsigned)pp.ndwg, kDenseThreads, 0, stream>>>(                               \
        pp.dwg_unit, pp.dunit_tile, pp.dunit_block, pp.dhdr, pp.dA, B, ldb, P, f);                                     \
    break;
    switch ((f + 15) / 16) {
      CG_PANEL_NARROW(1)
      CG_PANEL_NARROW(2)
      CG_PANEL_NARROW(3)
      CG_PANEL_NARROW(4)
      default:
        CG_FAIL(CG_ERR_UNSUPPORTED, "narrow panel product: no kernel for f=%d", f);
    }
#undef CG_PANEL_NARROW
    CG_LAUNCH_CHECK();
    if (pp.nsplit > 0) {
      const dim3 grid((unsigned)ceil_div64((int64_t)kPanelRows * f, kSpmmThreads), (unsigned)pp.nsplit);
      panel_reduce_kernel<<<grid, kSpmmThreads, 0, stream>>>(pp.split, P, f, kPanelRows);
      CG_LAUNCH_CHECK();
    }
  }
  *P_out = P;
  return CG_OK;
}

static int launch_panel_add_rows(const PanelPlan &pp, const float *P, float *C, int64_t ldc, int32_t rows, int32_t f,
                                 hipStream_t stream) {
  ProfScope prof("spmm_panel_add", f, stream);
  panel_add_rows_kernel<<<(unsigned)ceil_div64((int64_t)rows * f, kSpmmThreads), kSpmmThreads, 0, stream>>>(C, ldc, P, pp.dslot,
                                                                                                            rows, f);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

}  // namespace cg
