// Tall-skinny dense products of GCNFunc on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: exact
// fp32 multiply-add, 16x16 output tile per wavefront, 4 reduction steps per instruction).
// One dimension of each product is the vertex count, the others are feature widths of 16..602, so
// each kernel is one pass over a large operand; the matrix instruction is used because it turns a
// 64-lane load straight into 1024 multiply-adds without staging the large operand in LDS.
//
// Register layout of the instruction (lane l of 64):
//   A (16 x 4): lane holds A[l % 16][l / 16]        B (4 x 16): lane holds B[l / 16][l % 16]
//   D (16 x 16) in 4 registers: register v of lane l holds D[4 * (l / 16) + v][l % 16]
//
//   xw_mfma  : Z[n, fo]   = X[n, k] * W[k, fo]  (+ReLU)   computed as Z^T = W^T X^T: rows of X on the tile
//                                                         columns, W staged in LDS
//   xtg_mfma : dW[k, fo]  = X[n, k]^T * G[n, fo]          columns of X on the tile rows, vertices reduced
// (dX = G W^T is bound by its stores: dense_rows.hip for wide results, the vector kernel of dense.hip
// for narrow ones.)
#include "common.h"

namespace cg {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kMfmaThreads = 256;
constexpr int kMfmaWaves = kMfmaThreads / kWave;

__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// r = the VEC floats at p.  Loads are unconditional, from an address clamped into the operand, and
// the values of dead lanes are zeroed where they are consumed (keep_k): with no branch around the
// load and no use right behind it, the compiler counts outstanding loads exactly and loads issued
// for a later step stay in flight across the multiplies of the current one.
template <int VEC>
__device__ __forceinline__ void load_k(const float *p, float (&r)[VEC]) {
  if (VEC == 4) {
    const float4 t = *reinterpret_cast<const float4 *>(p);
    r[0] = t.x; r[1 % VEC] = t.y; r[2 % VEC] = t.z; r[3 % VEC] = t.w;
  } else if (VEC == 2) {
    const float2 t = *reinterpret_cast<const float2 *>(p);
    r[0] = t.x; r[1 % VEC] = t.y;
  } else {
    r[0] = p[0];
  }
}
__device__ __forceinline__ float keep_k(bool ok, float v) { return ok ? v : 0.f; }

// ---------------------------------------------------------------------------------------------
// Z = X W.  A wavefront owns 16 rows of X; lane (m, q) = (l % 16, l / 16) reads VEC consecutive
// k-values of row m per step, which feed VEC instructions as the B operand (X^T); the A operand
// (W^T) comes from the W chunk staged in LDS.  NT output tiles of 16 columns share every X value.
// ---------------------------------------------------------------------------------------------
constexpr int kXwChunk = 256;        // rows of W staged per pass when W does not fit LDS whole
constexpr int kXwLdsBytes = 64 * 1024;

constexpr int kXwSteps = 4;  // load steps a wavefront keeps in flight

// acc += X[row, c0 + kb .. c0 + kb + NS * STEP) * Ws for NS load steps.  Every load of X and every
// LDS read of W is issued before the first multiply (the scheduling barrier keeps the compiler from
// sinking them between the multiplies).  RAGGED: the last step crosses the end of the chunk; its
// lanes past clen read a clamped address of X and contribute zeros.
template <int VEC, int NT, int NS, bool RAGGED>
__device__ __forceinline__ void xw_span(const float *__restrict__ xrow, int32_t c0, int32_t clen, int32_t kb,
                                        const float *__restrict__ Ws, int m, int q, floatx4 (&acc)[NT]) {
  constexpr int STEP = 4 * VEC;  // k-values one load step covers
  float x[NS][VEC], w[NS][VEC][NT];
#pragma unroll
  for (int u = 0; u < NS; ++u) {
    const int32_t kk = kb + u * STEP + q * VEC;
    const bool live = !RAGGED || u < NS - 1 || kk < clen;  // VEC divides the chunk length: all or nothing
    load_k<VEC>(xrow + c0 + (live ? kk : 0), x[u]);
#pragma unroll
    for (int s = 0; s < VEC; ++s)  // rows clen .. round_up(clen, span) of Ws exist and hold zeros
#pragma unroll
      for (int t = 0; t < NT; ++t) w[u][s][t] = Ws[(size_t)(kk + s) * (16 * NT) + t * 16 + m];
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int u = 0; u < NS; ++u) {
    const bool live = !RAGGED || u < NS - 1 || kb + u * STEP + q * VEC < clen;
#pragma unroll
    for (int s = 0; s < VEC; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = mfma16(w[u][s][t], keep_k(live, x[u][s]), acc[t]);
  }
}

// acc += X[rows of the wave, c0 .. c0+clen) * Ws, for the chunk of W staged in LDS (zero padded to whole spans)
template <int VEC, int NT>
__device__ __forceinline__ void xw_accumulate(const float *__restrict__ xrow, int32_t c0, int32_t clen,
                                              const float *__restrict__ Ws, int m, int q, floatx4 (&acc)[NT]) {
  constexpr int STEP = 4 * VEC, SPAN = STEP * kXwSteps;
  int32_t kb = 0;
  for (; kb + SPAN <= clen; kb += SPAN) xw_span<VEC, NT, kXwSteps, false>(xrow, c0, clen, kb, Ws, m, q, acc);
  const int32_t left = clen - kb;  // < SPAN: up to kXwSteps - 1 whole steps and maybe a ragged one
  static_assert(kXwSteps == 4, "the tail dispatch below lists the step counts of a 4-step span");
  switch ((left + STEP - 1) / STEP) {  // wave-uniform
    case 1:
      if (left % STEP) xw_span<VEC, NT, 1, true>(xrow, c0, clen, kb, Ws, m, q, acc);
      else xw_span<VEC, NT, 1, false>(xrow, c0, clen, kb, Ws, m, q, acc);
      break;
    case 2:
      if (left % STEP) xw_span<VEC, NT, 2, true>(xrow, c0, clen, kb, Ws, m, q, acc);
      else xw_span<VEC, NT, 2, false>(xrow, c0, clen, kb, Ws, m, q, acc);
      break;
    case 3:
      if (left % STEP) xw_span<VEC, NT, 3, true>(xrow, c0, clen, kb, Ws, m, q, acc);
      else xw_span<VEC, NT, 3, false>(xrow, c0, clen, kb, Ws, m, q, acc);
      break;
    case 4:  // left < SPAN: the fourth step is ragged
      xw_span<VEC, NT, 4, true>(xrow, c0, clen, kb, Ws, m, q, acc);
      break;
    default:
      break;
  }
}

// rows past the end of the chunk are read (as zeros) by the last load steps: they are staged too
template <int VEC, int NT>
__device__ __forceinline__ void xw_stage(const float *__restrict__ W, int64_t ldw, int32_t c0, int32_t clen,
                                         int32_t fo, float *__restrict__ Ws, int32_t cap) {
  constexpr int kStepRows = 4 * VEC * kXwSteps;
  int32_t stage_rows = (clen + kStepRows - 1) / kStepRows * kStepRows;
  if (stage_rows > cap) stage_rows = cap;
  for (int idx = threadIdx.x; idx < stage_rows * 16 * NT; idx += kMfmaThreads) {
    const int kk = idx / (16 * NT), c = idx % (16 * NT);
    Ws[idx] = (kk < clen && c < fo) ? W[(int64_t)(c0 + kk) * ldw + c] : 0.f;
  }
}

// The accumulators hold the transposed tile (W^T on the A side, X^T on the B side): register v of
// lane (m, q) is Z[r0 + m][16 t + 4 q + v], so a lane stores four consecutive columns of one row and
// a wavefront writes whole 64-byte row pieces (the whole 1 KB tile when ldz = 16).
template <int NT>
__device__ __forceinline__ void xw_store(const floatx4 (&acc)[NT], float *__restrict__ Z, int64_t ldz, int64_t r0,
                                         int64_t n, int32_t fo, int relu, int m, int q) {
  const int64_t orow = r0 + m;
  if (orow >= n) return;
  const bool vec_ok = ldz % 4 == 0 && ((uintptr_t)Z) % 16 == 0;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int32_t col = t * 16 + 4 * q;
    floatx4 o = acc[t];
    if (relu) {
#pragma unroll
      for (int v = 0; v < 4; ++v) o[v] = o[v] < 0.f ? 0.f : o[v];
    }
    float *dst = Z + orow * ldz + col;
    if (vec_ok && col + 4 <= fo) {
      *reinterpret_cast<floatx4 *>(dst) = o;
    } else {
#pragma unroll
      for (int v = 0; v < 4; ++v)
        if (col + v < fo) dst[v] = o[v];
    }
  }
}

// cap: rows of W the LDS buffer holds.  cap >= k: W is staged once and the workgroup then walks row
// tiles (grid-stride) without another barrier; otherwise one row tile per workgroup, W in chunks.
template <int VEC, int NT>
__global__ __launch_bounds__(kMfmaThreads) void xw_mfma_kernel(const float *__restrict__ X, int64_t ldx,
                                                               const float *__restrict__ W, int64_t ldw,
                                                               float *__restrict__ Z, int64_t ldz, int64_t n,
                                                               int32_t k, int32_t fo, int relu, int32_t cap) {
  extern __shared__ float Ws[];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int m = lane & 15, q = lane >> 4;
  const int64_t tiles = (n + 16 * kMfmaWaves - 1) / (16 * kMfmaWaves);
  if (cap >= k) {
    xw_stage<VEC, NT>(W, ldw, 0, k, fo, Ws, cap);
    __syncthreads();
    for (int64_t tb = blockIdx.x; tb < tiles; tb += gridDim.x) {
      const int64_t r0 = (tb * kMfmaWaves + wave) * 16;
      int64_t row = r0 + m;
      if (row >= n) row = n - 1;  // clamp: the extra rows are computed and dropped
      floatx4 acc[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
      xw_accumulate<VEC, NT>(X + row * ldx, 0, k, Ws, m, q, acc);
      xw_store<NT>(acc, Z, ldz, r0, n, fo, relu, m, q);
    }
    return;
  }
  const int64_t r0 = ((int64_t)blockIdx.x * kMfmaWaves + wave) * 16;
  int64_t row = r0 + m;
  if (row >= n) row = n - 1;
  floatx4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int32_t c0 = 0; c0 < k; c0 += cap) {
    const int32_t clen = k - c0 < cap ? k - c0 : cap;
    __syncthreads();
    xw_stage<VEC, NT>(W, ldw, c0, clen, fo, Ws, cap);
    __syncthreads();
    xw_accumulate<VEC, NT>(X + row * ldx, c0, clen, Ws, m, q, acc);
  }
  xw_store<NT>(acc, Z, ldz, r0, n, fo, relu, m, q);
}

// ---------------------------------------------------------------------------------------------
// dW = X^T G.  A wavefront owns CT adjacent column tiles of X (16 * VEC columns each: the whole
// row when k <= CT * 16 * VEC) and all fo columns of G, and walks a contiguous range of vertices
// 4 at a time: lane (m, q) reads VEC consecutive columns per tile of vertex row r + q, lane (j, q)
// of the B side reads G[r + q][16 t + j].  A wavefront therefore reads whole contiguous pieces of
// rows by itself -- rows split between wavefronts at boundaries that are not cache-line aligned
// were measured a fifth slower -- and writes one partial product; the partial products of all
// ranges are added in order afterwards.
// ---------------------------------------------------------------------------------------------
template <int CT>
struct XtgSteps {  // 4-vertex steps in flight: about 8 to 10 loads of X per lane
  static constexpr int value = CT == 1 ? 8 : CT == 2 ? 4 : CT == 3 ? 3 : 2;
};

template <int VEC, int NT, int CT>
__global__ __launch_bounds__(kWave) void xtg_mfma_kernel(const float *__restrict__ X, int64_t ldx,
                                                         const float *__restrict__ G, int64_t ldg,
                                                         float *__restrict__ P, int64_t n, int32_t k, int32_t fo,
                                                         int64_t rows_per_range) {
  constexpr int U = XtgSteps<CT>::value;
  const int lane = threadIdx.x, m = lane & 15, q = lane >> 4;
  const int32_t kt0 = blockIdx.y * (CT * 16 * VEC);  // first column of this wavefront
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_range;
  const int64_t r1 = r0 + rows_per_range < n ? r0 + rows_per_range : n;

  // VEC divides k: the columns of a lane are all inside or all outside
  int32_t xoff[CT];
  bool xlive[CT];
  int32_t goff[NT];
  bool glive[NT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int32_t col = kt0 + c * 16 * VEC + m * VEC;
    xlive[c] = col + VEC <= k;
    xoff[c] = xlive[c] ? col : 0;
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    glive[t] = t * 16 + m < fo;
    goff[t] = glive[t] ? t * 16 + m : 0;
  }

  floatx4 acc[CT][VEC][NT];
#pragma unroll
  for (int c = 0; c < CT; ++c)
#pragma unroll
    for (int s = 0; s < VEC; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t) acc[c][s][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int64_t r = r0; r < r1; r += 4 * U) {
    float x[U][CT][VEC], g[U][NT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t rr = r + u * 4 + q;
      const int64_t row = rr < r1 ? rr : r0;  // clamped, dropped below
#pragma unroll
      for (int c = 0; c < CT; ++c) load_k<VEC>(X + row * ldx + xoff[c], x[u][c]);
#pragma unroll
      for (int t = 0; t < NT; ++t) g[u][t] = G[row * ldg + goff[t]];
    }
    __builtin_amdgcn_sched_barrier(0);  // every load of the round is issued before its first multiply
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool live = r + u * 4 + q < r1;
#pragma unroll
      for (int t = 0; t < NT; ++t) g[u][t] = keep_k(live && glive[t], g[u][t]);
#pragma unroll
      for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int s = 0; s < VEC; ++s) {
          const float xv = keep_k(live && xlive[c], x[u][c][s]);
#pragma unroll
          for (int t = 0; t < NT; ++t) acc[c][s][t] = mfma16(xv, g[u][t], acc[c][s][t]);
        }
    }
  }
  float *out = P + (int64_t)blockIdx.x * k * fo;
#pragma unroll
  for (int c = 0; c < CT; ++c)
#pragma unroll
    for (int s = 0; s < VEC; ++s)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          // tile row i = 4q + v of tile c holds column kt0 + 16 c VEC + i VEC + s
          const int32_t kc = kt0 + c * 16 * VEC + (4 * q + v) * VEC + s;
          const int32_t col = t * 16 + m;
          if (kc < k && col < fo) out[(int64_t)kc * fo + col] = acc[c][s][t][v];
        }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
// widest aligned load that divides k, so no load straddles the end of a row
static int pick_kvec(const float *X, int64_t ldx, int32_t k) {
  if (ldx % 4 == 0 && ((uintptr_t)X) % 16 == 0 && k % 4 == 0) return 4;
  if (ldx % 2 == 0 && ((uintptr_t)X) % 8 == 0 && k % 2 == 0) return 2;
  return 1;
}

int xw_mfma(const float *X, int64_t ldx, const float *W, int64_t ldw, float *Z, int64_t ldz, int64_t n, int32_t k,
            int32_t fo, int relu, hipStream_t stream) {
  const int nt = (fo + 15) / 16;
  const int vec = pick_kvec(X, ldx, k);
  const int64_t tiles = ceil_div64(n, 16 * kMfmaWaves);
  if (tiles > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "cg_dense_xw: grid too large");
  // W whole in LDS when it fits (rows rounded up to what the last load steps touch)
  const int step_rows = 4 * vec * kXwSteps;
  const int64_t whole = ceil_div64(k, step_rows) * step_rows;
  const size_t row_bytes = (size_t)16 * nt * sizeof(float);
  int32_t cap = kXwChunk;
  int64_t blocks = tiles;
  if ((size_t)whole * row_bytes <= (size_t)kXwLdsBytes) {
    cap = (int32_t)whole;
    const int64_t resident = 256 * 8;  // workgroups that keep every CU busy; each walks several row tiles
    if (blocks > resident) blocks = resident;
  }
  const unsigned grid = (unsigned)blocks;
  const size_t lds = (size_t)cap * row_bytes;
#define CG_CASE(V, T)                                                                                         \
  if (vec == V && nt == T) {                                                                                  \
    xw_mfma_kernel<V, T><<<grid, kMfmaThreads, lds, stream>>>(X, ldx, W, ldw, Z, ldz, n, k, fo, relu, cap);   \
    CG_LAUNCH_CHECK();                                                                                        \
    return CG_OK;                                                                                             \
  }
#define CG_CASES(V) CG_CASE(V, 1) CG_CASE(V, 2) CG_CASE(V, 3) CG_CASE(V, 4)
  CG_CASES(1) CG_CASES(2) CG_CASES(4)
#undef CG_CASES
#undef CG_CASE
  CG_FAIL(CG_ERR_UNSUPPORTED, "cg_dense_xw: fo=%d has no matrix-core variant", fo);
}

// Columns of X a lane reads per vertex: as wide as alignment allows, but no wider than keeps the 16
// lanes of a tile row on live columns (k = 16 -> one column per lane).
static int xtg_vec(const float *X, int64_t ldx, int32_t k) {
  int vec = pick_kvec(X, ldx, k);
  while (vec > 1 && 16 * vec > k) vec >>= 1;
  return vec;
}

// column tiles one wavefront owns: bounded by the accumulator registers (CT * VEC * NT tiles of 4)
static int xtg_tiles_per_wave(int32_t k, int vec, int nt, int64_t *groups) {
  const int64_t tiles = ceil_div64(k, 16 * vec);
  const int cap = nt == 1 ? 5 : (nt == 2 ? 3 : 2);
  *groups = ceil_div64(tiles, cap);
  return (int)ceil_div64(tiles, *groups);
}

// Vertex ranges of X^T G: one wavefront per (range, column group).  About 4096 wavefronts in all
// (several per SIMD in flight, with slack so the last ones do not run alone), ranges of at least
// 512 vertices so the partial product a range writes stays small beside what it reads and a
// wavefront lives long enough to pay for its start (232,965 x 602: 154 us with 256, 132 with 512,
// 169 with 768).
void xtg_plan(const float *X, int64_t ldx, int64_t n, int32_t k, int32_t fo, int64_t *nranges,
              int64_t *rows_per_range) {
  int64_t groups = 1;
  xtg_tiles_per_wave(k, xtg_vec(X, ldx, k), (fo + 15) / 16, &groups);
  int64_t ranges = ceil_div64(4096, groups);
  int64_t rows = ceil_div64(ceil_div64(n, ranges), 16) * 16;
  if (rows < 512) rows = 512;
  *rows_per_range = rows;
  *nranges = ceil_div64(n, rows);
}

int xtg_mfma(const float *X, int64_t ldx, const float *G, int64_t ldg, float *P, int64_t n, int32_t k, int32_t fo,
             int64_t rows_per_range, int64_t nranges, hipStream_t stream) {
  const int nt = (fo + 15) / 16;
  const int vec = xtg_vec(X, ldx, k);
  int64_t groups = 1;
  const int ct = xtg_tiles_per_wave(k, vec, nt, &groups);
  if (nranges > 0x7fffffffLL || groups > 65535) CG_FAIL(CG_ERR_SIZE, "cg_dense_xtg: grid too large");
  dim3 grid((unsigned)nranges, (unsigned)groups);
#define CG_CASE(V, T, C)                                                                                      \
  if (vec == V && nt == T && ct == C) {                                                                       \
    xtg_mfma_kernel<V, T, C><<<grid, kWave, 0, stream>>>(X, ldx, G, ldg, P, n, k, fo, rows_per_range);        \
    CG_LAUNCH_CHECK();                                                                                        \
    return CG_OK;                                                                                             \
  }
#define CG_CASES(V)                                                                                           \
  CG_CASE(V, 1, 1) CG_CASE(V, 1, 2) CG_CASE(V, 1, 3) CG_CASE(V, 1, 4) CG_CASE(V, 1, 5) CG_CASE(V, 2, 1)       \
  CG_CASE(V, 2, 2) CG_CASE(V, 2, 3) CG_CASE(V, 3, 1) CG_CASE(V, 3, 2) CG_CASE(V, 4, 1) CG_CASE(V, 4, 2)
  CG_CASES(1) CG_CASES(2) CG_CASES(4)
#undef CG_CASES
#undef CG_CASE
  CG_FAIL(CG_ERR_UNSUPPORTED, "cg_dense_xtg: fo=%d has no matrix-core variant", fo);
}

}  // namespace cg
