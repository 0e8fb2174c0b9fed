// dX[n, k] = G[n, fo] * W[k, fo]^T for a wide result and a short reduction (k > 64, fo <= 64):
// the input-gradient product of the first layer (torch.mm(ag, weight.t()), gcn_distr.py:330).
//
// The product is bound by the n * k * 4 bytes it stores, so everything is arranged around the
// stores.  A wavefront owns 16 rows at a time and walks the column tiles of its chunk of W (staged
// in LDS) on the fp32 matrix core, computing the transposed tile (W on the A side, G^T on the B
// side) so that a lane ends up with 4 consecutive columns of one row.  Tiles go to a row buffer in
// LDS private to the wavefront; when the 16 rows are complete the wavefront copies them out as one
// run of consecutive 16-byte pieces (the whole 16 * k block when the rows are contiguous), i.e.
// every store instruction writes 1 KB of consecutive addresses.  Storing tiles straight from the
// accumulators (64-byte pieces of 16 rows per instruction) and a vector-ALU form (one thread per
// 4 columns, weights in registers) were both measured slower: the first stalls on the matrix-core
// results and writes partial lines, the second is bound by its multiply-adds.
#include "common.h"

namespace cg {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kGwtWaves = 4;  // wavefronts per workgroup: each brings a 16-row buffer of its own
constexpr int kGwtThreads = kGwtWaves * kWave;
constexpr int kGwtLdsBytes = 100 * 1024;
constexpr int kGwtGroup = 4;  // column tiles computed together
constexpr int kGwtCopy = 4;   // row-buffer pieces a lane copies out together

// FB: 16-wide blocks of the reduction (fo <= 16 FB).  GVEC 4: rows of G are read as 16-byte
// pieces; SVEC: floats per store of dX.
template <int FB, int GVEC, int SVEC>
__global__ __launch_bounds__(kGwtThreads) void gwt_mfma_kernel(const float *__restrict__ G, int64_t ldg,
                                                               const float *__restrict__ W, int64_t ldw,
                                                               float *__restrict__ dX, int64_t lddx, int64_t n,
                                                               int32_t k, int32_t fo, int32_t kc) {
  constexpr int FOP = 16 * FB;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int32_t c0 = blockIdx.y * kc;                    // first column of this chunk
  const int32_t kcl = k - c0 < kc ? k - c0 : kc;         // live columns of the chunk
  const int32_t ctiles = (kcl + 15) / 16;
  float *Ws = lds;                                        // [ctiles * 16][FOP], zero padded
  float *T = lds + (size_t)kc * FOP + (size_t)(threadIdx.x / kWave) * 16 * kc;  // [16][kc] of this wavefront
  for (int32_t i = threadIdx.x; i < ctiles * 16 * FOP; i += kGwtThreads) {
    const int32_t col = i / FOP, j = i % FOP;
    Ws[i] = (col < kcl && j < fo) ? W[(int64_t)(c0 + col) * ldw + j] : 0.f;
  }
  __syncthreads();

  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int m = lane & 15, q = lane >> 4;
  const int64_t tiles = (n + 15) / 16;
  const int64_t stride = (int64_t)gridDim.x * kGwtWaves;

  // reduction index of step (b, s) in lane (., q): 16 b + 4 q + s, the same on both operands
  auto load_g = [&](int64_t tb, float (&g)[FB][4]) {
    int64_t row = tb * 16 + m;
    if (row >= n) row = n - 1;  // clamped: those rows are not stored
    const float *gp = G + row * ldg;
#pragma unroll
    for (int b = 0; b < FB; ++b) {
      const int32_t j = 16 * b + 4 * q;
      if (GVEC == 4) {  // fo is a multiple of 4: a piece is inside or outside
        const float4 t = *reinterpret_cast<const float4 *>(gp + (j < fo ? j : 0));
        g[b][0] = t.x; g[b][1] = t.y; g[b][2] = t.z; g[b][3] = t.w;
      } else {
#pragma unroll
        for (int s = 0; s < 4; ++s) g[b][s] = gp[j + s < fo ? j + s : 0];
      }
    }
  };

  // copy-out geometry: the 16 x kcl block in pieces of SVEC floats, 64 pieces per instruction
  const int32_t rowvecs = kcl / SVEC;  // SVEC divides kcl
  const int32_t pieces = 16 * rowvecs;
  const int32_t dq = kWave / rowvecs, dr = kWave % rowvecs;
  const int lane0 = threadIdx.x & (kWave - 1);
  const int32_t rr0 = lane0 / rowvecs, cv0 = lane0 % rowvecs;

  int64_t tb = (int64_t)blockIdx.x * kGwtWaves + wave;
  if (tb >= tiles) return;  // no barrier below
  float g[FB][4], gn[FB][4];
  load_g(tb, gn);
  for (; tb < tiles; tb += stride) {
#pragma unroll
    for (int b = 0; b < FB; ++b)
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int32_t j = 16 * b + 4 * q + s;
        g[b][s] = j < fo ? gn[b][s] : 0.f;
      }
    // the rows of the next tile are requested before this tile's stores are queued
    load_g(tb + stride < tiles ? tb + stride : tb, gn);
    // column tiles in groups of kGwtGroup: the W pieces of the group are read first, then the
    // matrix instructions run round-robin over the group's independent accumulators (the
    // wavefront is alone on its SIMD most of the time, so the latency must be covered from inside)
    for (int32_t c = 0; c < ctiles; c += kGwtGroup) {
      floatx4 w[kGwtGroup][FB], acc[kGwtGroup];
#pragma unroll
      for (int t = 0; t < kGwtGroup; ++t) {
        const int32_t ct = c + t < ctiles ? c + t : ctiles - 1;  // past the end: recomputed, not written
        const float *wp = Ws + (size_t)(ct * 16 + m) * FOP + 4 * q;
#pragma unroll
        for (int b = 0; b < FB; ++b) w[t][b] = *reinterpret_cast<const floatx4 *>(wp + 16 * b);
        acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int b = 0; b < FB; ++b)
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
          for (int t = 0; t < kGwtGroup; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[t][b][s], g[b][s], acc[t], 0, 0, 0);
      // register v of lane (m, q) is dX[r0 + m][c0 + 16 (c + t) + 4 q + v]
#pragma unroll
      for (int t = 0; t < kGwtGroup; ++t)
        if (c + t < ctiles) *reinterpret_cast<floatx4 *>(T + (size_t)m * kc + (c + t) * 16 + 4 * q) = acc[t];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int64_t r0 = tb * 16;
    int32_t rr = rr0, cv = cv0;
    // kGwtCopy pieces per lane at a time: their LDS reads are issued together, then their stores
    for (int32_t p = lane; p < pieces; p += kGwtCopy * kWave) {
      float v[kGwtCopy][SVEC];
      float *dst[kGwtCopy];
      bool ok[kGwtCopy];
#pragma unroll
      for (int i = 0; i < kGwtCopy; ++i) {
        ok[i] = p + i * kWave < pieces && r0 + rr < n;
        const float *src = T + (size_t)(ok[i] ? rr : 0) * kc + cv * SVEC;
        dst[i] = dX + (r0 + rr) * lddx + c0 + cv * SVEC;
        if (SVEC == 4) {
          const floatx4 t = *reinterpret_cast<const floatx4 *>(src);
          v[i][0] = t[0]; v[i][1 % SVEC] = t[1]; v[i][2 % SVEC] = t[2]; v[i][3 % SVEC] = t[3];
        } else if (SVEC == 2) {
          const float2 t = *reinterpret_cast<const float2 *>(src);
          v[i][0] = t.x; v[i][1 % SVEC] = t.y;
        } else {
          v[i][0] = src[0];
        }
        rr += dq;
        cv += dr;
        if (cv >= rowvecs) {
          cv -= rowvecs;
          ++rr;
        }
      }
#pragma unroll
      for (int i = 0; i < kGwtCopy; ++i) {
        if (ok[i]) {
          if (SVEC == 4) *reinterpret_cast<floatx4 *>(dst[i]) = floatx4{v[i][0], v[i][1 % SVEC], v[i][2 % SVEC], v[i][3 % SVEC]};
          else if (SVEC == 2) *reinterpret_cast<float2 *>(dst[i]) = make_float2(v[i][0], v[i][1 % SVEC]);
          else dst[i][0] = v[i][0];
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}

int gwt_rows(const float *G, int64_t ldg, const float *W, int64_t ldw, float *dX, int64_t lddx, int64_t n, int32_t k,
             int32_t fo, hipStream_t stream) {
  if (fo > 64) CG_FAIL(CG_ERR_UNSUPPORTED, "gwt_rows: fo=%d exceeds 64", fo);
  const int fb = (fo + 15) / 16;
  const int gvec = (ldg % 4 == 0 && ((uintptr_t)G) % 16 == 0 && fo % 4 == 0) ? 4 : 1;
  // column chunk: W chunk and the row buffers of the wavefronts share the LDS budget; chunks start
  // at multiples of 16 columns
  const int32_t per_col = (16 * fb + kGwtWaves * 16) * (int32_t)sizeof(float);
  int32_t kc = kGwtLdsBytes / per_col / 16 * 16;
  const int32_t kpad = (k + 15) / 16 * 16;
  int64_t chunks = ceil_div64(kpad, kc);
  kc = (int32_t)(ceil_div64(ceil_div64(kpad, chunks), 16) * 16);  // even chunks
  chunks = ceil_div64(k, kc);
  // store width: pieces must not straddle the end of a chunk's live columns (kc is a multiple of 16,
  // so only the width of the last chunk, k - (chunks - 1) kc, matters) and must be aligned in dX
  int svec = 1;
  if (lddx % 4 == 0 && ((uintptr_t)dX) % 16 == 0 && k % 4 == 0) svec = 4;
  else if (lddx % 2 == 0 && ((uintptr_t)dX) % 8 == 0 && k % 2 == 0) svec = 2;
  const int64_t tiles = ceil_div64(n, 16);
  int64_t blocks = ceil_div64(tiles, kGwtWaves);
  if (chunks > 65535) CG_FAIL(CG_ERR_SIZE, "gwt_rows: grid too large");
  const size_t lds = (size_t)kc * per_col;
  // as many workgroups as are resident at once (LDS bound); each walks several row tiles
  int64_t per_cu = (160 * 1024) / (int64_t)lds;
  if (per_cu > 8) per_cu = 8;
  const int64_t resident = ceil_div64(256 * per_cu, chunks);
  if (blocks > resident) blocks = resident;
  dim3 grid((unsigned)blocks, (unsigned)chunks);
#define CG_CASE(F, GV, SV)                                                                                    \
  if (fb == F && gvec == GV && svec == SV) {                                                                  \
    if (lds > 64 * 1024) /* more than 64 KB of dynamic LDS must be asked for (per device, so on every launch) */ \
      CG_HIP(hipFuncSetAttribute((const void *)gwt_mfma_kernel<F, GV, SV>,                                     \
                                 hipFuncAttributeMaxDynamicSharedMemorySize, kGwtLdsBytes));                   \
    gwt_mfma_kernel<F, GV, SV><<<grid, kGwtThreads, lds, stream>>>(G, ldg, W, ldw, dX, lddx, n, k, fo, kc);   \
    CG_LAUNCH_CHECK();                                                                                        \
    return CG_OK;                                                                                             \
  }
#define CG_CASES(F) CG_CASE(F, 4, 4) CG_CASE(F, 4, 2) CG_CASE(F, 4, 1) CG_CASE(F, 1, 4) CG_CASE(F, 1, 2) CG_CASE(F, 1, 1)
  CG_CASES(1) CG_CASES(2) CG_CASES(3) CG_CASES(4)
#undef CG_CASES
#undef CG_CASE
  CG_FAIL(CG_ERR_UNSUPPORTED, "gwt_rows: no variant for fo=%d", fo);
}

}  // namespace cg
