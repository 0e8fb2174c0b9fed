// dX[n, k] = G[n, fo] * W[k, fo]^T for a wide result and a short reduction (k > 64, fo <= 64):
// the input-gradient product of the first layer (torch.mm(ag, weight.t()), gcn_distr.py:330).
//
// The product is bound by the n * k * 4 bytes it stores.  A thread owns VEC consecutive columns
// of dX and keeps their fo weights in registers; a workgroup steps through consecutive rows, so
// each step stores `rows per step` whole rows as one contiguous run.  The G rows of a workgroup are
// staged in LDS.
#include "common.h"

namespace cg {

constexpr int kRowsMaxThreads = 1024;

constexpr int kRowsLds = 16384;  // floats of G staged per workgroup

template <int FO, int VEC>
__global__ __launch_bounds__(kRowsMaxThreads) void gwt_rows_kernel(const float *__restrict__ G, int64_t ldg,
                                                                const float *__restrict__ W, int64_t ldw,
                                                                float *__restrict__ dX, int64_t lddx, int64_t n,
                                                                int32_t k, int32_t fo, int32_t tpr, int32_t nchunk,
                                                                int32_t rows_per_block) {
  // The G rows of the workgroup are staged in LDS once: the row loop then has no global load, so
  // it never waits on the memory counter its own stores are queued on.
  __shared__ __attribute__((aligned(16))) float Gs[kRowsLds];
  const int64_t r0 = (int64_t)blockIdx.x * rows_per_block;
  const int32_t nrows = (int32_t)(r0 + rows_per_block < n ? rows_per_block : n - r0);
  for (int32_t i = threadIdx.x; i < nrows * FO; i += blockDim.x) {
    const int32_t row = i / FO, j = i % FO;
    Gs[i] = j < fo ? G[(r0 + row) * ldg + j] : 0.f;
  }
  __syncthreads();
  const int rps = blockDim.x / tpr;  // rows per step
  const int rs = threadIdx.x / tpr, cv = threadIdx.x % tpr;
  if (rs >= rps) return;  // no barrier below
  for (int32_t chunk = 0; chunk < nchunk; ++chunk) {
    const int32_t col = (chunk * tpr + cv) * VEC;
    if (col >= k) continue;
    float w[VEC][FO];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const bool live = col + v < k;
      const float *wrow = W + (int64_t)(live ? col + v : col) * ldw;
#pragma unroll
      for (int j = 0; j < FO; ++j) w[v][j] = (live && j < fo) ? wrow[j] : 0.f;
    }
    for (int32_t rl = rs; rl < nrows; rl += rps) {
      float g[FO];
#pragma unroll
      for (int j = 0; j < FO; j += 4) {
        const float4 t = *reinterpret_cast<const float4 *>(&Gs[rl * FO + j]);
        g[j] = t.x;
        g[j + 1] = t.y;
        g[j + 2] = t.z;
        g[j + 3] = t.w;
      }
      float out[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < FO; ++j) s = fmaf(g[j], w[v][j], s);
        out[v] = s;
      }
      float *dst = dX + (r0 + rl) * lddx + col;
      if (col + VEC <= k) {
        if (VEC == 4) *reinterpret_cast<float4 *>(dst) = make_float4(out[0], out[1 % VEC], out[2 % VEC], out[3 % VEC]);
        else if (VEC == 2) *reinterpret_cast<float2 *>(dst) = make_float2(out[0], out[1 % VEC]);
        else dst[0] = out[0];
      } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v)
          if (col + v < k) dst[v] = out[v];
      }
    }
  }
}

int gwt_rows(const float *G, int64_t ldg, const float *W, int64_t ldw, float *dX, int64_t lddx, int64_t n, int32_t k,
             int32_t fo, hipStream_t stream) {
  if (fo > 64) CG_FAIL(CG_ERR_UNSUPPORTED, "gwt_rows: fo=%d exceeds 64", fo);
  const int FO = fo <= 8 ? 8 : (fo <= 16 ? 16 : (fo <= 24 ? 24 : (fo <= 32 ? 32 : (fo <= 48 ? 48 : 64))));
  int vec = 1;
  if (lddx % 4 == 0 && ((uintptr_t)dX) % 16 == 0) vec = 4;
  else if (lddx % 2 == 0 && ((uintptr_t)dX) % 8 == 0) vec = 2;
  while (vec > 1 && vec * FO > 64) vec >>= 1;  // the weights of a thread's columns stay in registers
  const int32_t cvs = (k + vec - 1) / vec;  // column vectors of a row
  // workgroup size: the one that leaves the fewest threads without a column
  int threads = 256, nchunk = 1, tpr = 1;
  double best = -1.0;
  for (int t = 256; t <= kRowsMaxThreads; t *= 2) {
    const int nc = (cvs + t - 1) / t;
    const int per = (cvs + nc - 1) / nc;  // threads per row
    const double used = (double)cvs / nc * (t / per) / t;
    if (used > best + 0.02) {
      best = used;
      threads = t;
      nchunk = nc;
      tpr = per;
    }
  }
  const int rps = threads / tpr;
  int32_t rows_per_block = rps * 128;  // amortises the weight loads of a workgroup
  if (rows_per_block > kRowsLds / FO) rows_per_block = kRowsLds / FO / rps * rps;
  if (rows_per_block < rps) rows_per_block = rps;
  const int64_t blocks = ceil_div64(n, rows_per_block);
  if (blocks > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "gwt_rows: grid too large");
#define CG_CASE(F, V)                                                                                        \
  if (FO == F && vec == V) {                                                                                 \
    gwt_rows_kernel<F, V><<<(unsigned)blocks, (unsigned)threads, 0, stream>>>(G, ldg, W, ldw, dX, lddx, n, k, fo, \
                                                                         tpr, nchunk, rows_per_block);          \
    CG_LAUNCH_CHECK();                                                                                       \
    return CG_OK;                                                                                            \
  }
  CG_CASE(8, 4) CG_CASE(8, 2) CG_CASE(8, 1)
  CG_CASE(16, 4) CG_CASE(16, 2) CG_CASE(16, 1)
  CG_CASE(24, 2) CG_CASE(24, 1)
  CG_CASE(32, 2) CG_CASE(32, 1)
  CG_CASE(48, 1) CG_CASE(64, 1)
#undef CG_CASE
  CG_FAIL(CG_ERR_UNSUPPORTED, "gwt_rows: no variant for fo=%d vec=%d", fo, vec);
}

}  // namespace cg
