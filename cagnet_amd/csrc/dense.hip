// Tall-skinny dense products of GCNFunc (torch.mm at gcn_distr.py:275, :330, :187) as one
// LDS-tiled fp32 kernel: C[M,N] = op(A)[M,K] * op(B)[K,N], 256 threads per workgroup, a 4x4
// register tile per thread, K consumed 16 at a time.  One of M, N, K is the vertex count and the
// other two are feature widths (16..602), so each product streams one large operand once from HBM
// and is bandwidth bound; the tiles are shaped so that operand is read with full cache lines.
//   xw : A = X (row-major, normal), B = W (normal)           M = n, K = k,  N = fo
//   gwt: A = G (normal),            B = W^T (W is k x fo)    M = n, K = fo, N = k
//   xtg: A = X^T (X is n x k),      B = G (normal)           M = k, K = n,  N = fo, split over K:
//        every K-slice writes a partial product, a second kernel adds the slices in order.
#include "common.h"

#include <atomic>

namespace cg {

// dense_mfma.hip
int xw_mfma(const float *X, int64_t ldx, const float *W, int64_t ldw, float *Z, int64_t ldz, int64_t n, int32_t k,
            int32_t fo, int relu, hipStream_t stream);
int xtg_mfma(const float *X, int64_t ldx, const float *G, int64_t ldg, float *P, int64_t n, int32_t k, int32_t fo,
             int64_t rows_per_block, int64_t nblocks, hipStream_t stream);
void xtg_plan(const float *X, int64_t ldx, int64_t n, int32_t k, int32_t fo, int64_t *nranges,
              int64_t *rows_per_range);
// dense_rows.hip
int gwt_rows(const float *G, int64_t ldg, const float *W, int64_t ldw, float *dX, int64_t lddx, int64_t n, int32_t k,
             int32_t fo, hipStream_t stream);

// cg_tune_set("dense_mfma", -1) routes every product through the LDS-tiled vector kernel below
std::atomic<int> g_tune_dense_mfma{0};

constexpr int kGemmThreads = 256;
constexpr int kKT = 16;  // K tile

struct GemmArgs {
  const float *A;
  int64_t lda;
  const float *B;
  int64_t ldb;
  float *C;       // output, or partial slices [split][M][N] when splits > 1 (then ldc == N)
  int64_t ldc;
  int64_t M;
  int32_t N;
  int64_t K;
  int64_t kchunk;  // K range per grid.z slice (multiple of kKT)
  int32_t splits;
  int32_t relu;
};

// AT: A is stored transposed (element (r, kk) at A[kk*lda + r]).  BT likewise for B.
template <int BN, bool AT, bool BT>
__global__ __launch_bounds__(kGemmThreads) void gemm_tile_kernel(const GemmArgs g) {
  constexpr int BM = 4096 / BN;
  constexpr int CQ = BN / 4;  // column quads per tile
  __shared__ __attribute__((aligned(16))) float As[kKT][BM];
  __shared__ __attribute__((aligned(16))) float Bs[kKT][BN];

  const int t = threadIdx.x;
  const int64_t m0 = (int64_t)blockIdx.x * BM;
  const int32_t n0 = blockIdx.y * BN;
  const int tx = t % CQ, ty = t / CQ;
  const int64_t kbeg = (int64_t)blockIdx.z * g.kchunk;
  const int64_t kend = kbeg + g.kchunk < g.K ? kbeg + g.kchunk : g.K;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const bool a_vec4 = !AT && (g.lda % 4 == 0) && (((uintptr_t)g.A) % 16 == 0);
  const bool a_vec2 = !AT && (g.lda % 2 == 0) && (((uintptr_t)g.A) % 8 == 0);

  for (int64_t k0 = kbeg; k0 < kend; k0 += kKT) {
    // ---- A tile -> As[kk][r]
    if (!AT) {
      constexpr int TPR = kGemmThreads / BM > 0 ? kGemmThreads / BM : 1;  // threads per row
      constexpr int KPT = kKT / TPR;                                      // consecutive k per thread
      constexpr int RPT = BM / (kGemmThreads / TPR);                      // rows per thread (BM = 256 -> 1)
#pragma unroll
      for (int rr = 0; rr < RPT; ++rr) {
        const int r = (t % (kGemmThreads / TPR)) + rr * (kGemmThreads / TPR);
        const int kk0 = (t / (kGemmThreads / TPR)) * KPT;
        const int64_t row = m0 + r;
        float v[KPT];
#pragma unroll
        for (int i = 0; i < KPT; ++i) v[i] = 0.f;
        if (row < g.M) {
          const float *src = g.A + row * g.lda + k0 + kk0;
          if (k0 + kk0 + KPT <= kend) {
            if (KPT % 4 == 0 && a_vec4) {
#pragma unroll
              for (int i = 0; i < KPT; i += 4) {
                const float4 q = *reinterpret_cast<const float4 *>(src + i);
                v[i] = q.x; v[i + 1] = q.y; v[i + 2] = q.z; v[i + 3] = q.w;
              }
            } else if (KPT % 2 == 0 && a_vec2) {
#pragma unroll
              for (int i = 0; i < KPT; i += 2) {
                const float2 q = *reinterpret_cast<const float2 *>(src + i);
                v[i] = q.x; v[i + 1] = q.y;
              }
            } else {
#pragma unroll
              for (int i = 0; i < KPT; ++i) v[i] = src[i];
            }
          } else {
#pragma unroll
            for (int i = 0; i < KPT; ++i)
              if (k0 + kk0 + i < kend) v[i] = src[i];
          }
        }
#pragma unroll
        for (int i = 0; i < KPT; ++i) As[kk0 + i][r] = v[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < (BM * kKT) / kGemmThreads; ++i) {
        const int idx = i * kGemmThreads + t;
        const int kk = idx / BM, r = idx % BM;
        float v = 0.f;
        if (m0 + r < g.M && k0 + kk < kend) v = g.A[(k0 + kk) * g.lda + m0 + r];
        As[kk][r] = v;
      }
    }
    // ---- B tile -> Bs[kk][c]
    if (!BT) {
#pragma unroll
      for (int i = 0; i < (BN * kKT + kGemmThreads - 1) / kGemmThreads; ++i) {
        const int idx = i * kGemmThreads + t;
        if (idx < BN * kKT) {
          const int kk = idx / BN, c = idx % BN;
          float v = 0.f;
          if (n0 + c < g.N && k0 + kk < kend) v = g.B[(k0 + kk) * g.ldb + n0 + c];
          Bs[kk][c] = v;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < (BN * kKT + kGemmThreads - 1) / kGemmThreads; ++i) {
        const int idx = i * kGemmThreads + t;
        if (idx < BN * kKT) {
          const int kk = idx % kKT, c = idx / kKT;
          float v = 0.f;
          if (n0 + c < g.N && k0 + kk < kend) v = g.B[(int64_t)(n0 + c) * g.ldb + k0 + kk];
          Bs[kk][c] = v;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kKT; ++kk) {
      const float4 a4 = *reinterpret_cast<const float4 *>(&As[kk][ty * 4]);
      const float4 b4 = *reinterpret_cast<const float4 *>(&Bs[kk][tx * 4]);
      const float av[4] = {a4.x, a4.y, a4.z, a4.w};
      const float bv[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }

  float *Cbase = g.C;
  int64_t ldc = g.ldc;
  if (g.splits > 1) Cbase += (int64_t)blockIdx.z * g.M * g.N;
  const int32_t c0 = n0 + tx * 4;
  const bool full4 = c0 + 4 <= g.N;
  const bool st4 = full4 && (ldc % 4 == 0) && (((uintptr_t)Cbase) % 16 == 0);
  const bool st2 = full4 && (ldc % 2 == 0) && (((uintptr_t)Cbase) % 8 == 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t row = m0 + ty * 4 + i;
    if (row >= g.M) continue;
    float o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = (g.relu && acc[i][j] < 0.f) ? 0.f : acc[i][j];
    float *dst = Cbase + row * ldc + c0;
    if (st4) {
      *reinterpret_cast<float4 *>(dst) = make_float4(o[0], o[1], o[2], o[3]);
    } else if (st2) {
      *reinterpret_cast<float2 *>(dst) = make_float2(o[0], o[1]);
      *reinterpret_cast<float2 *>(dst + 2) = make_float2(o[2], o[3]);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (c0 + j < g.N) dst[j] = o[j];
    }
  }
}

// C[i] = sum over slices z of P[z][i].  A workgroup owns 16 consecutive outputs; its 16 z-lanes
// per output add slices z, z+16, ... in order and are then combined by a fixed xor butterfly, so
// the order of additions depends only on the number of slices.
constexpr int kSumOut = 16;
__global__ __launch_bounds__(kGemmThreads) void gemm_slice_sum_kernel(const float *__restrict__ P, int64_t elems,
                                                                      int32_t splits, float *__restrict__ C,
                                                                      int64_t ldc, int32_t N) {
  const int e = threadIdx.x % kSumOut;
  const int zl = threadIdx.x / kSumOut;  // 0..15; the 16 z-lanes of one output sit 16 lanes apart
  const int64_t idx = (int64_t)blockIdx.x * kSumOut + e;
  float s = 0.f;
  if (idx < elems)
    for (int32_t z = zl; z < splits; z += kGemmThreads / kSumOut) s += P[(int64_t)z * elems + idx];
  // lanes of one wave: zl = 4*wave + lane/16 -> combine the 4 z-lanes inside the wave, then the 4 waves
  s += __shfl_xor(s, 16, kWave);
  s += __shfl_xor(s, 32, kWave);
  __shared__ float part[kGemmThreads / kWave][kSumOut];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane < kSumOut) part[wave][lane] = s;
  __syncthreads();
  if (threadIdx.x < kSumOut && idx < elems) {
    float t = part[0][e];
#pragma unroll
    for (int w = 1; w < kGemmThreads / kWave; ++w) t += part[w][e];
    C[(idx / N) * ldc + (idx % N)] = t;
  }
}

template <bool AT, bool BT>
static int launch_gemm(GemmArgs g, hipStream_t stream) {
  if (g.M == 0 || g.N == 0) return CG_OK;
  const int bn = g.N <= 16 ? 16 : (g.N <= 32 ? 32 : 64);
  const int bm = 4096 / bn;
  const int64_t gy = ceil_div64(g.M, bm);
  const int64_t gx = ceil_div64(g.N, bn);
  // grid.x takes the row tiles (up to 2^31-1 of them); y and z are limited to 65535
  if (gy > 0x7fffffffLL || gx > 65535 || g.splits > 65535) CG_FAIL(CG_ERR_SIZE, "dense product: grid too large");
  dim3 grid((unsigned)gy, (unsigned)gx, (unsigned)g.splits);
  if (bn == 16) gemm_tile_kernel<16, AT, BT><<<grid, kGemmThreads, 0, stream>>>(g);
  else if (bn == 32) gemm_tile_kernel<32, AT, BT><<<grid, kGemmThreads, 0, stream>>>(g);
  else gemm_tile_kernel<64, AT, BT><<<grid, kGemmThreads, 0, stream>>>(g);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

static int check_gemm(const char *who, const void *a, const void *b, const void *c, int64_t n, int32_t k, int32_t fo) {
  if (n < 0 || k <= 0 || fo <= 0) CG_FAIL(CG_ERR_SIZE, "%s: bad sizes n=%lld k=%d fo=%d", who, (long long)n, k, fo);
  if (!b || !c || (n > 0 && !a)) CG_FAIL(CG_ERR_NULL, "%s: null operand", who);
  return CG_OK;
}

}  // namespace cg

extern "C" {

int cg_dense_xw(const float *d_X, int64_t ldx, const float *d_W, int64_t ldw, float *d_Z, int64_t ldz, int64_t n,
                int32_t k, int32_t fo, int relu, cg_stream_t stream) {
  using namespace cg;
  CG_TRY(check_gemm("cg_dense_xw", d_X, d_W, d_Z, n, k, fo));
  if (ldx < k || ldw < fo || ldz < fo) CG_FAIL(CG_ERR_SIZE, "cg_dense_xw: leading dimension too small");
  if (n == 0) return CG_OK;
  GemmArgs g{d_X, ldx, d_W, ldw, d_Z, ldz, n, fo, k, ceil_div64(k, kKT) * kKT, 1, relu ? 1 : 0};
  ProfScope prof("dense_xw", k, (hipStream_t)stream);
  if (fo <= 64 && g_tune_dense_mfma.load(std::memory_order_relaxed) >= 0)
    return xw_mfma(d_X, ldx, d_W, ldw, d_Z, ldz, n, k, fo, relu ? 1 : 0, (hipStream_t)stream);
  return launch_gemm<false, false>(g, (hipStream_t)stream);
}

int cg_dense_gwt(const float *d_G, int64_t ldg, const float *d_W, int64_t ldw, float *d_dX, int64_t lddx, int64_t n,
                 int32_t k, int32_t fo, cg_stream_t stream) {
  using namespace cg;
  CG_TRY(check_gemm("cg_dense_gwt", d_G, d_W, d_dX, n, k, fo));
  if (ldg < fo || ldw < fo || lddx < k) CG_FAIL(CG_ERR_SIZE, "cg_dense_gwt: leading dimension too small");
  if (n == 0) return CG_OK;
  GemmArgs g{d_G, ldg, d_W, ldw, d_dX, lddx, n, k, fo, ceil_div64(fo, kKT) * kKT, 1, 0};
  ProfScope prof("dense_gwt", k, (hipStream_t)stream);
  // wide result: bound by its stores, matrix-core tiles through an LDS row buffer (dense_rows.hip);
  // narrow result: the LDS-tiled vector kernel (the matrix-core form measured the same there)
  if (fo <= 64 && k > 64 && g_tune_dense_mfma.load(std::memory_order_relaxed) >= 0)
    return gwt_rows(d_G, ldg, d_W, ldw, d_dX, lddx, n, k, fo, (hipStream_t)stream);
  return launch_gemm<false, true>(g, (hipStream_t)stream);
}

int cg_dense_xtg(const float *d_X, int64_t ldx, const float *d_G, int64_t ldg, float *d_dW, int64_t lddw, int64_t n,
                 int32_t k, int32_t fo, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  CG_TRY(check_gemm("cg_dense_xtg", d_X, d_G, d_dW, n, k, fo));
  if (ldx < k || ldg < fo || lddw < fo) CG_FAIL(CG_ERR_SIZE, "cg_dense_xtg: leading dimension too small");
  if (fo <= 64 && n > 0 && g_tune_dense_mfma.load(std::memory_order_relaxed) >= 0) {
    ProfScope prof("dense_xtg", k, stream);
    int64_t nblocks = 0, rows_per_block = 0;
    xtg_plan(d_X, ldx, n, k, fo, &nblocks, &rows_per_block);
    const int64_t elems = (int64_t)k * fo;
    void *p = nullptr;
    CG_TRY(scratch_get(stream, kSlotA, (size_t)nblocks * elems * sizeof(float), &p));
    CG_TRY(xtg_mfma(d_X, ldx, d_G, ldg, (float *)p, n, k, fo, rows_per_block, nblocks, stream));
    gemm_slice_sum_kernel<<<(unsigned)ceil_div64(elems, kSumOut), kGemmThreads, 0, stream>>>(
        (const float *)p, elems, (int32_t)nblocks, d_dW, lddw, fo);
    CG_LAUNCH_CHECK();
    return CG_OK;
  }
  // slices over the vertex dimension: enough workgroups to fill 256 CUs several times over
  const int bn = fo <= 16 ? 16 : (fo <= 32 ? 32 : 64);
  const int64_t tiles = ceil_div64(k, 4096 / bn) * ceil_div64(fo, bn);
  int64_t splits = ceil_div64(2048, tiles);
  if (splits > 512) splits = 512;
  int64_t kchunk = ceil_div64(ceil_div64(n > 0 ? n : 1, splits), kKT) * kKT;
  if (kchunk < 4 * kKT) kchunk = 4 * kKT;
  splits = n > 0 ? ceil_div64(n, kchunk) : 1;
  GemmArgs g{d_X, ldx, d_G, ldg, d_dW, lddw, k, fo, n, kchunk, (int32_t)splits, 0};
  ProfScope prof("dense_xtg", k, stream);
  if (splits <= 1) {
    g.splits = 1;
    g.kchunk = ceil_div64(n > 0 ? n : 1, kKT) * kKT;
    return launch_gemm<true, false>(g, stream);
  }
  const int64_t elems = (int64_t)k * fo;
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotA, (size_t)splits * elems * sizeof(float), &p));
  g.C = (float *)p;
  g.ldc = fo;
  CG_TRY((launch_gemm<true, false>(g, stream)));
  gemm_slice_sum_kernel<<<(unsigned)ceil_div64(elems, kSumOut), kGemmThreads, 0, stream>>>(
      (const float *)p, elems, (int32_t)splits, d_dW, lddw, fo);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

}  // extern "C"
