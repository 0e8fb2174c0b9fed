// Device kernels of the CSR SpMM  C[rows,f] = beta*C + A*B  for gfx950 (64-wide wavefronts).
//
// Replaces cusparseSpMM(CSRMM_ALG1, alpha = 1, beta = 1) of the reference operator
// (sparse-extension/sparse_coo_tensor.cu:215-226) on row-major B and C, without atomics.
//
// Work decomposition
//   task    = a row segment: at most `seg` consecutive stored entries of one row.  Rows of degree
//             <= seg are one task and go straight to C; longer rows write one partial row per task
//             that spmm_reduce_kernel adds in segment order.
//   team    = LPR lanes that together cover the f output columns, VEC floats per lane and chunk.
//             A wavefront holds G = 64 / LPR teams.
//   window  = up to 64 consecutive tasks (a new window every S stored entries).  Tasks are
//             contiguous in the entry stream, so the wavefront that takes a window reads one
//             contiguous piece of (colind, val) and pays start-up latency once per window.
// Summation order is a function of the matrix, f and the schedule only: results are bit-identical
// from run to run.
#pragma once
#include "common.h"

namespace cg {

constexpr int kSpmmThreads = 256;
constexpr int kWavesPerBlock = kSpmmThreads / kWave;

template <int VEC>
struct VecT;
template <>
struct VecT<1> {
  typedef float type;
};
template <>
struct VecT<2> {
  typedef float2 type;
};
template <>
struct VecT<4> {
  typedef float4 type;
};

template <int VEC>
__device__ __forceinline__ void load_vec(const float *p, float (&r)[VEC]) {
  typedef typename VecT<VEC>::type V;
  const V t = *reinterpret_cast<const V *>(p);
  const float *tp = reinterpret_cast<const float *>(&t);
#pragma unroll
  for (int i = 0; i < VEC; ++i) r[i] = tp[i];
}

template <int VEC>
__device__ __forceinline__ void store_vec(float *p, const float (&r)[VEC]) {
  typedef typename VecT<VEC>::type V;
  V t;
  float *tp = reinterpret_cast<float *>(&t);
#pragma unroll
  for (int i = 0; i < VEC; ++i) tp[i] = r[i];
  *reinterpret_cast<V *>(p) = t;
}

// p[0] + p[f] + ... + p[(nseg - 1) f] in that order.  The longest rows of a power-law graph have
// hundreds of segments and one lane adds them all: the loads go out eight at a time.
__device__ __forceinline__ float sum_segments(const float *__restrict__ p, int32_t nseg, int32_t f) {
  float s = 0.f;
  int32_t i = 0;
  for (; i + 8 <= nseg; i += 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = p[(int64_t)(i + u) * f];
#pragma unroll
    for (int u = 0; u < 8; ++u) s += v[u];
  }
  for (; i < nseg; ++i) s += p[(int64_t)i * f];
  return s;
}

// C[row, :] = beta*C[row, :] + sum over the row's partial rows, in segment order.
__global__ __launch_bounds__(kSpmmThreads) void spmm_reduce_kernel(const int32_t *__restrict__ multi_rows,
                                                                   int64_t nmulti_host,
                                                                   const uint32_t *__restrict__ d_nmulti,
                                                                   const int32_t *__restrict__ rowptr,
                                                                   const int32_t *__restrict__ pbase, int32_t seg,
                                                                   const float *__restrict__ P, float *__restrict__ C,
                                                                   int64_t ldc, int32_t f, float beta,
                                                                   int64_t p_cap,
                                                                   const int32_t *__restrict__ fold_tbase,
                                                                   const float *__restrict__ fold_P,
                                                                   int32_t fold_classes, int32_t fold_rows,
                                                                   const float *__restrict__ fold_D,
                                                                   const int32_t *__restrict__ fold_dslot) {
  const int64_t idx = (int64_t)blockIdx.x * kSpmmThreads + threadIdx.x;
  const int64_t mr = idx / f;
  const int32_t col = (int32_t)(idx % f);
  int64_t nmulti = nmulti_host;  // capacity of multi_rows when the exact count is on the device
  if (d_nmulti && (int64_t)*d_nmulti < nmulti) nmulti = (int64_t)*d_nmulti;
  if (mr >= nmulti) return;
  const int32_t row = multi_rows[mr];
  const int32_t deg = rowptr[row + 1] - rowptr[row];
  const int32_t nseg = (deg + seg - 1) / seg;
  if (p_cap > 0 && (int64_t)pbase[row] + nseg > p_cap) return;  // only a malformed (unsorted) input gets here
  const float *p = P + (int64_t)pbase[row] * f + col;
  float s = sum_segments(p, nseg, f);
  if (fold_tbase) {  // same fold as in the main kernel, for rows that were split
    for (int32_t cls = 0; cls < fold_classes; ++cls) {
      const int32_t *tb = fold_tbase + (int64_t)cls * fold_rows + row;
      for (int32_t t = tb[0]; t < tb[1]; ++t) s += fold_P[(int64_t)t * f + col];
    }
  }
  if (fold_dslot) {
    const int32_t ds = fold_dslot[row];
    if (ds >= 0) s += fold_D[(int64_t)ds * f + col];
  }
  float *c = C + (int64_t)row * ldc + col;
  *c = beta != 0.f ? fmaf(beta, *c, s) : s;
}

struct StreamArgs {
  const int32_t *task_start, *task_dst, *wstart;
  const int32_t *colind;
  const float *val;
  int64_t win_first[9];
  int32_t groups;  // 1: windows run anywhere; 2/4/8: windows of class g run on XCDs x % groups == g
  int32_t clamp_m;   // > 0: column indices are clamped into [0, clamp_m) (entry point that does not validate)
  int64_t p_cap;     // > 0: partial rows with a slot >= p_cap are dropped (same entry point: keeps a
                     // malformed, unsorted input from writing outside the partial buffer)
  const uint32_t *d_nwin;  // groups == 1 only: when set, the number of windows is read from the device
                           // (tables built without a host round trip; the grid is an upper bound)
  const float *B;
  int64_t ldb;
  float *C;
  int64_t ldc;
  float *P;
  int32_t f;
  float beta;
  // Fold (wide teams, groups == 1): a row that goes straight to C also receives the partial rows
  // fold_P[t] for t in [fold_tbase[c * fold_rows + row], fold_tbase[c * fold_rows + row + 1]) of
  // every class c < fold_classes, added in (class, t) order after the row's own entries.
  // fold_any (nullable): one byte per row, 0 for rows that have no partial rows at all, so that
  // the many short rows of a low-degree matrix do not pay the per-class look-ups.
  const int32_t *fold_tbase;
  const float *fold_P;
  const uint8_t *fold_any;
  int32_t fold_classes, fold_rows;
  // Direct fold (wide teams, groups == 1): row r also receives the one partial row
  // fold_D[fold_dslot[r] * f ...] when fold_dslot[r] >= 0 (the panel plan's share of the row), added last.
  const float *fold_D;
  const int32_t *fold_dslot;
  // Epilogue (wide teams, groups == 1): a finished row r = beta*C[row] + (A B)[row] is not stored
  // but multiplied by epi_W (f x epi_fo): epi_Z[row, :] = act(r * epi_W), the layer's (A H) W
  // without the n x f intermediate.  epi_fop = epi_fo rounded up to 16, 32 or 64.
  const float *epi_W;
  int64_t epi_ldw;
  float *epi_Z;
  int64_t epi_ldz;
  int32_t epi_fo, epi_fop, epi_relu;
};

// LDS of an epilogue launch: W transposed as [fop][fpad] floats, then one row buffer of fpad floats
// per wave.  fpad = f rounded up to 16, plus 4 (keeps 16-byte alignment, spreads the rows of W^T
// over the banks); everything past f is zero.
__device__ __forceinline__ int32_t epi_fpad(int32_t f) { return (f + 15) / 16 * 16 + 4; }

__device__ __forceinline__ void epi_stage_w(float *lds, const float *__restrict__ W, int64_t ldw, int32_t f, int32_t fo,
                                            int32_t fop, int threads) {
  const int32_t fpad = epi_fpad(f);
  for (int32_t idx = threadIdx.x; idx < fpad * fop; idx += threads) {
    const int32_t k = idx / fop, j = idx % fop;  // j fastest: coalesced reads of W
    lds[j * fpad + k] = (k < f && j < fo) ? W[(int64_t)k * ldw + j] : 0.f;
  }
  float *rows = lds + (size_t)fop * fpad;  // tails of the row buffers: read by the last steps, never written again
  for (int32_t idx = threadIdx.x; idx < kWavesPerBlock * (fpad - f); idx += threads)
    rows[(idx / (fpad - f)) * fpad + f + idx % (fpad - f)] = 0.f;
}

// z[j] = sum_k row[k] * W[k][j] by one wavefront: lane = (part, j); a part owns a contiguous range
// of k and walks it four at a time (one 16-byte LDS read of the row, one of W^T); the parts are
// then added by a fixed xor butterfly; lanes of part 0 store.
__device__ __forceinline__ void epi_row(const float *row, const float *Wt, int32_t f, int32_t fop, int32_t fo, int lane,
                                        float *zrow, int relu) {
  const int32_t fpad = epi_fpad(f);
  const int j = lane & (fop - 1);
  const int part = lane / fop, parts = kWave / fop;
  const int32_t kper = ((f + parts - 1) / parts + 3) / 4 * 4;
  const float *r = row + part * kper;
  const float *w = Wt + (size_t)j * fpad + part * kper;
  float s0 = 0.f, s1 = 0.f;
  for (int32_t k = 0; k < kper; k += 4) {
    const float4 x = *reinterpret_cast<const float4 *>(r + k);
    const float4 y = *reinterpret_cast<const float4 *>(w + k);
    s0 = fmaf(x.x, y.x, s0);
    s1 = fmaf(x.y, y.y, s1);
    s0 = fmaf(x.z, y.z, s0);
    s1 = fmaf(x.w, y.w, s1);
  }
  float s = s0 + s1;
  for (int off = fop; off < kWave; off <<= 1) s += __shfl_xor(s, off, kWave);
  if (lane < fop && j < fo) zrow[j] = (relu && s < 0.f) ? 0.f : s;
}

// The same for a launch with an epilogue: one wavefront per split row rebuilds the row in LDS
// (partials in segment order, then the folded partial rows) and sends it through W.
struct ReduceEpiArgs {
  const int32_t *multi_rows;
  int64_t nmulti;
  const int32_t *rowptr, *pbase;
  int32_t seg;
  const float *P;
  const float *C;  // read only (beta != 0)
  int64_t ldc;
  int32_t f;
  float beta;
  const int32_t *fold_tbase;
  const float *fold_P;
  int32_t fold_classes, fold_rows;
  const float *epi_W;
  int64_t epi_ldw;
  float *epi_Z;
  int64_t epi_ldz;
  int32_t epi_fo, epi_fop, epi_relu;
};

__global__ __launch_bounds__(kSpmmThreads) void spmm_reduce_epi_kernel(const ReduceEpiArgs a) {
  extern __shared__ float epi_lds[];
  epi_stage_w(epi_lds, a.epi_W, a.epi_ldw, a.f, a.epi_fo, a.epi_fop, kSpmmThreads);
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int64_t mr = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  if (mr >= a.nmulti) return;
  const int32_t row = a.multi_rows[mr];
  const int32_t deg = a.rowptr[row + 1] - a.rowptr[row];
  const int32_t nseg = (deg + a.seg - 1) / a.seg;
  float *rowbuf = epi_lds + ((size_t)a.epi_fop + wave) * epi_fpad(a.f);
  for (int32_t col = lane; col < a.f; col += kWave) {
    const float *p = a.P + (int64_t)a.pbase[row] * a.f + col;
    float s = sum_segments(p, nseg, a.f);
    if (a.fold_tbase) {
      for (int32_t cls = 0; cls < a.fold_classes; ++cls) {
        const int32_t *tb = a.fold_tbase + (int64_t)cls * a.fold_rows + row;
        for (int32_t t = tb[0]; t < tb[1]; ++t) s += a.fold_P[(int64_t)t * a.f + col];
      }
    }
    rowbuf[col] = a.beta != 0.f ? fmaf(a.beta, a.C[(int64_t)row * a.ldc + col], s) : s;
  }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
  epi_row(rowbuf, epi_lds, a.f, a.epi_fop, a.epi_fo, lane, a.epi_Z + (int64_t)row * a.epi_ldz, a.epi_relu);
}

// Full-wave teams (one stored entry per wave step, f covered by CHUNKS x 64 lanes x VEC floats).
template <int VEC, int CHUNKS>
__global__ __launch_bounds__(kSpmmThreads) void spmm_stream_wide_kernel(const StreamArgs a) {
  const int lane = threadIdx.x & (kWave - 1);
  const int x = blockIdx.x & 7;
  const int per = 8 / a.groups;
  const int grp = x % a.groups;
  const int64_t lblock = (int64_t)(blockIdx.x >> 3) * per + x / a.groups;
  const int64_t wl = lblock * kWavesPerBlock + threadIdx.x / kWave;
  const int64_t nwin_here = a.d_nwin ? (int64_t)*a.d_nwin : a.win_first[grp + 1] - a.win_first[grp];
  extern __shared__ float epi_lds[];
  if (a.epi_W) {  // every wave of the workgroup stages W before any of them may leave
    epi_stage_w(epi_lds, a.epi_W, a.epi_ldw, a.f, a.epi_fo, a.epi_fop, kSpmmThreads);
    __syncthreads();
  }
  if (wl >= nwin_here) return;
  float *epi_rowbuf = epi_lds + ((size_t)a.epi_fop + threadIdx.x / kWave) * epi_fpad(a.f);
  const int32_t w = __builtin_amdgcn_readfirstlane((int32_t)(a.win_first[grp] + wl));
  const int32_t t0 = a.wstart[w], t1 = a.wstart[w + 1];
  const int ntask = t1 - t0;  // 1..64
  int32_t m_end = 0, m_dst = 0;
  if (lane < ntask) {
    m_end = a.task_start[t0 + lane + 1];
    m_dst = a.task_dst[t0 + lane];
  }
  const int32_t e_begin = a.task_start[t0];
  const int32_t e_end = __builtin_amdgcn_readlane(m_end, ntask - 1);

  const int nslots = a.f / VEC;
  bool active[CHUNKS];
  int64_t boff[CHUNKS];
#pragma unroll
  for (int ch = 0; ch < CHUNKS; ++ch) {
    active[ch] = (ch * kWave + lane) < nslots;
    boff[ch] = (int64_t)(ch * kWave + (active[ch] ? lane : 0)) * VEC;
  }
  float acc[CHUNKS][VEC];
#pragma unroll
  for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[ch][v] = 0.f;

  constexpr int U = 4;
  int tk = 0;
  int32_t tbeg = e_begin;
  int32_t tend = __builtin_amdgcn_readlane(m_end, 0);

  int32_t c_next = 0;
  float v_next = 0.f;
  if (e_begin + lane < e_end) {
    c_next = a.colind[e_begin + lane];
    v_next = a.val[e_begin + lane];
  }
  for (int32_t base = e_begin;; base += kWave) {
    int32_t c = c_next;
    const float v = v_next;
    if (a.clamp_m > 0) c = c < 0 ? 0 : (c >= a.clamp_m ? a.clamp_m - 1 : c);
    const int32_t nb = base + kWave + lane;
    c_next = 0;
    v_next = 0.f;
    if (nb < e_end) {
      c_next = a.colind[nb];
      v_next = a.val[nb];
    }
    int cnt = e_end - base;
    cnt = cnt > kWave ? kWave : (cnt < 0 ? 0 : cnt);
    int i = 0;
    for (;;) {
      while (tend == base + i) {  // the current task is complete (also true at once for an empty task)
        const int32_t dst = __builtin_amdgcn_readlane(m_dst, tk);
        if (dst >= 0) {
          bool folded = false;
          if (a.fold_tbase && (!a.fold_any || a.fold_any[dst])) {
            for (int32_t cls = 0; cls < a.fold_classes; ++cls) {
              const int32_t *tb = a.fold_tbase + (int64_t)cls * a.fold_rows + dst;
              const int32_t p0 = __builtin_amdgcn_readfirstlane(tb[0]);
              const int32_t p1 = __builtin_amdgcn_readfirstlane(tb[1]);
              for (int32_t t = p0; t < p1; ++t) {
                const float *prow = a.fold_P + (int64_t)t * a.f;
                float pv[CHUNKS][VEC];
#pragma unroll
                for (int ch = 0; ch < CHUNKS; ++ch) load_vec<VEC>(prow + boff[ch], pv[ch]);
#pragma unroll
                for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
                  for (int q = 0; q < VEC; ++q) acc[ch][q] += pv[ch][q];
                folded = true;
              }
            }
          }
          if (a.fold_dslot) {
            const int32_t ds = __builtin_amdgcn_readfirstlane(a.fold_dslot[dst]);
            if (ds >= 0) {
              const float *prow = a.fold_D + (int64_t)ds * a.f;
              float pv[CHUNKS][VEC];
#pragma unroll
              for (int ch = 0; ch < CHUNKS; ++ch) load_vec<VEC>(prow + boff[ch], pv[ch]);
#pragma unroll
              for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
                for (int q = 0; q < VEC; ++q) acc[ch][q] += pv[ch][q];
              folded = true;
            }
          }
          if (a.epi_W) {
            // the finished row goes to LDS and from there through W; C is only read (beta != 0)
            const float *crow = a.C + (int64_t)dst * a.ldc;
#pragma unroll
            for (int ch = 0; ch < CHUNKS; ++ch) {
              if (active[ch]) {
                float out[VEC];
                if (a.beta != 0.f) {
                  float old[VEC];
                  load_vec<VEC>(crow + boff[ch], old);
#pragma unroll
                  for (int q = 0; q < VEC; ++q) out[q] = fmaf(a.beta, old[q], acc[ch][q]);
                } else {
#pragma unroll
                  for (int q = 0; q < VEC; ++q) out[q] = acc[ch][q];
                }
#pragma unroll
                for (int q = 0; q < VEC; ++q) epi_rowbuf[boff[ch] + q] = out[q];
              }
            }
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
            __builtin_amdgcn_wave_barrier();
            epi_row(epi_rowbuf, epi_lds, a.f, a.epi_fop, a.epi_fo, lane, a.epi_Z + (int64_t)dst * a.epi_ldz, a.epi_relu);
            __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
            __builtin_amdgcn_wave_barrier();
          } else if (folded || !(tend == tbeg && a.beta == 1.0f)) {  // an empty row leaves C alone when beta == 1
            float *crow = a.C + (int64_t)dst * a.ldc;
#pragma unroll
            for (int ch = 0; ch < CHUNKS; ++ch) {
              if (active[ch]) {
                float out[VEC];
                if (a.beta != 0.f) {
                  float old[VEC];
                  load_vec<VEC>(crow + boff[ch], old);
#pragma unroll
                  for (int q = 0; q < VEC; ++q) out[q] = fmaf(a.beta, old[q], acc[ch][q]);
                } else {
#pragma unroll
                  for (int q = 0; q < VEC; ++q) out[q] = acc[ch][q];
                }
                store_vec<VEC>(crow + boff[ch], out);
              }
            }
          }
        } else if (a.p_cap <= 0 || (int64_t)(-(dst + 1)) < a.p_cap) {
          float *prow = a.P + (int64_t)(-(dst + 1)) * a.f;
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch)
            if (active[ch]) store_vec<VEC>(prow + boff[ch], acc[ch]);
        }
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
          for (int q = 0; q < VEC; ++q) acc[ch][q] = 0.f;
        if (++tk == ntask) return;
        tbeg = tend;
        tend = __builtin_amdgcn_readlane(m_end, tk);
      }
      if (i >= cnt) break;
      int run = tend - base;
      run = run < cnt ? run : cnt;
      if (run <= i) return;  // cannot happen with monotone task starts; guarantees termination
      for (; i + U <= run; i += U) {
        float b[U][CHUNKS][VEC];
        float vv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int32_t cc = __builtin_amdgcn_readlane(c, i + u);
          vv[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i + u));
          const float *brow = a.B + (int64_t)cc * a.ldb;
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch) load_vec<VEC>(brow + boff[ch], b[u][ch]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
            for (int q = 0; q < VEC; ++q) acc[ch][q] = fmaf(vv[u], b[u][ch][q], acc[ch][q]);
      }
      for (; i < run; ++i) {
        const int32_t cc = __builtin_amdgcn_readlane(c, i);
        const float vv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), i));
        const float *brow = a.B + (int64_t)cc * a.ldb;
        float b[CHUNKS][VEC];
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch) load_vec<VEC>(brow + boff[ch], b[ch]);
#pragma unroll
        for (int ch = 0; ch < CHUNKS; ++ch)
#pragma unroll
          for (int q = 0; q < VEC; ++q) acc[ch][q] = fmaf(vv, b[ch][q], acc[ch][q]);
      }
    }
  }
}

// Teams of LPR < 64 lanes (f <= 64 * VEC floats): the window's entries and task table are staged
// in LDS.  Long tasks (>= kLongFactor * G entries) are worked on by all G teams together (entries
// dealt round robin, partial sums combined by the xor butterfly); the short ones are dealt to the
// teams whole, G at a time, so rows of a few entries cost neither a butterfly nor an idle wave.
constexpr int kNarrowLds = 1024;  // entries a window may hold (window length S plus one task, both <= 512)
constexpr int kLongFactor = 4;

// acc += sum over u < U of val[i + u * stride] * B[col[i + u * stride], own columns]: U rows of B in flight
template <int VEC, int U>
__device__ __forceinline__ void narrow_gather(const int32_t *cw, const float *vw, int32_t i, int stride,
                                              const float *__restrict__ B, int64_t ldb, int64_t boff,
                                              float (&acc)[VEC]) {
  float b[U][VEC], vv[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int32_t cc = cw[i + u * stride];
    vv[u] = vw[i + u * stride];
    load_vec<VEC>(B + (int64_t)cc * ldb + boff, b[u]);
  }
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int q = 0; q < VEC; ++q) acc[q] = fmaf(vv[u], b[u][q], acc[q]);
}

// entries i, i + stride, ... below e, in that order: blocks of 8, then 4, 2, 1
template <int VEC>
__device__ __forceinline__ void narrow_sweep(const int32_t *cw, const float *vw, int32_t i, int32_t e, int stride,
                                             const float *__restrict__ B, int64_t ldb, int64_t boff,
                                             float (&acc)[VEC]) {
  for (; i + 7 * stride < e; i += 8 * stride) narrow_gather<VEC, 8>(cw, vw, i, stride, B, ldb, boff, acc);
  if (i + 3 * stride < e) {
    narrow_gather<VEC, 4>(cw, vw, i, stride, B, ldb, boff, acc);
    i += 4 * stride;
  }
  if (i + stride < e) {
    narrow_gather<VEC, 2>(cw, vw, i, stride, B, ldb, boff, acc);
    i += 2 * stride;
  }
  if (i < e) narrow_gather<VEC, 1>(cw, vw, i, stride, B, ldb, boff, acc);
}

template <int VEC, int LPR>
__global__ __launch_bounds__(kSpmmThreads) void spmm_stream_narrow_kernel(const StreamArgs a) {
  constexpr int G = kWave / LPR;
  __shared__ int32_t s_col[kWavesPerBlock][kNarrowLds];
  __shared__ float s_val[kWavesPerBlock][kNarrowLds];
  __shared__ int32_t s_beg[kWavesPerBlock][kWave], s_end[kWavesPerBlock][kWave], s_dst[kWavesPerBlock][kWave];
  __shared__ int32_t s_short[kWavesPerBlock][kWave];

  const int lane = threadIdx.x & (kWave - 1);
  const int wv = threadIdx.x / kWave;
  const int x = blockIdx.x & 7;
  const int per = 8 / a.groups;
  const int grp = x % a.groups;
  const int64_t lblock = (int64_t)(blockIdx.x >> 3) * per + x / a.groups;
  const int64_t wl = lblock * kWavesPerBlock + wv;
  const int64_t nwin_here = a.d_nwin ? (int64_t)*a.d_nwin : a.win_first[grp + 1] - a.win_first[grp];
  if (wl >= nwin_here) return;
  const int32_t w = __builtin_amdgcn_readfirstlane((int32_t)(a.win_first[grp] + wl));
  const int32_t t0 = a.wstart[w], t1 = a.wstart[w + 1];
  const int ntask = t1 - t0;  // 1..64
  const bool valid = lane < ntask;
  int32_t m_beg = 0, m_end = 0, m_dst = 0;
  if (valid) {
    m_beg = a.task_start[t0 + lane];
    m_end = a.task_start[t0 + lane + 1];
    m_dst = a.task_dst[t0 + lane];
  }
  const int32_t e_begin = __builtin_amdgcn_readlane(m_beg, 0);
  const int32_t e_end = __builtin_amdgcn_readlane(m_end, ntask - 1);
  const int32_t nent = e_end - e_begin;
  if (nent > kNarrowLds) return;  // excluded by the schedule (S + seg <= kNarrowLds); keeps LDS writes in bounds

  for (int32_t k = lane; k < nent; k += kWave) {
    int32_t c = a.colind[e_begin + k];
    if (a.clamp_m > 0) c = c < 0 ? 0 : (c >= a.clamp_m ? a.clamp_m - 1 : c);
    s_col[wv][k] = c;
    s_val[wv][k] = a.val[e_begin + k];
  }
  const int32_t r_beg = m_beg - e_begin, r_end = m_end - e_begin;  // relative to the window
  s_beg[wv][lane] = r_beg;
  s_end[wv][lane] = r_end;
  s_dst[wv][lane] = m_dst;
  const int32_t len = r_end - r_beg;
  const bool is_long = valid && len >= kLongFactor * G;
  // an empty row that goes straight to C needs no work when beta == 1
  const bool is_short = valid && !is_long && !(len == 0 && m_dst >= 0 && a.beta == 1.0f);

  const int g = lane / LPR, j = lane % LPR;
  const bool active = j * VEC < a.f;
  const int64_t boff = active ? (int64_t)j * VEC : 0;
  const int32_t *cw = s_col[wv];
  const float *vw = s_val[wv];

  const uint64_t short_mask = __ballot(is_short);
  if (is_short) s_short[wv][__popcll(short_mask & ((1ull << lane) - 1ull))] = lane;
  const int nshort = __popcll(short_mask);
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();  // the staged window and tables are visible to every lane of the wave

  // ---- long tasks: all teams together
  uint64_t long_mask = __ballot(is_long);
  while (long_mask) {
    const int k = __builtin_ctzll(long_mask);
    long_mask &= long_mask - 1;
    const int32_t s = __builtin_amdgcn_readlane(r_beg, k);
    const int32_t e = __builtin_amdgcn_readlane(r_end, k);
    const int32_t d = __builtin_amdgcn_readlane(m_dst, k);
    float acc[VEC];
#pragma unroll
    for (int q = 0; q < VEC; ++q) acc[q] = 0.f;
    narrow_sweep<VEC>(cw, vw, s + g, e, G, a.B, a.ldb, boff, acc);
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1)
#pragma unroll
      for (int q = 0; q < VEC; ++q) acc[q] += __shfl_xor(acc[q], off, kWave);
    if (g == 0 && active) {
      if (d >= 0) {
        float *crow = a.C + (int64_t)d * a.ldc + boff;
        float out[VEC];
        if (a.beta != 0.f) {
          float old[VEC];
          load_vec<VEC>(crow, old);
#pragma unroll
          for (int q = 0; q < VEC; ++q) out[q] = fmaf(a.beta, old[q], acc[q]);
        } else {
#pragma unroll
          for (int q = 0; q < VEC; ++q) out[q] = acc[q];
        }
        store_vec<VEC>(crow, out);
      } else if (a.p_cap <= 0 || (int64_t)(-(d + 1)) < a.p_cap) {
        store_vec<VEC>(a.P + (int64_t)(-(d + 1)) * a.f + boff, acc);
      }
    }
  }

  // ---- short tasks: one team each, G per round
  for (int q0 = 0; q0 < nshort; q0 += G) {
    const int my = q0 + g;
    const bool has = my < nshort;
    const int k = has ? s_short[wv][my] : 0;
    const int32_t s = s_beg[wv][k];
    const int32_t e = has ? s_end[wv][k] : s;
    const int32_t d = s_dst[wv][k];
    float acc[VEC];
#pragma unroll
    for (int q = 0; q < VEC; ++q) acc[q] = 0.f;
    narrow_sweep<VEC>(cw, vw, s, e, 1, a.B, a.ldb, boff, acc);
    if (has && active) {
      if (d >= 0) {
        float *crow = a.C + (int64_t)d * a.ldc + boff;
        float out[VEC];
        if (a.beta != 0.f) {
          float old[VEC];
          load_vec<VEC>(crow, old);
#pragma unroll
          for (int q = 0; q < VEC; ++q) out[q] = fmaf(a.beta, old[q], acc[q]);
        } else {
#pragma unroll
          for (int q = 0; q < VEC; ++q) out[q] = acc[q];
        }
        store_vec<VEC>(crow, out);
      } else if (a.p_cap <= 0 || (int64_t)(-(d + 1)) < a.p_cap) {
        store_vec<VEC>(a.P + (int64_t)(-(d + 1)) * a.f + boff, acc);
      }
    }
  }
}

// C[r, :] += sum of the partial rows of r's hot tasks, in (group, segment) order.  One wavefront
// per row: lane g fetches the task range of group g, then the lanes sweep the row's columns with
// the partial rows of all tasks in flight together.
template <int NC>  // classes the unrolled loops cover (nclass <= NC)
__global__ __launch_bounds__(kSpmmThreads) void hub_reduce_kernel(const int32_t *__restrict__ tbase, int32_t n,
                                                                  int32_t nclass, const float *__restrict__ P,
                                                                  float *__restrict__ C, int64_t ldc, int32_t f) {
  const int64_t r = ((int64_t)blockIdx.x * kSpmmThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (r >= n) return;
  int32_t t0 = 0, t1 = 0;
  if (lane < nclass) {
    const int64_t v = (int64_t)lane * n + r;
    t0 = tbase[v];
    t1 = tbase[v + 1];
  }
  int32_t first[NC], count[NC];
  int32_t total = 0;
#pragma unroll
  for (int g = 0; g < NC; ++g) {
    first[g] = __builtin_amdgcn_readlane(t0, g);
    count[g] = __builtin_amdgcn_readlane(t1, g) - first[g];
    total += count[g];
  }
  if (total == 0) return;
  float *crow = C + r * ldc;
  for (int32_t c0 = 0; c0 < f; c0 += kWave) {
    const int32_t col = c0 + lane;
    if (col < f) {
      // the first partial row of every class is loaded before anything is added (classes without one
      // read slot 0, which exists because total > 0, and are skipped in the sum); classes with more
      // than one partial row (rows split into segments) add the rest in order
      float v[NC];
#pragma unroll
      for (int g = 0; g < NC; ++g) v[g] = P[(int64_t)(count[g] > 0 ? first[g] : 0) * f + col];
      float s = 0.f;
#pragma unroll
      for (int g = 0; g < NC; ++g) {
        if (count[g] > 0) s += v[g];
        if (count[g] > 1) {
          const float *p = P + (int64_t)first[g] * f + col;
          for (int32_t t = 1; t < count[g]; ++t) s += p[(int64_t)t * f];
        }
      }
      crow[col] += s;
    }
  }
}

}  // namespace cg
