// Activations and loss of GCNFunc / train as streaming kernels.
//   ReLU and its mask gradient            (F.relu, gcn_distr.py:288 and :317-322)
//   row-wise log_softmax and its gradient (F.log_softmax, gcn_distr.py:286 and :315-322)
//   masked mean NLL and its gradient      (F.nll_loss(outputs[mask], y[mask]), gcn_distr.py:356)
//   fused gradient of NLL(log_softmax(z)) with respect to z
// Rows of 8..256 classes are handled by 16-lane teams (4 rows per wavefront); the loss reduction
// is two fixed-order passes (per workgroup, then one workgroup over the partial sums).
#include "common.h"

namespace cg {

constexpr int kEwThreads = 256;
constexpr int kTeam = 16;                       // lanes per row
constexpr int kRowsPerBlock = kEwThreads / kTeam;

__global__ __launch_bounds__(kEwThreads) void relu_fwd_kernel(const float *__restrict__ z, float *__restrict__ h,
                                                              int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (i < count) {
    const float v = z[i];
    h[i] = v > 0.f ? v : 0.f;
  }
}

__global__ __launch_bounds__(kEwThreads) void relu_bwd_kernel(const float *__restrict__ g, const float *__restrict__ h,
                                                              float *__restrict__ dz, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (i < count) dz[i] = h[i] > 0.f ? g[i] : 0.f;
}

__device__ __forceinline__ float team_max(float v) {
#pragma unroll
  for (int off = kTeam / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}
__device__ __forceinline__ float team_sum(float v) {
#pragma unroll
  for (int off = kTeam / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__global__ __launch_bounds__(kEwThreads) void log_softmax_fwd_kernel(const float *__restrict__ z, int64_t ldz,
                                                                     float *__restrict__ out, int64_t ldo, int64_t n,
                                                                     int32_t c) {
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kTeam;
  const int j = threadIdx.x % kTeam;
  const bool live = row < n;
  const float *zr = z + (live ? row : 0) * ldz;
  float mx = -INFINITY;
  if (live)
    for (int32_t k = j; k < c; k += kTeam) mx = fmaxf(mx, zr[k]);
  mx = team_max(mx);
  float s = 0.f;
  if (live)
    for (int32_t k = j; k < c; k += kTeam) s += expf(zr[k] - mx);
  s = team_sum(s);
  const float lse = mx + logf(s);
  if (live) {
    float *orow = out + row * ldo;
    for (int32_t k = j; k < c; k += kTeam) orow[k] = zr[k] - lse;
  }
}

__global__ __launch_bounds__(kEwThreads) void log_softmax_bwd_kernel(const float *__restrict__ g, int64_t ldg,
                                                                     const float *__restrict__ out, int64_t ldo,
                                                                     float *__restrict__ dz, int64_t lddz, int64_t n,
                                                                     int32_t c) {
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kTeam;
  const int j = threadIdx.x % kTeam;
  const bool live = row < n;
  const float *gr = g + (live ? row : 0) * ldg;
  const float *orow = out + (live ? row : 0) * ldo;
  float s = 0.f;
  if (live)
    for (int32_t k = j; k < c; k += kTeam) s += gr[k];
  s = team_sum(s);
  if (live) {
    float *d = dz + row * lddz;
    for (int32_t k = j; k < c; k += kTeam) d[k] = gr[k] - expf(orow[k]) * s;
  }
}

// pass 1: per-workgroup sums of -logp[i, y_i] and of the mask, in a fixed tree order
__global__ __launch_bounds__(kEwThreads) void nll_partial_kernel(const float *__restrict__ logp, int64_t ld,
                                                                 const int64_t *__restrict__ y,
                                                                 const uint8_t *__restrict__ mask, int64_t n,
                                                                 int32_t c, float *__restrict__ psum,
                                                                 int64_t *__restrict__ pcnt) {
  __shared__ float ssum[kEwThreads / kWave];
  __shared__ int scnt[kEwThreads / kWave];
  const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  float v = 0.f;
  int cnt = 0;
  if (i < n && (!mask || mask[i])) {
    cnt = 1;
    const int64_t label = y[i];
    if (label >= 0 && label < c) v = -logp[i * ld + label];
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    v += __shfl_xor(v, off, kWave);
    cnt += __shfl_xor(cnt, off, kWave);
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) {
    ssum[wave] = v;
    scnt[wave] = cnt;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    int64_t k = 0;
    for (int w = 0; w < kEwThreads / kWave; ++w) {
      s += ssum[w];
      k += scnt[w];
    }
    psum[blockIdx.x] = s;
    pcnt[blockIdx.x] = k;
  }
}

// pass 2: one workgroup; thread t adds partials t, t+256, ... in order, then a fixed tree
__global__ __launch_bounds__(kEwThreads) void nll_final_kernel(const float *__restrict__ psum,
                                                               const int64_t *__restrict__ pcnt, int64_t nparts,
                                                               float *__restrict__ loss, int64_t *__restrict__ count) {
  __shared__ float ssum[kEwThreads];
  __shared__ int64_t scnt[kEwThreads];
  float s = 0.f;
  int64_t k = 0;
  for (int64_t i = threadIdx.x; i < nparts; i += kEwThreads) {
    s += psum[i];
    k += pcnt[i];
  }
  ssum[threadIdx.x] = s;
  scnt[threadIdx.x] = k;
  __syncthreads();
  for (int off = kEwThreads / 2; off > 0; off >>= 1) {
    if ((int)threadIdx.x < off) {
      ssum[threadIdx.x] += ssum[threadIdx.x + off];
      scnt[threadIdx.x] += scnt[threadIdx.x + off];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const int64_t total = scnt[0];
    *count = total;
    *loss = total > 0 ? ssum[0] / (float)total : 0.f;
  }
}

template <bool FUSED>
__global__ __launch_bounds__(kEwThreads) void nll_bwd_kernel(const float *__restrict__ logp, int64_t ld,
                                                             const int64_t *__restrict__ y,
                                                             const uint8_t *__restrict__ mask,
                                                             const int64_t *__restrict__ count,
                                                             const float *__restrict__ gscale, float *__restrict__ dst,
                                                             int64_t ldd, int64_t n, int32_t c) {
  const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kTeam;
  const int j = threadIdx.x % kTeam;
  if (row >= n) return;
  const int64_t total = *count;
  const bool on = total > 0 && (!mask || mask[row]);
  const float w = on ? (gscale ? *gscale : 1.f) / (float)total : 0.f;
  const int64_t label = y[row];
  float *d = dst + row * ldd;
  for (int32_t k = j; k < c; k += kTeam) {
    const float onehot = (k == label) ? 1.f : 0.f;
    float v;
    if (FUSED) v = on ? w * (expf(logp[row * ld + k]) - onehot) : 0.f;
    else v = -w * onehot;
    d[k] = v;
  }
}

static int check_rows(const char *who, int64_t n, int32_t c) {
  if (n < 0 || c <= 0) CG_FAIL(CG_ERR_SIZE, "%s: bad sizes n=%lld c=%d", who, (long long)n, c);
  if (ceil_div64(n, kRowsPerBlock) > 0x7fffffffLL) CG_FAIL(CG_ERR_SIZE, "%s: too many rows", who);
  return CG_OK;
}

}  // namespace cg

extern "C" {

int cg_relu_fwd(const float *d_z, float *d_h, int64_t count, cg_stream_t stream) {
  using namespace cg;
  if (count < 0) CG_FAIL(CG_ERR_SIZE, "cg_relu_fwd: negative count");
  if (count == 0) return CG_OK;
  if (!d_z || !d_h) CG_FAIL(CG_ERR_NULL, "cg_relu_fwd: null pointer");
  relu_fwd_kernel<<<(unsigned)ceil_div64(count, kEwThreads), kEwThreads, 0, (hipStream_t)stream>>>(d_z, d_h, count);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_relu_bwd(const float *d_g, const float *d_h, float *d_dz, int64_t count, cg_stream_t stream) {
  using namespace cg;
  if (count < 0) CG_FAIL(CG_ERR_SIZE, "cg_relu_bwd: negative count");
  if (count == 0) return CG_OK;
  if (!d_g || !d_h || !d_dz) CG_FAIL(CG_ERR_NULL, "cg_relu_bwd: null pointer");
  relu_bwd_kernel<<<(unsigned)ceil_div64(count, kEwThreads), kEwThreads, 0, (hipStream_t)stream>>>(d_g, d_h, d_dz,
                                                                                                  count);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_log_softmax_fwd(const float *d_z, int64_t ldz, float *d_out, int64_t ldo, int64_t n, int32_t c,
                       cg_stream_t stream) {
  using namespace cg;
  CG_TRY(check_rows("cg_log_softmax_fwd", n, c));
  if (n == 0) return CG_OK;
  if (!d_z || !d_out) CG_FAIL(CG_ERR_NULL, "cg_log_softmax_fwd: null pointer");
  if (ldz < c || ldo < c) CG_FAIL(CG_ERR_SIZE, "cg_log_softmax_fwd: leading dimension smaller than c");
  log_softmax_fwd_kernel<<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, (hipStream_t)stream>>>(
      d_z, ldz, d_out, ldo, n, c);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_log_softmax_bwd(const float *d_g, int64_t ldg, const float *d_out, int64_t ldo, float *d_dz, int64_t lddz,
                       int64_t n, int32_t c, cg_stream_t stream) {
  using namespace cg;
  CG_TRY(check_rows("cg_log_softmax_bwd", n, c));
  if (n == 0) return CG_OK;
  if (!d_g || !d_out || !d_dz) CG_FAIL(CG_ERR_NULL, "cg_log_softmax_bwd: null pointer");
  if (ldg < c || ldo < c || lddz < c) CG_FAIL(CG_ERR_SIZE, "cg_log_softmax_bwd: leading dimension smaller than c");
  log_softmax_bwd_kernel<<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, (hipStream_t)stream>>>(
      d_g, ldg, d_out, ldo, d_dz, lddz, n, c);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_nll_loss_fwd(const float *d_logp, int64_t ld, const int64_t *d_y, const uint8_t *d_mask, int64_t n, int32_t c,
                    float *d_loss, int64_t *d_count, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  CG_TRY(check_rows("cg_nll_loss_fwd", n, c));
  if (!d_loss || !d_count) CG_FAIL(CG_ERR_NULL, "cg_nll_loss_fwd: null output");
  if (n > 0 && (!d_logp || !d_y)) CG_FAIL(CG_ERR_NULL, "cg_nll_loss_fwd: null input");
  if (ld < c) CG_FAIL(CG_ERR_SIZE, "cg_nll_loss_fwd: leading dimension smaller than c");
  const int64_t parts = ceil_div64(n, kEwThreads);
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, (size_t)(parts + 1) * (sizeof(float) + sizeof(int64_t)) + 16, &p));
  int64_t *pcnt = (int64_t *)p;                 // 8-byte aligned part first
  float *psum = (float *)(pcnt + parts + 1);
  if (parts > 0) {
    nll_partial_kernel<<<(unsigned)parts, kEwThreads, 0, stream>>>(d_logp, ld, d_y, d_mask, n, c, psum, pcnt);
    CG_LAUNCH_CHECK();
  }
  nll_final_kernel<<<1, kEwThreads, 0, stream>>>(psum, pcnt, parts, d_loss, d_count);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_nll_loss_bwd(const int64_t *d_y, const uint8_t *d_mask, const int64_t *d_count, const float *d_gscale,
                    float *d_dlogp, int64_t ld, int64_t n, int32_t c, cg_stream_t stream) {
  using namespace cg;
  CG_TRY(check_rows("cg_nll_loss_bwd", n, c));
  if (n == 0) return CG_OK;
  if (!d_y || !d_count || !d_dlogp) CG_FAIL(CG_ERR_NULL, "cg_nll_loss_bwd: null pointer");
  if (ld < c) CG_FAIL(CG_ERR_SIZE, "cg_nll_loss_bwd: leading dimension smaller than c");
  nll_bwd_kernel<false><<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, (hipStream_t)stream>>>(
      nullptr, 0, d_y, d_mask, d_count, d_gscale, d_dlogp, ld, n, c);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_log_softmax_nll_bwd(const float *d_logp, int64_t ld, const int64_t *d_y, const uint8_t *d_mask,
                           const int64_t *d_count, const float *d_gscale, float *d_dz, int64_t lddz, int64_t n,
                           int32_t c, cg_stream_t stream) {
  using namespace cg;
  CG_TRY(check_rows("cg_log_softmax_nll_bwd", n, c));
  if (n == 0) return CG_OK;
  if (!d_logp || !d_y || !d_count || !d_dz) CG_FAIL(CG_ERR_NULL, "cg_log_softmax_nll_bwd: null pointer");
  if (ld < c || lddz < c) CG_FAIL(CG_ERR_SIZE, "cg_log_softmax_nll_bwd: leading dimension smaller than c");
  nll_bwd_kernel<true><<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, (hipStream_t)stream>>>(
      d_logp, ld, d_y, d_mask, d_count, d_gscale, d_dz, lddz, n, c);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

}  // extern "C"
