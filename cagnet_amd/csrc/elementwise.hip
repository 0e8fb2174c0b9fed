// Activations and loss of GCNFunc / train as streaming kernels.
//   ReLU and its mask gradient            (F.relu, gcn_distr.py:288 and :317-322)
//   row-wise log_softmax and its gradient (F.log_softmax, gcn_distr.py:286 and :315-322)
//   masked mean NLL and its gradient      (F.nll_loss(outputs[mask], y[mask]), gcn_distr.py:356)
//   fused gradient of NLL(log_softmax(z)) with respect to z
// Rows whose length is a multiple of 4 (up to 64) and whose storage is 16-byte aligned are handled
// by teams of 1..16 lanes holding one 16-byte piece each, several rows per wavefront and
// instruction, one read and one write of every operand; other rows by 16-lane teams with one
// element per lane and step.  ReLU moves 16 bytes per lane when the operands are aligned.  The loss
// reduction is two fixed-order passes (per workgroup, then one workgroup over the partial sums).
#include "common.h"
#include <mutex>

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

// 16 bytes per lane, grid-stride; the count % 4 tail elements are done by the first threads
__global__ __launch_bounds__(kEwThreads) void relu_fwd_vec_kernel(const float *__restrict__ z, float *__restrict__ h,
                                                                  int64_t count) {
  const int64_t n4 = count / 4, tid = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  for (int64_t i = tid; i < n4; i += (int64_t)gridDim.x * kEwThreads) {
    float4 v = reinterpret_cast<const float4 *>(z)[i];
    v.x = v.x > 0.f ? v.x : 0.f;
    v.y = v.y > 0.f ? v.y : 0.f;
    v.z = v.z > 0.f ? v.z : 0.f;
    v.w = v.w > 0.f ? v.w : 0.f;
    reinterpret_cast<float4 *>(h)[i] = v;
  }
  if (tid < count - n4 * 4) {
    const float v = z[n4 * 4 + tid];
    h[n4 * 4 + tid] = v > 0.f ? v : 0.f;
  }
}

__global__ __launch_bounds__(kEwThreads) void relu_bwd_vec_kernel(const float *__restrict__ g,
                                                                  const float *__restrict__ h, float *__restrict__ dz,
                                                                  int64_t count) {
  const int64_t n4 = count / 4, tid = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  for (int64_t i = tid; i < n4; i += (int64_t)gridDim.x * kEwThreads) {
    const float4 a = reinterpret_cast<const float4 *>(g)[i];
    const float4 b = reinterpret_cast<const float4 *>(h)[i];
    float4 v;
    v.x = b.x > 0.f ? a.x : 0.f;
    v.y = b.y > 0.f ? a.y : 0.f;
    v.z = b.z > 0.f ? a.z : 0.f;
    v.w = b.w > 0.f ? a.w : 0.f;
    reinterpret_cast<float4 *>(dz)[i] = v;
  }
  if (tid < count - n4 * 4) dz[n4 * 4 + tid] = h[n4 * 4 + tid] > 0.f ? g[n4 * 4 + tid] : 0.f;
}

static bool aligned16(const void *a, const void *b, const void *c = nullptr) {
  return (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15) == 0;
}
static unsigned vec_grid(int64_t count4) {  // enough 16-byte lanes to cover the chip several times, each looping
  int64_t blocks = ceil_div64(count4 > 0 ? count4 : 1, kEwThreads);
  if (blocks > 256 * 32) blocks = 256 * 32;
  return (unsigned)blocks;
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

// LOSS: the lane that holds the label's column also writes the row's contribution to the masked NLL,
// rowloss[row] = -out[row, y[row]] (0 for rows outside the mask or with a label outside [0, c)),
// so that the loss needs no second pass over the n x c array.
template <bool LOSS>
__global__ __launch_bounds__(kEwThreads) void log_softmax_fwd_kernel(const float *__restrict__ z, int64_t ldz,
                                                                     float *__restrict__ out, int64_t ldo, int64_t n,
                                                                     int32_t c, const int64_t *__restrict__ y,
                                                                     const uint8_t *__restrict__ mask,
                                                                     float *__restrict__ rowloss) {
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
    if (LOSS) {
      const int64_t label = y[row];
      const bool counted = (!mask || mask[row]) && label >= 0 && label < c;
      const int writer = counted ? (int)(label % kTeam) : 0;
      if (j == writer) rowloss[row] = counted ? -(zr[label] - lse) : 0.f;
    }
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

// ---------------------------------------------------------------------------------------------
// Rows of c = 4, 8, ..., 64 floats in 16-byte aligned storage: T lanes per row (T = 1..16, a power
// of two >= c / 4), each holding one 16-byte piece; a wavefront covers 64 / T consecutive rows with
// one load instruction.  Loads are unconditional (clamped address) and dead lanes are neutralised
// in registers.
// ---------------------------------------------------------------------------------------------
template <int T>
__device__ __forceinline__ float vteam_max(float v) {
#pragma unroll
  for (int off = T / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}
template <int T>
__device__ __forceinline__ float vteam_sum(float v) {
#pragma unroll
  for (int off = T / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

struct RowWalk {  // the rows of a grid of wavefronts, 64 / T at a time
  int64_t first, step;
  int sub, j;
};
template <int T>
__device__ __forceinline__ RowWalk row_walk() {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t gw = ((int64_t)blockIdx.x * kEwThreads + threadIdx.x) / kWave;
  const int64_t nw = (int64_t)gridDim.x * (kEwThreads / kWave);
  return RowWalk{gw * (kWave / T), nw * (kWave / T), lane / T, lane % T};
}

template <int T, bool LOSS>
__global__ __launch_bounds__(kEwThreads) void log_softmax_fwd_vec_kernel(const float *__restrict__ z, int64_t ldz,
                                                                         float *__restrict__ out, int64_t ldo,
                                                                         int64_t n, int32_t c,
                                                                         const int64_t *__restrict__ y,
                                                                         const uint8_t *__restrict__ mask,
                                                                         float *__restrict__ rowloss) {
  const RowWalk w = row_walk<T>();
  const bool col_live = 4 * w.j < c;
  const int32_t col = col_live ? 4 * w.j : 0;
  for (int64_t r0 = w.first; r0 < n; r0 += w.step) {
    const int64_t row = r0 + w.sub;
    const bool live = row < n && col_live;
    const int64_t rc = row < n ? row : n - 1;
    const float4 v = *reinterpret_cast<const float4 *>(z + rc * ldz + col);
    int64_t label = 0;
    bool counted = false;
    if (LOSS) {  // every lane of the team reads the same two words (unconditional, clamped row)
      label = y[rc];
      counted = (!mask || mask[rc]) && label >= 0 && label < c;
    }
    float mx = live ? fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w)) : -INFINITY;
    mx = vteam_max<T>(mx);
    float s = live ? (expf(v.x - mx) + expf(v.y - mx)) + (expf(v.z - mx) + expf(v.w - mx)) : 0.f;
    s = vteam_sum<T>(s);
    const float lse = mx + logf(s);
    const float4 o = make_float4(v.x - lse, v.y - lse, v.z - lse, v.w - lse);
    if (live) *reinterpret_cast<float4 *>(out + row * ldo + col) = o;
    if (LOSS && row < n) {
      const int writer = counted ? (int)(label >> 2) : 0;  // the lane whose piece holds the label (its columns are live)
      if (w.j == writer) {
        const int q = (int)(label & 3);
        const float at = q == 0 ? o.x : (q == 1 ? o.y : (q == 2 ? o.z : o.w));
        rowloss[row] = counted ? -at : 0.f;
      }
    }
  }
}

template <int T>
__global__ __launch_bounds__(kEwThreads) void log_softmax_bwd_vec_kernel(const float *__restrict__ g, int64_t ldg,
                                                                         const float *__restrict__ out, int64_t ldo,
                                                                         float *__restrict__ dz, int64_t lddz,
                                                                         int64_t n, int32_t c) {
  const RowWalk w = row_walk<T>();
  const bool col_live = 4 * w.j < c;
  const int32_t col = col_live ? 4 * w.j : 0;
  for (int64_t r0 = w.first; r0 < n; r0 += w.step) {
    const int64_t row = r0 + w.sub;
    const bool live = row < n && col_live;
    const int64_t rc = row < n ? row : n - 1;
    const float4 a = *reinterpret_cast<const float4 *>(g + rc * ldg + col);
    const float4 o = *reinterpret_cast<const float4 *>(out + rc * ldo + col);
    float s = live ? (a.x + a.y) + (a.z + a.w) : 0.f;
    s = vteam_sum<T>(s);
    if (live)
      *reinterpret_cast<float4 *>(dz + row * lddz + col) =
          make_float4(a.x - expf(o.x) * s, a.y - expf(o.y) * s, a.z - expf(o.z) * s, a.w - expf(o.w) * s);
  }
}

template <int T, bool FUSED>
__global__ __launch_bounds__(kEwThreads) void nll_bwd_vec_kernel(const float *__restrict__ logp, int64_t ld,
                                                                 const int64_t *__restrict__ y,
                                                                 const uint8_t *__restrict__ mask,
                                                                 const int64_t *__restrict__ count,
                                                                 const float *__restrict__ gscale,
                                                                 float *__restrict__ dst, int64_t ldd, int64_t n,
                                                                 int32_t c) {
  const RowWalk w = row_walk<T>();
  const bool col_live = 4 * w.j < c;
  const int32_t col = col_live ? 4 * w.j : 0;
  const int64_t total = *count;
  const float unit = total > 0 ? (gscale ? *gscale : 1.f) / (float)total : 0.f;
  for (int64_t r0 = w.first; r0 < n; r0 += w.step) {
    const int64_t row = r0 + w.sub;
    const int64_t rc = row < n ? row : n - 1;
    const bool on = total > 0 && (!mask || mask[rc]) && y[rc] >= 0 && y[rc] < c;
    const float wgt = on ? unit : 0.f;
    const int32_t hit = (int32_t)(y[rc] - col);  // 0..3 when the label falls into this lane's piece
    float4 v;
    if (FUSED) {
      const float4 lp = *reinterpret_cast<const float4 *>(logp + rc * ld + col);
      v.x = on ? wgt * (expf(lp.x) - (hit == 0 ? 1.f : 0.f)) : 0.f;
      v.y = on ? wgt * (expf(lp.y) - (hit == 1 ? 1.f : 0.f)) : 0.f;
      v.z = on ? wgt * (expf(lp.z) - (hit == 2 ? 1.f : 0.f)) : 0.f;
      v.w = on ? wgt * (expf(lp.w) - (hit == 3 ? 1.f : 0.f)) : 0.f;
    } else {
      v.x = -wgt * (hit == 0 ? 1.f : 0.f);
      v.y = -wgt * (hit == 1 ? 1.f : 0.f);
      v.z = -wgt * (hit == 2 ? 1.f : 0.f);
      v.w = -wgt * (hit == 3 ? 1.f : 0.f);
    }
    if (row < n && col_live) *reinterpret_cast<float4 *>(dst + row * ldd + col) = v;
  }
}

// lanes per row of the 16-byte form, or 0 when the rows do not qualify
static int vec_team(int32_t c, int64_t ld0, int64_t ld1, int64_t ld2, const void *p0, const void *p1, const void *p2) {
  if (c % 4 != 0 || c > 64 || ld0 % 4 != 0 || ld1 % 4 != 0 || ld2 % 4 != 0 || !aligned16(p0, p1, p2)) return 0;
  int t = 1;
  while (4 * t < c) t *= 2;
  return t;
}
static unsigned row_grid(int64_t n, int team) {
  int64_t blocks = ceil_div64(n, (int64_t)(kWave / team) * (kEwThreads / kWave));
  if (blocks > 256 * 16) blocks = 256 * 16;
  return (unsigned)(blocks > 0 ? blocks : 1);
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
    const int64_t label = y[i];
    if (label >= 0 && label < c) {  // other labels are ignored, as F.nll_loss ignores ignore_index rows
      cnt = 1;
      v = -logp[i * ld + label];
    }
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
// The same partial sums from the per-row contributions a fused forward pass left behind: same rows
// per workgroup and the same order of additions as nll_partial_kernel, so the loss is the same float.
__global__ __launch_bounds__(kEwThreads) void nll_rows_partial_kernel(const float *__restrict__ rowloss,
                                                                      const int64_t *__restrict__ y,
                                                                      const uint8_t *__restrict__ mask, int64_t n,
                                                                      int32_t c, float *__restrict__ psum,
                                                                      int64_t *__restrict__ pcnt) {
  __shared__ float ssum[kEwThreads / kWave];
  __shared__ int scnt[kEwThreads / kWave];
  const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  float v = 0.f;
  int cnt = 0;
  if (i < n && (!mask || mask[i]) && y[i] >= 0 && y[i] < c) {
    cnt = 1;
    v = rowloss[i];
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
  const int64_t label = y[row];
  const bool on = total > 0 && (!mask || mask[row]) && label >= 0 && label < c;
  const float w = on ? (gscale ? *gscale : 1.f) / (float)total : 0.f;
  float *d = dst + row * ldd;
  for (int32_t k = j; k < c; k += kTeam) {
    const float onehot = (k == label) ? 1.f : 0.f;
    float v;
    if (FUSED) v = on ? w * (expf(logp[row * ld + k]) - onehot) : 0.f;
    else v = -w * onehot;
    d[k] = v;
  }
}

// ---- partial sums of cg_nll_loss_fwd_static: device memory that exists from load to exit --------------------
// Room for the per-workgroup partial sums of kStaticNllMaxRows rows: (parts + 1) int64 counts, then
// (parts + 1) float sums, laid out as in cg_nll_loss_fwd.  About 768 KiB per device.
constexpr int64_t kStaticNllMaxRows = (int64_t)1 << 24;
constexpr int64_t kStaticNllMaxParts = kStaticNllMaxRows / kEwThreads;
constexpr size_t kStaticNllBytes = (size_t)(kStaticNllMaxParts + 1) * (sizeof(int64_t) + sizeof(float)) + 16;
static __device__ __align__(256) unsigned char scratch[kStaticNllBytes];

// In host code `scratch` is only a name to look the array up by; the address the kernels may use is
// the one hipGetSymbolAddress returns, and every device holds its own copy at its own address.
constexpr int kStaticMaxDevices = 64;
static std::mutex g_static_mu;
static void *g_static_ptr[kStaticMaxDevices] = {nullptr};

static int static_scratch(void **out) {
  int dev = 0;
  CG_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kStaticMaxDevices) CG_FAIL(CG_ERR_UNSUPPORTED, "device ordinal %d beyond %d", dev, kStaticMaxDevices);
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_ptr[dev]) {
    void *p = nullptr;
    CG_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) CG_FAIL(CG_ERR_HIP, "hipGetSymbolAddress returned a null address for the static scratch array");
    g_static_ptr[dev] = p;
  }
  *out = g_static_ptr[dev];
  return CG_OK;
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
  ProfScope prof("relu_fwd", -1, (hipStream_t)stream);
  if (aligned16(d_z, d_h))
    relu_fwd_vec_kernel<<<vec_grid(count / 4), kEwThreads, 0, (hipStream_t)stream>>>(d_z, d_h, count);
  else
    relu_fwd_kernel<<<(unsigned)ceil_div64(count, kEwThreads), kEwThreads, 0, (hipStream_t)stream>>>(d_z, d_h, count);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_relu_bwd(const float *d_g, const float *d_h, float *d_dz, int64_t count, cg_stream_t stream) {
  using namespace cg;
  if (count < 0) CG_FAIL(CG_ERR_SIZE, "cg_relu_bwd: negative count");
  if (count == 0) return CG_OK;
  if (!d_g || !d_h || !d_dz) CG_FAIL(CG_ERR_NULL, "cg_relu_bwd: null pointer");
  ProfScope prof("relu_bwd", -1, (hipStream_t)stream);
  if (aligned16(d_g, d_h, d_dz))
    relu_bwd_vec_kernel<<<vec_grid(count / 4), kEwThreads, 0, (hipStream_t)stream>>>(d_g, d_h, d_dz, count);
  else
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
  hipStream_t s = (hipStream_t)stream;
  ProfScope prof("log_softmax_fwd", c, s);
  switch (vec_team(c, ldz, ldo, 4, d_z, d_out, nullptr)) {
#define CG_CASE(T)                                                                                        \
  case T:                                                                                                 \
    log_softmax_fwd_vec_kernel<T, false><<<row_grid(n, T), kEwThreads, 0, s>>>(d_z, ldz, d_out, ldo, n, c, nullptr, \
                                                                               nullptr, nullptr);        \
    break;
    CG_CASE(1) CG_CASE(2) CG_CASE(4) CG_CASE(8) CG_CASE(16)
#undef CG_CASE
    default:
      log_softmax_fwd_kernel<false><<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, s>>>(d_z, ldz, d_out, ldo, n,
                                                                                                  c, nullptr, nullptr, nullptr);
  }
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
  hipStream_t s = (hipStream_t)stream;
  ProfScope prof("log_softmax_bwd", c, s);
  switch (vec_team(c, ldg, ldo, lddz, d_g, d_out, d_dz)) {
#define CG_CASE(T)                                                                                              \
  case T:                                                                                                       \
    log_softmax_bwd_vec_kernel<T><<<row_grid(n, T), kEwThreads, 0, s>>>(d_g, ldg, d_out, ldo, d_dz, lddz, n, c); \
    break;
    CG_CASE(1) CG_CASE(2) CG_CASE(4) CG_CASE(8) CG_CASE(16)
#undef CG_CASE
    default:
      log_softmax_bwd_kernel<<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, s>>>(d_g, ldg, d_out, ldo, d_dz,
                                                                                           lddz, n, c);
  }
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
  ProfScope prof("nll_fwd", c, stream);
  if (parts > 0) {
    nll_partial_kernel<<<(unsigned)parts, kEwThreads, 0, stream>>>(d_logp, ld, d_y, d_mask, n, c, psum, pcnt);
    CG_LAUNCH_CHECK();
  }
  nll_final_kernel<<<1, kEwThreads, 0, stream>>>(psum, pcnt, parts, d_loss, d_count);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_nll_loss_fwd_static(const float *d_logp, int64_t ld, const int64_t *d_y, const uint8_t *d_mask, int64_t n,
                           int32_t c, float *d_loss, int64_t *d_count, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  CG_TRY(check_rows("cg_nll_loss_fwd_static", n, c));
  if (n > kStaticNllMaxRows)
    CG_FAIL(CG_ERR_SIZE, "cg_nll_loss_fwd_static: n=%lld exceeds the %lld rows the static scratch holds partial sums for",
            (long long)n, (long long)kStaticNllMaxRows);
  if (!d_loss || !d_count) CG_FAIL(CG_ERR_NULL, "cg_nll_loss_fwd_static: null output");
  if (n > 0 && (!d_logp || !d_y)) CG_FAIL(CG_ERR_NULL, "cg_nll_loss_fwd_static: null input");
  if (ld < c) CG_FAIL(CG_ERR_SIZE, "cg_nll_loss_fwd_static: leading dimension smaller than c");
  void *p = nullptr;
  CG_TRY(static_scratch(&p));
  const int64_t parts = ceil_div64(n, kEwThreads);
  int64_t *pcnt = (int64_t *)p;  // same layout as cg_nll_loss_fwd: the 8-byte aligned part first
  float *psum = (float *)(pcnt + parts + 1);
  // Nothing has to start at zero: the first pass writes every partial sum the second one reads.
  if (parts > 0) {
    nll_partial_kernel<<<(unsigned)parts, kEwThreads, 0, stream>>>(d_logp, ld, d_y, d_mask, n, c, psum, pcnt);
    CG_LAUNCH_CHECK();
  }
  nll_final_kernel<<<1, kEwThreads, 0, stream>>>(psum, pcnt, parts, d_loss, d_count);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

int cg_log_softmax_nll_fwd(const float *d_z, int64_t ldz, const int64_t *d_y, const uint8_t *d_mask, float *d_out,
                           int64_t ldo, int64_t n, int32_t c, float *d_loss, int64_t *d_count, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t s = (hipStream_t)stream_;
  CG_TRY(check_rows("cg_log_softmax_nll_fwd", n, c));
  if (!d_loss || !d_count) CG_FAIL(CG_ERR_NULL, "cg_log_softmax_nll_fwd: null output");
  if (n > 0 && (!d_z || !d_out || !d_y)) CG_FAIL(CG_ERR_NULL, "cg_log_softmax_nll_fwd: null pointer");
  if (ldz < c || ldo < c) CG_FAIL(CG_ERR_SIZE, "cg_log_softmax_nll_fwd: leading dimension smaller than c");
  const int64_t parts = ceil_div64(n, kEwThreads);
  void *p = nullptr;
  const size_t head = (size_t)(parts + 1) * (sizeof(float) + sizeof(int64_t)) + 16;
  CG_TRY(scratch_get(s, kSlotB, head + (size_t)(n > 0 ? n : 1) * sizeof(float), &p));
  int64_t *pcnt = (int64_t *)p;  // 8-byte aligned part first
  float *psum = (float *)(pcnt + parts + 1);
  float *rowloss = (float *)((char *)p + (head & ~(size_t)15));
  if (n > 0) {
    ProfScope prof("log_softmax_fwd", c, s);
    switch (vec_team(c, ldz, ldo, 4, d_z, d_out, nullptr)) {
#define CG_CASE(T)                                                                                                 \
  case T:                                                                                                          \
    log_softmax_fwd_vec_kernel<T, true><<<row_grid(n, T), kEwThreads, 0, s>>>(d_z, ldz, d_out, ldo, n, c, d_y, d_mask, \
                                                                              rowloss);                            \
    break;
      CG_CASE(1) CG_CASE(2) CG_CASE(4) CG_CASE(8) CG_CASE(16)
#undef CG_CASE
      default:
        log_softmax_fwd_kernel<true><<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, s>>>(d_z, ldz, d_out, ldo, n, c,
                                                                                                   d_y, d_mask, rowloss);
    }
    CG_LAUNCH_CHECK();
  }
  ProfScope prof("nll_fwd", c, s);
  if (parts > 0) {
    nll_rows_partial_kernel<<<(unsigned)parts, kEwThreads, 0, s>>>(rowloss, d_y, d_mask, n, c, psum, pcnt);
    CG_LAUNCH_CHECK();
  }
  nll_final_kernel<<<1, kEwThreads, 0, s>>>(psum, pcnt, parts, d_loss, d_count);
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
  hipStream_t s = (hipStream_t)stream;
  ProfScope prof("nll_bwd", c, s);
  switch (vec_team(c, ld, 4, 4, d_dlogp, nullptr, nullptr)) {
#define CG_CASE(T)                                                                                                \
  case T:                                                                                                         \
    nll_bwd_vec_kernel<T, false><<<row_grid(n, T), kEwThreads, 0, s>>>(nullptr, 0, d_y, d_mask, d_count, d_gscale, \
                                                                       d_dlogp, ld, n, c);                        \
    break;
    CG_CASE(1) CG_CASE(2) CG_CASE(4) CG_CASE(8) CG_CASE(16)
#undef CG_CASE
    default:
      nll_bwd_kernel<false><<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, s>>>(nullptr, 0, d_y, d_mask, d_count,
                                                                                          d_gscale, d_dlogp, ld, n, c);
  }
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
  hipStream_t s = (hipStream_t)stream;
  ProfScope prof("log_softmax_nll_bwd", c, s);
  switch (vec_team(c, ld, lddz, 4, d_logp, d_dz, nullptr)) {
#define CG_CASE(T)                                                                                               \
  case T:                                                                                                        \
    nll_bwd_vec_kernel<T, true><<<row_grid(n, T), kEwThreads, 0, s>>>(d_logp, ld, d_y, d_mask, d_count, d_gscale, \
                                                                      d_dz, lddz, n, c);                         \
    break;
    CG_CASE(1) CG_CASE(2) CG_CASE(4) CG_CASE(8) CG_CASE(16)
#undef CG_CASE
    default:
      nll_bwd_kernel<true><<<(unsigned)ceil_div64(n, kRowsPerBlock), kEwThreads, 0, s>>>(d_logp, ld, d_y, d_mask, d_count,
                                                                                         d_gscale, d_dz, lddz, n, c);
  }
  CG_LAUNCH_CHECK();
  return CG_OK;
}

}  // extern "C"
