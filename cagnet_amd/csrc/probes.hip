// Machine probes: small kernels that measure the ceilings the design notes argue from, on the device the
// library runs on.  They have no counterpart in the reference and no part in any product.
//   LDS read bandwidth (ds_read_b32 / b64 / b128, conflict free, every lane)
//   streaming read and copy bandwidth of device memory
//   a dense fp32 matrix-core product P[K x f] = D[K x K] * B[rows picked from a larger B] in the tile shape a
//   dense hub block of the SpMM would take (64-row panels, 16-column blocks of D staged as MFMA operands,
//   the matching 16 rows of B staged in LDS)
#include "common.h"

namespace cg {

template <int W>
__global__ __launch_bounds__(1024) void probe_lds_kernel(float *out, int iters, int lds_floats) {
  extern __shared__ float probe_lds[];
  for (int i = threadIdx.x; i < lds_floats; i += blockDim.x) probe_lds[i] = (float)i;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // every read of a wave covers 64 * W contiguous bytes; eight reads in flight per wave
  const unsigned addr = (unsigned)((wave * 64 * W * 8 + lane * W) % (lds_floats * 4 - 8 * 64 * W));
  float a0 = 0, a1 = 0, a2 = 0, a3 = 0;
  for (int it = 0; it < iters; ++it) {
    if (W == 16) {
      float4 v0, v1, v2, v3, v4, v5, v6, v7;
      asm volatile(
          "ds_read_b128 %0, %8\n ds_read_b128 %1, %8 offset:1024\n ds_read_b128 %2, %8 offset:2048\n ds_read_b128 %3, %8 offset:3072\n"
          "ds_read_b128 %4, %8 offset:4096\n ds_read_b128 %5, %8 offset:5120\n ds_read_b128 %6, %8 offset:6144\n ds_read_b128 %7, %8 offset:7168\n"
          "s_waitcnt lgkmcnt(0)\n"
          : "=v"(v0), "=v"(v1), "=v"(v2), "=v"(v3), "=v"(v4), "=v"(v5), "=v"(v6), "=v"(v7)
          : "v"(addr));
      a0 += v0.x + v7.w; a1 += v1.y + v6.z; a2 += v2.z + v5.y; a3 += v3.w + v4.x;
    } else if (W == 8) {
      float2 v0, v1, v2, v3, v4, v5, v6, v7;
      asm volatile(
          "ds_read_b64 %0, %8\n ds_read_b64 %1, %8 offset:512\n ds_read_b64 %2, %8 offset:1024\n ds_read_b64 %3, %8 offset:1536\n"
          "ds_read_b64 %4, %8 offset:2048\n ds_read_b64 %5, %8 offset:2560\n ds_read_b64 %6, %8 offset:3072\n ds_read_b64 %7, %8 offset:3584\n"
          "s_waitcnt lgkmcnt(0)\n"
          : "=v"(v0), "=v"(v1), "=v"(v2), "=v"(v3), "=v"(v4), "=v"(v5), "=v"(v6), "=v"(v7)
          : "v"(addr));
      a0 += v0.x + v7.y; a1 += v1.y + v6.x; a2 += v2.x + v5.y; a3 += v3.y + v4.x;
    } else {
      float v0, v1, v2, v3, v4, v5, v6, v7;
      asm volatile(
          "ds_read_b32 %0, %8\n ds_read_b32 %1, %8 offset:256\n ds_read_b32 %2, %8 offset:512\n ds_read_b32 %3, %8 offset:768\n"
          "ds_read_b32 %4, %8 offset:1024\n ds_read_b32 %5, %8 offset:1280\n ds_read_b32 %6, %8 offset:1536\n ds_read_b32 %7, %8 offset:1792\n"
          "s_waitcnt lgkmcnt(0)\n"
          : "=v"(v0), "=v"(v1), "=v"(v2), "=v"(v3), "=v"(v4), "=v"(v5), "=v"(v6), "=v"(v7)
          : "v"(addr));
      a0 += v0 + v7; a1 += v1 + v6; a2 += v2 + v5; a3 += v3 + v4;
    }
  }
  if (a0 + a1 + a2 + a3 == 12345.678f) out[threadIdx.x] = a0;  // keeps the reads alive
}

// `passes` sweeps over the buffer inside one launch: a working set that fits a cache is then read from it
__global__ __launch_bounds__(256) void probe_read_kernel(const float4 *__restrict__ src, int64_t count, int passes, float *out) {
  float s = 0.f;
  for (int p = 0; p < passes; ++p)
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
      const float4 v = src[i];
      s += v.x + v.y + v.z + v.w;
    }
  if (s == 12345.678f) out[0] = s;
}

__global__ __launch_bounds__(256) void probe_copy_kernel(const float4 *__restrict__ src, float4 *__restrict__ dst, int64_t count) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void probe_fill_kernel(float *p, int64_t count, uint32_t seed) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (int64_t)gridDim.x * 256) {
    uint32_t x = (uint32_t)i * 2654435761u + seed;
    x ^= x >> 15;
    x *= 2246822519u;
    x ^= x >> 13;
    p[i] = (float)(x & 0xffff) * (1.0f / 65536.0f) - 0.5f;
  }
}

// ---- dense matrix-core product ---------------------------------------------------------------------
typedef float floatx4 __attribute__((ext_vector_type(4)));
constexpr int kProbeKB = 16, kProbePM = 64, kProbeStride = 612;  // 4 * stride = 16 (mod 64): conflict-free operand reads

// Dt: [panel][column block][4 row tiles][64 lanes][4]: lane (r, g) of row tile m holds D[16 m + r][4 g .. 4 g + 3]
// of the block, i.e. the A operands of the four matrix instructions of a block, one 16-byte load per tile.
template <int NT>
__global__ __launch_bounds__(256) void probe_mfma_kernel(const float *__restrict__ Dt, int nkb, const int32_t *__restrict__ qidx,
                                                         const float *__restrict__ B, int64_t ldb, float *__restrict__ P, int f,
                                                         int ntn) {
  __shared__ float lds[2][kProbeKB * kProbeStride];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int panel = blockIdx.x, nsplit = blockIdx.y;
  const int wg_n0 = nsplit * (4 * NT * 16);
  int wg_cols = f - wg_n0;
  if (wg_cols > 4 * NT * 16) wg_cols = 4 * NT * 16;
  const int nt0 = nsplit * 4 * NT + wave * NT;
  int ntc = ntn - nt0;
  ntc = ntc > NT ? NT : (ntc < 0 ? 0 : ntc);
  floatx4 acc[4][NT];
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int n = 0; n < NT; ++n) acc[m][n] = (floatx4){0.f, 0.f, 0.f, 0.f};
  const int npair = (wg_cols + 1) / 2;
  constexpr int kIt = (4 * NT * 16 / 2 + 63) / 64;
  float2 st[4][kIt];
  auto stage_load = [&](int kb) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int q = qidx[kb * kProbeKB + wave * 4 + r];
      const float *src = B + (int64_t)q * ldb + wg_n0;
#pragma unroll
      for (int i = 0; i < kIt; ++i) {
        int p = lane + 64 * i;
        p = p < npair ? p : npair - 1;
        st[r][i] = *reinterpret_cast<const float2 *>(src + 2 * p);
      }
    }
  };
  auto stage_store = [&](int buf) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int i = 0; i < kIt; ++i) {
        const int p = lane + 64 * i;
        if (p < npair) *reinterpret_cast<float2 *>(&lds[buf][(wave * 4 + r) * kProbeStride + 2 * p]) = st[r][i];
      }
  };
  float4 av[4], av_next[4];
  auto a_load = [&](int kb, float4 (&dst)[4]) {
    const float4 *src = reinterpret_cast<const float4 *>(Dt) + ((int64_t)panel * nkb + kb) * 256 + lane;
#pragma unroll
    for (int m = 0; m < 4; ++m) dst[m] = src[m * 64];
  };
  stage_load(0);
  a_load(0, av);
  stage_store(0);
  __syncthreads();
  for (int kb = 0; kb < nkb; ++kb) {
    const int buf = kb & 1;
    const bool more = kb + 1 < nkb;
    if (more) {
      stage_load(kb + 1);
      a_load(kb + 1, av_next);
    }
    const float *lb = &lds[buf][wave * NT * 16 + c];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      float b[NT];
#pragma unroll
      for (int n = 0; n < NT; ++n) b[n] = lb[(4 * g + s) * kProbeStride + n * 16];
#pragma unroll
      for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const float am = s == 0 ? av[m].x : (s == 1 ? av[m].y : (s == 2 ? av[m].z : av[m].w));
          acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x4f32(am, b[n], acc[m][n], 0, 0, 0);
        }
    }
    if (more) {
      stage_store(buf ^ 1);
#pragma unroll
      for (int m = 0; m < 4; ++m) av[m] = av_next[m];
    }
    __syncthreads();
  }
#pragma unroll
  for (int n = 0; n < NT; ++n) {
    if (n < ntc) {
      const int col = (nt0 + n) * 16 + c;
      if (col < f) {
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
          for (int v = 0; v < 4; ++v) P[(int64_t)(panel * kProbePM + 16 * m + 4 * g + v) * f + col] = acc[m][n][v];
      }
    }
  }
}

__global__ __launch_bounds__(256) void probe_qidx_kernel(int32_t *q, int count, int rows) {
  const int k = blockIdx.x * 256 + threadIdx.x;
  if (k < count) q[k] = (int32_t)(((int64_t)k * 7919 + 13) % rows);
}

struct ProbeMem {  // frees what a probe allocated, also on an early return
  void *p[8] = {nullptr};
  int n = 0;
  ~ProbeMem() {
    for (int i = 0; i < n; ++i)
      if (p[i]) (void)hipFree(p[i]);
  }
  int get(void **out, size_t bytes) {
    hipError_t e = hipMalloc(out, bytes);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      CG_FAIL(CG_ERR_ALLOC, "probe: hipMalloc of %zu bytes failed", bytes);
    }
    p[n++] = *out;
    return CG_OK;
  }
};

static int time_ms(hipEvent_t e0, hipEvent_t e1, float *ms) {
  CG_HIP(hipEventSynchronize(e1));
  CG_HIP(hipEventElapsedTime(ms, e0, e1));
  return CG_OK;
}

}  // namespace cg

extern "C" {

int cg_probe_lds_read(int32_t bytes_per_lane, int32_t threads_per_workgroup, double *tb_per_s) {
  using namespace cg;
  if (!tb_per_s) CG_FAIL(CG_ERR_NULL, "cg_probe_lds_read: null result");
  if ((bytes_per_lane != 4 && bytes_per_lane != 8 && bytes_per_lane != 16) || threads_per_workgroup < 64 ||
      threads_per_workgroup > 1024 || threads_per_workgroup % 64)
    CG_FAIL(CG_ERR_SIZE, "cg_probe_lds_read: bytes_per_lane must be 4, 8 or 16 and threads a multiple of 64 up to 1024");
  hipDeviceProp_t prop;
  int dev = 0;
  CG_HIP(hipGetDevice(&dev));
  CG_HIP(hipGetDeviceProperties(&prop, dev));
  ProbeMem mem;
  float *out = nullptr;
  CG_TRY(mem.get((void **)&out, 4096));
  const int iters = 4000, lds_floats = 16 * 1024;  // 64 KB per workgroup: two workgroups per CU
  const int grid = prop.multiProcessorCount * 8;
  hipEvent_t e0, e1;
  CG_HIP(hipEventCreate(&e0));
  CG_HIP(hipEventCreate(&e1));
  float best = 1e30f;
  for (int rep = 0; rep < 4; ++rep) {
    CG_HIP(hipEventRecord(e0, nullptr));
    if (bytes_per_lane == 16) probe_lds_kernel<16><<<grid, threads_per_workgroup, lds_floats * 4>>>(out, iters, lds_floats);
    else if (bytes_per_lane == 8) probe_lds_kernel<8><<<grid, threads_per_workgroup, lds_floats * 4>>>(out, iters, lds_floats);
    else probe_lds_kernel<4><<<grid, threads_per_workgroup, lds_floats * 4>>>(out, iters, lds_floats);
    CG_LAUNCH_CHECK();
    CG_HIP(hipEventRecord(e1, nullptr));
    float ms = 0.f;
    CG_TRY(time_ms(e0, e1, &ms));
    if (rep > 0 && ms < best) best = ms;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *tb_per_s = (double)grid * threads_per_workgroup * iters * 8.0 * bytes_per_lane / (best * 1e-3) / 1e12;
  return CG_OK;
}

int cg_probe_stream(int64_t bytes, int32_t copy, double *tb_per_s) {
  using namespace cg;
  if (!tb_per_s) CG_FAIL(CG_ERR_NULL, "cg_probe_stream: null result");
  if (bytes < (1 << 20) || bytes % 16) CG_FAIL(CG_ERR_SIZE, "cg_probe_stream: bytes must be a multiple of 16, at least 1 MiB");
  ProbeMem mem;
  float *src = nullptr, *dst = nullptr, *out = nullptr;
  CG_TRY(mem.get((void **)&src, (size_t)bytes));
  if (copy) CG_TRY(mem.get((void **)&dst, (size_t)bytes));
  CG_TRY(mem.get((void **)&out, 64));
  probe_fill_kernel<<<4096, 256>>>(src, bytes / 4, 1u);
  CG_LAUNCH_CHECK();
  hipEvent_t e0, e1;
  CG_HIP(hipEventCreate(&e0));
  CG_HIP(hipEventCreate(&e1));
  float best = 1e30f;
  // Up to 32 MiB (the L2 caches together) the sweeps of a read run inside one launch: a launch would
  // otherwise take longer to start than to run.  Larger working sets are swept by back-to-back launches, so
  // that every sweep goes through the whole buffer before the next one starts (sweeps inside a launch would
  // let every workgroup re-read its own few KB from L2).
  const bool inside = !copy && bytes <= ((int64_t)32 << 20);
  const int reps = bytes <= ((int64_t)256 << 20) ? 32 : 4;
  const unsigned grid = (unsigned)(bytes / 16 / 256 < 8192 ? bytes / 16 / 256 : 8192);
  for (int rep = 0; rep < 4; ++rep) {
    CG_HIP(hipEventRecord(e0, nullptr));
    if (inside) {
      probe_read_kernel<<<grid, 256>>>((const float4 *)src, bytes / 16, reps, out);
    } else {
      for (int k = 0; k < reps; ++k) {
        if (copy) probe_copy_kernel<<<grid, 256>>>((const float4 *)src, (float4 *)dst, bytes / 16);
        else probe_read_kernel<<<grid, 256>>>((const float4 *)src, bytes / 16, 1, out);
      }
    }
    CG_LAUNCH_CHECK();
    CG_HIP(hipEventRecord(e1, nullptr));
    float ms = 0.f;
    CG_TRY(time_ms(e0, e1, &ms));
    if (rep > 0 && ms < best) best = ms;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *tb_per_s = (double)bytes * (copy ? 2.0 : 1.0) * reps / (best * 1e-3) / 1e12;
  return CG_OK;
}

int cg_probe_mfma_dense(int32_t k, int32_t f, double *ms_out, double *tflops) {
  using namespace cg;
  if (!ms_out || !tflops) CG_FAIL(CG_ERR_NULL, "cg_probe_mfma_dense: null result");
  if (k < 64 || k > 32768 || f < 16 || f > 640 || f % 2) CG_FAIL(CG_ERR_SIZE, "cg_probe_mfma_dense: 64 <= k <= 32768, even f in 16..640");
  const int npanels = k / kProbePM, nkb = k / kProbeKB;
  const int kr = npanels * kProbePM, kc = nkb * kProbeKB, rows_b = 232965;
  ProbeMem mem;
  float *Dt = nullptr, *B = nullptr, *P = nullptr;
  int32_t *q = nullptr;
  CG_TRY(mem.get((void **)&Dt, (size_t)kr * kc * 4));
  CG_TRY(mem.get((void **)&B, (size_t)rows_b * f * 4));
  CG_TRY(mem.get((void **)&P, (size_t)kr * f * 4));
  CG_TRY(mem.get((void **)&q, (size_t)kc * 4));
  probe_fill_kernel<<<4096, 256>>>(Dt, (int64_t)kr * kc, 7u);
  probe_fill_kernel<<<4096, 256>>>(B, (int64_t)rows_b * f, 11u);
  probe_qidx_kernel<<<(kc + 255) / 256, 256>>>(q, kc, rows_b);
  CG_LAUNCH_CHECK();
  const int ntn = (f + 15) / 16;
  const dim3 grid((unsigned)npanels, (unsigned)((ntn + 19) / 20));
  hipEvent_t e0, e1;
  CG_HIP(hipEventCreate(&e0));
  CG_HIP(hipEventCreate(&e1));
  float best = 1e30f;
  for (int rep = 0; rep < 5; ++rep) {
    CG_HIP(hipEventRecord(e0, nullptr));
    probe_mfma_kernel<5><<<grid, 256>>>(Dt, nkb, q, B, f, P, f, ntn);
    CG_LAUNCH_CHECK();
    CG_HIP(hipEventRecord(e1, nullptr));
    float ms = 0.f;
    CG_TRY(time_ms(e0, e1, &ms));
    if (rep > 0 && ms < best) best = ms;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  *ms_out = best;
  *tflops = 2.0 * kr * kc * f / (best * 1e-3) / 1e12;
  return CG_OK;
}

}  // extern "C"
