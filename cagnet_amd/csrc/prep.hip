// Input preparation of the GCN on the device: self-loops, D^-1/2 (A+I) D^-1/2 scaling and block
// extraction.  The reference does all three on the host (add_remaining_self_loops at
// gcn_distr.py:791, scale_elements at gcn_distr.py:412-470, split_coo at gcn_distr.py:398-409).
// Integer work is exact; the scaling follows the reference's arithmetic step by step, so the
// values equal the host result bit for bit.
#include "common.h"

namespace cg {

constexpr int kPrepThreads = 256;

// ---- degree and scaling -------------------------------------------------------------------------
// Runs of equal row indices inside a wavefront (the whole wavefront, for row-sorted input) are
// counted with one atomic each.
__global__ __launch_bounds__(kPrepThreads) void prep_degree_kernel(const int32_t *__restrict__ row, int64_t nnz,
                                                                   int32_t n, uint32_t *__restrict__ deg) {
  const int64_t k = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  int32_t r = -1;
  if (k < nnz) {
    r = row[k];
    if (r < 0 || r >= n) r = -1;
  }
  const int32_t prev = __shfl_up(r, 1, kWave);
  const bool leader = lane == 0 || r != prev;
  const uint64_t leaders = __ballot(leader);
  if (leader && r >= 0) {
    const uint64_t above = lane == kWave - 1 ? 0ull : leaders >> (lane + 1);
    const int run = above ? __builtin_ctzll(above) + 1 : kWave - lane;
    atomicAdd(&deg[r], (uint32_t)run);  // integer count: independent of arrival order
  }
}

// dinv[i] = fl32(deg_i ^ -1/2), the power taken in fp64 (gcn_distr.py:440-448); deg == 0 gives +inf
// like the reference's pow.  The fp64 square root and division are correctly rounded.
__global__ __launch_bounds__(kPrepThreads) void prep_dinv_kernel(const uint32_t *__restrict__ deg, int32_t n,
                                                                 float *__restrict__ dinv) {
  const int64_t i = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  if (i < n) dinv[i] = (float)(1.0 / sqrt((double)deg[i]));
}

// val = fl32(dinv[row] * fl32(1 * dinv[col])): scaled on the right, then on the left (gcn_distr.py:458-464)
__global__ __launch_bounds__(kPrepThreads) void prep_scale_kernel(const int32_t *__restrict__ row,
                                                                  const int32_t *__restrict__ col, int64_t nnz,
                                                                  int32_t n, const float *__restrict__ dinv,
                                                                  float *__restrict__ val) {
  const int64_t k = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  if (k >= nnz) return;
  const int32_t r = row[k], c = col[k];
  const bool ok = r >= 0 && r < n && c >= 0 && c < n;
  const float right = ok ? 1.0f * dinv[c] : 0.f;
  val[k] = ok ? dinv[r] * right : 0.f;
}

// ---- self-loops ---------------------------------------------------------------------------------
// Row i of the result = row i of the input without its diagonal entry, plus (i, i), columns
// ascending.  One wavefront per row.  count[i] = entries of output row i.
__global__ __launch_bounds__(kPrepThreads) void loops_count_kernel(const int32_t *__restrict__ rowptr,
                                                                   const int32_t *__restrict__ col, int32_t n,
                                                                   uint32_t *__restrict__ count) {
  const int64_t r = ((int64_t)blockIdx.x * kPrepThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (r > n) return;
  if (r == n) {  // the scan runs over n + 1 entries so that entry n receives the total
    if (lane == 0) count[r] = 0u;
    return;
  }
  const int32_t s = rowptr[r], e = rowptr[r + 1];
  uint32_t diag = 0;
  for (int32_t k = s + lane; k < e; k += kWave) diag += col[k] == (int32_t)r ? 1u : 0u;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) diag += __shfl_xor(diag, off, kWave);
  if (lane == 0) count[r] = (uint32_t)(e - s) - diag + 1u;
}

__global__ __launch_bounds__(kPrepThreads) void loops_fill_kernel(const int32_t *__restrict__ rowptr,
                                                                  const int32_t *__restrict__ col, int32_t n,
                                                                  const uint32_t *__restrict__ obase,
                                                                  int32_t *__restrict__ out_row,
                                                                  int32_t *__restrict__ out_col) {
  const int64_t r = ((int64_t)blockIdx.x * kPrepThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (r >= n) return;
  const int32_t s = rowptr[r], e = rowptr[r + 1];
  const int64_t o = obase[r];
  // entries below the diagonal keep their rank, the diagonal follows them, the rest moves by one
  // (or stays, when the row already held a diagonal entry that is dropped here)
  uint32_t below = 0;
  for (int32_t k = s + lane; k < e; k += kWave) below += col[k] < (int32_t)r ? 1u : 0u;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) below += __shfl_xor(below, off, kWave);
  if (lane == 0) {
    out_row[o + below] = (int32_t)r;
    out_col[o + below] = (int32_t)r;
  }
  // ranks among the entries above the diagonal: columns ascend, so the input position gives them
  uint32_t skipped = 0;  // diagonal entries of the input met so far
  for (int32_t base = s; base < e; base += kWave) {
    const int32_t k = base + lane;
    const int32_t c = k < e ? col[k] : -1;
    const bool is_diag = k < e && c == (int32_t)r;
    const uint64_t dmask = __ballot(is_diag);
    const uint32_t before = skipped + (uint32_t)__popcll(dmask & ((1ull << lane) - 1ull));
    if (k < e && !is_diag) {
      const int64_t pos = c < (int32_t)r ? (int64_t)(k - s) - before : (int64_t)(k - s) - before + 1;
      out_row[o + pos] = (int32_t)r;
      out_col[o + pos] = c;
    }
    skipped += (uint32_t)__popcll(dmask);
  }
}

// ---- block extraction ---------------------------------------------------------------------------
__global__ __launch_bounds__(kPrepThreads) void block_flag_kernel(const int32_t *__restrict__ row,
                                                                  const int32_t *__restrict__ col, int64_t nnz,
                                                                  int32_t r0, int32_t r1, int32_t c0, int32_t c1,
                                                                  uint32_t *__restrict__ flag) {
  const int64_t k = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  if (k > nnz) return;
  if (k == nnz) {
    flag[k] = 0u;
    return;
  }
  const int32_t r = row[k], c = col[k];
  flag[k] = (r >= r0 && r < r1 && c >= c0 && c < c1) ? 1u : 0u;
}

__global__ __launch_bounds__(kPrepThreads) void block_scatter_kernel(
    const int32_t *__restrict__ row, const int32_t *__restrict__ col, const float *__restrict__ val, int64_t nnz,
    int32_t r0, int32_t r1, int32_t c0, int32_t c1, const uint32_t *__restrict__ pos, int64_t capacity,
    int32_t *__restrict__ out_row, int32_t *__restrict__ out_col, float *__restrict__ out_val) {
  const int64_t k = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  if (k >= nnz) return;
  const int32_t r = row[k], c = col[k];
  if (!(r >= r0 && r < r1 && c >= c0 && c < c1)) return;
  const int64_t o = pos[k];
  if (o >= capacity) return;
  out_row[o] = r - r0;  // rebased like split_coo (gcn_distr.py:406)
  out_col[o] = c - c0;
  if (val) out_val[o] = val[k];
}

struct PrepTemp {
  void *p[4] = {nullptr, nullptr, nullptr, nullptr};
  int count = 0;
  ~PrepTemp() {
    for (int i = 0; i < count; ++i)
      if (p[i]) (void)hipFree(p[i]);
  }
  int alloc(void **out, size_t bytes) {
    hipError_t e = hipMalloc(out, bytes ? bytes : 4);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      *out = nullptr;
      set_error("hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
      return CG_ERR_ALLOC;
    }
    p[count++] = *out;
    return CG_OK;
  }
};

static unsigned grid_for(int64_t count) { return (unsigned)ceil_div64(count > 0 ? count : 1, kPrepThreads); }

}  // namespace cg

extern "C" {

int cg_gcn_normalize(const int32_t *d_row, const int32_t *d_col, int64_t nnz, int32_t n, float *d_val,
                     float *d_dinv, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  if (nnz < 0 || n < 0) CG_FAIL(CG_ERR_SIZE, "cg_gcn_normalize: negative size");
  if (nnz > 0x7fffffffLL - 1) CG_FAIL(CG_ERR_OVERFLOW, "cg_gcn_normalize: nnz=%lld exceeds int32", (long long)nnz);
  if (nnz > 0 && (!d_row || !d_col || !d_val)) CG_FAIL(CG_ERR_NULL, "cg_gcn_normalize: null operand");
  if (n == 0 || nnz == 0) return CG_OK;
  PrepTemp tmp;
  uint32_t *deg = nullptr;
  float *dinv = d_dinv;
  CG_TRY(tmp.alloc((void **)&deg, (size_t)n * sizeof(uint32_t)));
  if (!dinv) CG_TRY(tmp.alloc((void **)&dinv, (size_t)n * sizeof(float)));
  CG_HIP(hipMemsetAsync(deg, 0, (size_t)n * sizeof(uint32_t), stream));
  prep_degree_kernel<<<grid_for(nnz), kPrepThreads, 0, stream>>>(d_row, nnz, n, deg);
  CG_LAUNCH_CHECK();
  prep_dinv_kernel<<<grid_for(n), kPrepThreads, 0, stream>>>(deg, n, dinv);
  CG_LAUNCH_CHECK();
  prep_scale_kernel<<<grid_for(nnz), kPrepThreads, 0, stream>>>(d_row, d_col, nnz, n, dinv, d_val);
  CG_LAUNCH_CHECK();
  CG_HIP(hipStreamSynchronize(stream));  // the temporaries are freed on return
  return CG_OK;
}

int cg_add_self_loops(const int32_t *d_row, const int32_t *d_col, int64_t nnz, int32_t n, int32_t *d_out_row,
                      int32_t *d_out_col, int64_t capacity, int64_t *out_nnz, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  if (nnz < 0 || n < 0 || capacity < 0) CG_FAIL(CG_ERR_SIZE, "cg_add_self_loops: negative size");
  if (nnz + (int64_t)n > 0x7fffffffLL - 1)
    CG_FAIL(CG_ERR_OVERFLOW, "cg_add_self_loops: nnz + n = %lld exceeds int32", (long long)(nnz + n));
  if (!out_nnz) CG_FAIL(CG_ERR_NULL, "cg_add_self_loops: out_nnz is NULL");
  if (nnz > 0 && (!d_row || !d_col)) CG_FAIL(CG_ERR_NULL, "cg_add_self_loops: null operand");
  *out_nnz = 0;
  if (n == 0) {
    if (nnz > 0) CG_FAIL(CG_ERR_SIZE, "cg_add_self_loops: nnz > 0 with n == 0");
    return CG_OK;
  }
  CG_TRY(coo_check(d_row, d_col, nnz, n, n, 2, stream));  // the ranks below rely on (row, col) order
  PrepTemp tmp;
  int32_t *rowptr = nullptr;
  uint32_t *obase = nullptr, *d_total = nullptr;
  CG_TRY(tmp.alloc((void **)&rowptr, (size_t)(n + 1) * sizeof(int32_t)));
  CG_TRY(tmp.alloc((void **)&obase, (size_t)(n + 2) * sizeof(uint32_t)));
  d_total = obase + n + 1;
  CG_TRY(launch_rowptr(d_row, nnz, n, rowptr, stream));
  const unsigned wgrid = grid_for(((int64_t)n + 1) * kWave);
  loops_count_kernel<<<wgrid, kPrepThreads, 0, stream>>>(rowptr, d_col, n, obase);
  CG_LAUNCH_CHECK();
  CG_TRY(exclusive_scan_u32(obase, obase, (int64_t)n + 1, d_total, stream));
  uint32_t total = 0;
  CG_HIP(hipMemcpyAsync(&total, d_total, sizeof(total), hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  *out_nnz = total;
  if (!d_out_row && !d_out_col) return CG_OK;  // counting call
  if ((int64_t)total > capacity)
    CG_FAIL(CG_ERR_SIZE, "cg_add_self_loops: result has %u entries, capacity is %lld", total, (long long)capacity);
  if (!d_out_row || !d_out_col) CG_FAIL(CG_ERR_NULL, "cg_add_self_loops: null output");
  loops_fill_kernel<<<wgrid, kPrepThreads, 0, stream>>>(rowptr, d_col, n, obase, d_out_row, d_out_col);
  CG_LAUNCH_CHECK();
  CG_HIP(hipStreamSynchronize(stream));
  return CG_OK;
}

int cg_coo_block(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t r0, int32_t r1,
                 int32_t c0, int32_t c1, int32_t *d_out_row, int32_t *d_out_col, float *d_out_val, int64_t capacity,
                 int64_t *out_nnz, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  if (nnz < 0 || capacity < 0) CG_FAIL(CG_ERR_SIZE, "cg_coo_block: negative size");
  if (nnz > 0x7fffffffLL - 1) CG_FAIL(CG_ERR_OVERFLOW, "cg_coo_block: nnz=%lld exceeds int32", (long long)nnz);
  if (r1 < r0 || c1 < c0) CG_FAIL(CG_ERR_SIZE, "cg_coo_block: empty or reversed range");
  if (!out_nnz) CG_FAIL(CG_ERR_NULL, "cg_coo_block: out_nnz is NULL");
  if (nnz > 0 && (!d_row || !d_col)) CG_FAIL(CG_ERR_NULL, "cg_coo_block: null operand");
  *out_nnz = 0;
  if (nnz == 0) return CG_OK;
  PrepTemp tmp;
  uint32_t *flag = nullptr;
  CG_TRY(tmp.alloc((void **)&flag, (size_t)(nnz + 2) * sizeof(uint32_t)));
  uint32_t *d_total = flag + nnz + 1;
  block_flag_kernel<<<grid_for(nnz + 1), kPrepThreads, 0, stream>>>(d_row, d_col, nnz, r0, r1, c0, c1, flag);
  CG_LAUNCH_CHECK();
  CG_TRY(exclusive_scan_u32(flag, flag, nnz + 1, d_total, stream));
  uint32_t total = 0;
  CG_HIP(hipMemcpyAsync(&total, d_total, sizeof(total), hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  *out_nnz = total;
  if (total == 0 || (!d_out_row && !d_out_col && !d_out_val)) return CG_OK;  // empty block, or counting call
  if ((int64_t)total > capacity)
    CG_FAIL(CG_ERR_SIZE, "cg_coo_block: block has %u entries, capacity is %lld", total, (long long)capacity);
  if (!d_out_row || !d_out_col || (d_val && !d_out_val)) CG_FAIL(CG_ERR_NULL, "cg_coo_block: null output");
  block_scatter_kernel<<<grid_for(nnz), kPrepThreads, 0, stream>>>(d_row, d_col, d_val, nnz, r0, r1, c0, c1, flag,
                                                                  capacity, d_out_row, d_out_col, d_out_val);
  CG_LAUNCH_CHECK();
  CG_HIP(hipStreamSynchronize(stream));
  return CG_OK;
}

}  // extern "C"
