// COO -> CSR conversion, CSR transpose and input validation.
//
// Row compression replaces the cusparseXcoo2csr call of the reference operator
// (sparse-extension/sparse_coo_tensor.cu:136-142).  The general path (unsorted input) and the
// transpose are a stable radix sort followed by the same compression; the reference has neither
// (its callers coalesce on the CPU, gcn_distr.py:546, and its backward assumes A == A^T,
// gcn_distr.py:326).
#include "common.h"

namespace cg {

constexpr int kThreads = 256;

// One thread per boundary k in [0, nnz]: rows in (row[k-1], row[k]] start at position k.
// Long runs of empty rows are filled by the whole wave instead of one lane.
__global__ __launch_bounds__(kThreads) void rowptr_kernel(const int32_t *__restrict__ row, int64_t nnz, int32_t n,
                                                          int32_t *__restrict__ rowptr) {
  const int64_t k = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int lane = threadIdx.x & (kWave - 1);
  int32_t lo = 1, hi = 0;
  if (k <= nnz) {
    int32_t prev = k == 0 ? -1 : row[k - 1];
    int32_t cur = k == nnz ? n : row[k];
    prev = prev < -1 ? -1 : (prev > n - 1 ? n - 1 : prev);  // clamp: bad input must not write outside rowptr
    cur = cur < -1 ? -1 : (cur > n ? n : cur);
    lo = prev + 1;
    hi = cur;
  }
  const int32_t gap = hi - lo + 1;
  if (gap > 0 && gap <= 8) {
    for (int32_t i = lo; i <= hi; ++i) rowptr[i] = (int32_t)k;
  }
  uint64_t longs = __ballot(gap > 8);
  while (longs) {
    const int src = __builtin_ctzll(longs);
    longs &= longs - 1;
    const int32_t slo = __shfl(lo, src, kWave);
    const int32_t shi = __shfl(hi, src, kWave);
    const int32_t sk = (int32_t)__shfl((int32_t)k, src, kWave);
    for (int32_t i = slo + lane; i <= shi; i += kWave) rowptr[i] = sk;
  }
}

int launch_rowptr(const int32_t *d_row, int64_t nnz, int32_t n, int32_t *d_rowptr, hipStream_t stream) {
  const int64_t blocks = ceil_div64(nnz + 1, kThreads);
  rowptr_kernel<<<(unsigned)blocks, kThreads, 0, stream>>>(d_row, nnz, n, d_rowptr);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

// flags: bit0 index out of range, bit1 rows descend, bit2 (row, col) not strictly ascending
__global__ __launch_bounds__(kThreads) void coo_check_kernel(const int32_t *__restrict__ row,
                                                             const int32_t *__restrict__ col, int64_t nnz, int32_t n,
                                                             int32_t m, int care, int *__restrict__ flags) {
  const int64_t k = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  int f = 0;
  if (k < nnz) {
    const int32_t r = row[k];
    const int32_t c = col ? col[k] : 0;
    if (r < 0 || r >= n || c < 0 || c >= m) f |= 1;
    if (k > 0) {
      const int32_t pr = row[k - 1];
      if (pr > r) f |= 2;
      if (col && (pr > r || (pr == r && col[k - 1] >= c))) f |= 4;
    }
  }
  f &= care;  // only what the caller asked about (unsorted input is expected on the general path)
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) f |= __shfl_xor(f, off, kWave);
  if (f && (threadIdx.x & (kWave - 1)) == 0) atomicOr(flags, f);  // one per wavefront; integer OR: order independent
}

__global__ __launch_bounds__(kThreads) void gather_f32_kernel(const float *__restrict__ src,
                                                              const int32_t *__restrict__ perm,
                                                              float *__restrict__ dst, int64_t count) {
  const int64_t k = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (k < count) dst[k] = src[perm[k]];
}

// row index of every stored entry of a CSR matrix: one wave per row
__global__ __launch_bounds__(kThreads) void csr_expand_rows_kernel(const int32_t *__restrict__ rowptr, int32_t n,
                                                                   int32_t *__restrict__ row_out) {
  const int64_t wave = ((int64_t)blockIdx.x * kThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (wave >= n) return;
  const int32_t s = rowptr[wave], e = rowptr[wave + 1];
  for (int32_t k = s + lane; k < e; k += kWave) row_out[k] = (int32_t)wave;
}

int expand_rows(const int32_t *d_rowptr, int32_t n, int32_t *d_row, hipStream_t stream) {
  if (n <= 0) return CG_OK;
  csr_expand_rows_kernel<<<(unsigned)ceil_div64((int64_t)n * kWave, kThreads), kThreads, 0, stream>>>(d_rowptr, n,
                                                                                                     d_row);
  CG_LAUNCH_CHECK();
  return CG_OK;
}

static int check_common(int64_t nnz, int32_t n, int32_t m) {
  if (nnz < 0 || n < 0 || m < 0) CG_FAIL(CG_ERR_SIZE, "negative size: nnz=%lld n=%d m=%d", (long long)nnz, n, m);
  if (nnz > 0x7fffffffLL - 1) CG_FAIL(CG_ERR_OVERFLOW, "nnz=%lld does not fit the int32 rowptr contract", (long long)nnz);
  if (n == 0x7fffffff || m == 0x7fffffff) CG_FAIL(CG_ERR_OVERFLOW, "n + 1 overflows int32");
  return CG_OK;
}

int coo_check(const int32_t *d_row, const int32_t *d_col, int64_t nnz, int32_t n, int32_t m, int require_sorted,
              hipStream_t stream) {
  if (nnz == 0) return CG_OK;
  void *d_flags = nullptr;
  CG_TRY(scratch_get(stream, kSlotD, sizeof(int), &d_flags));
  CG_HIP(hipMemsetAsync(d_flags, 0, sizeof(int), stream));
  const int care = 1 | (require_sorted >= 1 ? 2 : 0) | (require_sorted >= 2 ? 4 : 0);
  coo_check_kernel<<<(unsigned)ceil_div64(nnz, kThreads), kThreads, 0, stream>>>(d_row, d_col, nnz, n, m, care,
                                                                                 (int *)d_flags);
  CG_LAUNCH_CHECK();
  int flags = 0;
  CG_HIP(hipMemcpyAsync(&flags, d_flags, sizeof(int), hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  if (flags & 1) CG_FAIL(CG_ERR_INDEX, "COO index outside [0,%d) x [0,%d)", n, m);
  if (require_sorted >= 1 && (flags & 2)) CG_FAIL(CG_ERR_UNSORTED, "COO rows are not ascending");
  if (require_sorted >= 2 && (flags & 4)) CG_FAIL(CG_ERR_UNSORTED, "COO (row, col) pairs are not strictly ascending");
  return CG_OK;
}

// One device allocation carved into the temporaries of an operation (every hipMalloc / hipFree of a
// few hundred MB costs milliseconds, more than the kernels that use it).
struct DevArena {
  char *base = nullptr;
  size_t cap = 0, off = 0;
  ~DevArena() {
    if (base) (void)hipFree(base);
  }
  static size_t pad(size_t bytes) { return (bytes + 255) & ~(size_t)255; }
  int reserve(size_t bytes) {
    hipError_t e = hipMalloc((void **)&base, bytes ? bytes : 256);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      base = nullptr;
      set_error("hipMalloc of %zu bytes failed: %s", bytes, hipGetErrorString(e));
      return CG_ERR_ALLOC;
    }
    cap = bytes;
    return CG_OK;
  }
  int take(void **out, size_t bytes) {
    const size_t need = pad(bytes);
    if (off + need > cap) CG_FAIL(CG_ERR_ALLOC, "temporary arena too small (%zu + %zu > %zu)", off, need, cap);
    *out = base + off;
    off += need;
    return CG_OK;
  }
};

static size_t sort_coo_bytes(int64_t count) { return 6 * DevArena::pad((size_t)count * sizeof(int32_t)); }

// Sort records (key_a major, key_b minor) from the caller's arrays into the caller's outputs.
// payload == nullptr with want_perm: the records carry their input position, d_out_p receives the
// sorting permutation.  payload != nullptr: its 32-bit words travel with the records (values need no
// gather by permutation afterwards).  Neither: the keys travel alone.
// `tmp` must have sort_coo_bytes(count) left; the caller synchronises before its arena goes away.
static int sort_coo(const int32_t *d_key_a, const int32_t *d_key_b, const int32_t *d_payload, bool want_perm,
                    int64_t count, int bits_a, int bits_b, int32_t *d_out_a, int32_t *d_out_b, int32_t *d_out_p,
                    DevArena &tmp, hipStream_t stream) {
  SortBuffers buf;
  const size_t bytes = (size_t)count * sizeof(int32_t);
  for (int s = 0; s < 2; ++s) {
    CG_TRY(tmp.take((void **)&buf.key_a[s], bytes));
    CG_TRY(tmp.take((void **)&buf.key_b[s], bytes));
    CG_TRY(tmp.take((void **)&buf.payload[s], bytes));
  }
  const SortIo io{d_key_a, d_key_b, d_payload, d_out_a, d_out_b, d_out_p, d_payload != nullptr || want_perm};
  return radix_sort_records(io, buf, count, bits_a, bits_b, stream);
}

// Values ride along as the payload unless the caller wants the permutation, in which case they are
// gathered by it afterwards.
struct ValuePlan {
  const int32_t *payload;
  int32_t *out_p;
  bool want_perm, gather;
  ValuePlan(const float *d_val, float *d_val_out, int32_t *d_perm) {
    const bool values = d_val && d_val_out;
    want_perm = d_perm != nullptr;
    gather = values && want_perm;
    payload = values && !want_perm ? reinterpret_cast<const int32_t *>(d_val) : nullptr;
    out_p = want_perm ? d_perm : (values ? reinterpret_cast<int32_t *>(d_val_out) : nullptr);
  }
};

int coo2csr_general(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n,
                    int32_t m, int32_t *d_rowptr, int32_t *d_colind, float *d_values, int32_t *d_perm,
                    hipStream_t stream) {
  DevArena tmp;
  const size_t ebytes = (size_t)nnz * sizeof(int32_t);
  CG_TRY(tmp.reserve(sort_coo_bytes(nnz) + DevArena::pad(ebytes)));
  int32_t *d_rows_sorted = nullptr;
  CG_TRY(tmp.take((void **)&d_rows_sorted, ebytes));
  const ValuePlan vp(d_val, d_values, d_perm);
  CG_TRY(sort_coo(d_row, d_col, vp.payload, vp.want_perm, nnz, bits_for(n), bits_for(m), d_rows_sorted, d_colind,
                  vp.out_p, tmp, stream));
  CG_TRY(launch_rowptr(d_rows_sorted, nnz, n, d_rowptr, stream));
  if (vp.gather && nnz > 0) {
    gather_f32_kernel<<<(unsigned)ceil_div64(nnz, kThreads), kThreads, 0, stream>>>(d_val, d_perm, d_values, nnz);
    CG_LAUNCH_CHECK();
  }
  CG_HIP(hipStreamSynchronize(stream));
  return CG_OK;
}

int csr_transpose(const int32_t *d_rowptr, const int32_t *d_colind, const float *d_values, int64_t nnz, int32_t n,
                  int32_t m, int32_t *d_colptr, int32_t *d_rowind, float *d_values_t, int32_t *d_perm,
                  hipStream_t stream) {
  DevArena tmp;
  const size_t ebytes = (size_t)nnz * sizeof(int32_t);
  CG_TRY(tmp.reserve(sort_coo_bytes(nnz) + 2 * DevArena::pad(ebytes)));
  int32_t *d_rows = nullptr, *d_cols_sorted = nullptr;
  CG_TRY(tmp.take((void **)&d_rows, ebytes));
  CG_TRY(tmp.take((void **)&d_cols_sorted, ebytes));
  if (n > 0) {
    csr_expand_rows_kernel<<<(unsigned)ceil_div64((int64_t)n * kWave, kThreads), kThreads, 0, stream>>>(d_rowptr, n,
                                                                                                       d_rows);
    CG_LAUNCH_CHECK();
  }
  // CSR order is (row, col) ascending, so a stable sort on col alone yields (col, row) order:
  // major key = col (key_a), minor key = row with zero bits (already in place).
  const ValuePlan vp(d_values, d_values_t, d_perm);
  CG_TRY(sort_coo(d_colind, d_rows, vp.payload, vp.want_perm, nnz, bits_for(m), 0, d_cols_sorted, d_rowind, vp.out_p, tmp,
                  stream));
  CG_TRY(launch_rowptr(d_cols_sorted, nnz, m, d_colptr, stream));
  if (vp.gather && nnz > 0) {
    gather_f32_kernel<<<(unsigned)ceil_div64(nnz, kThreads), kThreads, 0, stream>>>(d_values, d_perm, d_values_t, nnz);
    CG_LAUNCH_CHECK();
  }
  CG_HIP(hipStreamSynchronize(stream));
  return CG_OK;
}

}  // namespace cg

extern "C" {

int cg_coo2csr_rowptr(const int32_t *d_row, int64_t nnz, int32_t n, int32_t *d_rowptr, cg_stream_t stream) {
  CG_TRY(cg::check_common(nnz, n, 0));
  if (!d_rowptr || (nnz > 0 && !d_row)) CG_FAIL(CG_ERR_NULL, "cg_coo2csr_rowptr: null pointer");
  return cg::launch_rowptr(d_row, nnz, n, d_rowptr, (hipStream_t)stream);
}

int cg_coo_check(const int32_t *d_row, const int32_t *d_col, int64_t nnz, int32_t n, int32_t m, int require_sorted,
                 cg_stream_t stream) {
  CG_TRY(cg::check_common(nnz, n, m));
  if (nnz > 0 && !d_row) CG_FAIL(CG_ERR_NULL, "cg_coo_check: null row pointer");
  return cg::coo_check(d_row, d_col, nnz, n, m, require_sorted, (hipStream_t)stream);
}

int cg_coo2csr(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n, int32_t m,
               int32_t *d_rowptr, int32_t *d_colind, float *d_values, int32_t *d_perm, cg_stream_t stream) {
  CG_TRY(cg::check_common(nnz, n, m));
  if (!d_rowptr || (nnz > 0 && (!d_row || !d_col || !d_colind))) CG_FAIL(CG_ERR_NULL, "cg_coo2csr: null pointer");
  if (d_val && !d_values) CG_FAIL(CG_ERR_NULL, "cg_coo2csr: values given but no output for them");
  return cg::coo2csr_general(d_row, d_col, d_val, nnz, n, m, d_rowptr, d_colind, d_values, d_perm,
                             (hipStream_t)stream);
}

int cg_csr_transpose(const int32_t *d_rowptr, const int32_t *d_colind, const float *d_values, int64_t nnz, int32_t n,
                     int32_t m, int32_t *d_colptr, int32_t *d_rowind, float *d_values_t, int32_t *d_perm,
                     cg_stream_t stream) {
  CG_TRY(cg::check_common(nnz, n, m));
  if (!d_rowptr || !d_colptr || (nnz > 0 && (!d_colind || !d_rowind)))
    CG_FAIL(CG_ERR_NULL, "cg_csr_transpose: null pointer");
  if (d_values && !d_values_t) CG_FAIL(CG_ERR_NULL, "cg_csr_transpose: values given but no output for them");
  return cg::csr_transpose(d_rowptr, d_colind, d_values, nnz, n, m, d_colptr, d_rowind, d_values_t, d_perm,
                           (hipStream_t)stream);
}

}  // extern "C"
