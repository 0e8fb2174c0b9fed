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

__global__ __launch_bounds__(kPrepThreads) void fill_zero_u32_kernel(uint32_t *__restrict__ p, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  if (i < count) p[i] = 0u;
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
// ascending.  Per row (one thread, binary search in the ascending columns): below[i] = entries left
// of the diagonal, diag[i] = 1 if the input holds (i, i); count[i] = entries of output row i.
__global__ __launch_bounds__(kPrepThreads) void loops_rows_kernel(const int32_t *__restrict__ rowptr,
                                                                  const int32_t *__restrict__ col, int32_t n,
                                                                  uint32_t *__restrict__ count,
                                                                  int32_t *__restrict__ below,
                                                                  uint8_t *__restrict__ diag) {
  const int64_t r = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  if (r > n) return;
  if (r == n) {  // the scan runs over n + 1 entries so that entry n receives the total
    count[r] = 0u;
    return;
  }
  const int32_t s = rowptr[r], e = rowptr[r + 1];
  int32_t lo = s, hi = e;  // first position whose column is >= r
  while (lo < hi) {
    const int32_t mid = lo + (hi - lo) / 2;
    if (col[mid] < (int32_t)r) lo = mid + 1;
    else hi = mid;
  }
  const bool has = lo < e && col[lo] == (int32_t)r;
  below[r] = lo - s;
  diag[r] = has ? 1 : 0;
  count[r] = (uint32_t)(e - s) - (has ? 1u : 0u) + 1u;
}

// One thread per input entry: entries left of the diagonal keep their rank in the row, the others
// move by one for the inserted diagonal (and back by one if the input's own diagonal entry, which
// is dropped here, preceded them).
__global__ __launch_bounds__(kPrepThreads) void loops_entries_kernel(
    const int32_t *__restrict__ row, const int32_t *__restrict__ col, int64_t nnz, const int32_t *__restrict__ rowptr,
    const uint32_t *__restrict__ obase, const uint8_t *__restrict__ diag, int32_t *__restrict__ out_row,
    int32_t *__restrict__ out_col) {
  for (int64_t k = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x; k < nnz; k += (int64_t)gridDim.x * kPrepThreads) {
    const int32_t r = row[k], c = col[k];
    if (c == r) continue;
    int64_t pos = (int64_t)obase[r] + (k - rowptr[r]);
    if (c > r) pos += 1 - (int64_t)diag[r];
    out_row[pos] = r;
    out_col[pos] = c;
  }
}

__global__ __launch_bounds__(kPrepThreads) void loops_diag_kernel(const uint32_t *__restrict__ obase,
                                                                  const int32_t *__restrict__ below, int32_t n,
                                                                  int32_t *__restrict__ out_row,
                                                                  int32_t *__restrict__ out_col) {
  const int64_t r = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  if (r >= n) return;
  const int64_t pos = (int64_t)obase[r] + below[r];
  out_row[pos] = (int32_t)r;
  out_col[pos] = (int32_t)r;
}

// ---- block extraction ---------------------------------------------------------------------------
// Order-preserving compaction in tiles of kBlockTile entries: a count per tile, an exclusive scan of
// the tile counts, then every tile ranks its own matches (wave ballots, running counts) and writes
// them behind its base.  Wave w of a workgroup owns entries [tile + 1024 w, tile + 1024 (w + 1)).
constexpr int kBlockRounds = 16;
constexpr int kBlockWaveTile = kBlockRounds * kWave;
constexpr int kBlockTile = (kPrepThreads / kWave) * kBlockWaveTile;  // 4096

__device__ __forceinline__ bool in_block(int32_t r, int32_t c, int32_t r0, int32_t r1, int32_t c0, int32_t c1) {
  return r >= r0 && r < r1 && c >= c0 && c < c1;
}

__global__ __launch_bounds__(kPrepThreads) void block_count_kernel(const int32_t *__restrict__ row,
                                                                   const int32_t *__restrict__ col, int64_t nnz,
                                                                   int32_t r0, int32_t r1, int32_t c0, int32_t c1,
                                                                   int64_t tiles, uint32_t *__restrict__ tile_count) {
  __shared__ uint32_t wsum[kPrepThreads / kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if ((int64_t)blockIdx.x == tiles) {  // the scan runs over tiles + 1 entries so that the last receives the total
    if (threadIdx.x == 0) tile_count[tiles] = 0u;
    return;
  }
  const int64_t base = (int64_t)blockIdx.x * kBlockTile + (int64_t)wave * kBlockWaveTile;
  uint32_t cnt = 0;
#pragma unroll
  for (int i = 0; i < kBlockRounds; ++i) {
    const int64_t k = base + (int64_t)i * kWave + lane;
    const bool hit = k < nnz && in_block(row[k < nnz ? k : 0], col[k < nnz ? k : 0], r0, r1, c0, c1);
    cnt += (uint32_t)__popcll(__ballot(hit));
  }
  if (lane == 0) wsum[wave] = cnt;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t t = 0;
    for (int w = 0; w < kPrepThreads / kWave; ++w) t += wsum[w];
    tile_count[blockIdx.x] = t;
  }
}

__global__ __launch_bounds__(kPrepThreads) void block_compact_kernel(
    const int32_t *__restrict__ row, const int32_t *__restrict__ col, const float *__restrict__ val, int64_t nnz,
    int32_t r0, int32_t r1, int32_t c0, int32_t c1, const uint32_t *__restrict__ tile_base, int64_t capacity,
    int32_t *__restrict__ out_row, int32_t *__restrict__ out_col, float *__restrict__ out_val) {
  __shared__ uint32_t wsum[kPrepThreads / kWave];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const uint64_t lower = (1ull << lane) - 1ull;
  const int64_t base = (int64_t)blockIdx.x * kBlockTile + (int64_t)wave * kBlockWaveTile;
  int32_t rr[kBlockRounds], cc[kBlockRounds];
  uint32_t rank[kBlockRounds];  // rank of a match among the wave's matches; ~0u: not in the block
  uint32_t cnt = 0;
#pragma unroll
  for (int i = 0; i < kBlockRounds; ++i) {
    const int64_t k = base + (int64_t)i * kWave + lane;
    const int64_t kc = k < nnz ? k : 0;
    rr[i] = row[kc];
    cc[i] = col[kc];
    const bool hit = k < nnz && in_block(rr[i], cc[i], r0, r1, c0, c1);
    const uint64_t bal = __ballot(hit);
    rank[i] = hit ? cnt + (uint32_t)__popcll(bal & lower) : ~0u;
    cnt += (uint32_t)__popcll(bal);
  }
  if (lane == 0) wsum[wave] = cnt;
  __syncthreads();
  int64_t o = tile_base[blockIdx.x];
  for (int w = 0; w < wave; ++w) o += wsum[w];
#pragma unroll
  for (int i = 0; i < kBlockRounds; ++i) {
    if (rank[i] != ~0u) {
      const int64_t pos = o + rank[i];
      if (pos < capacity) {
        out_row[pos] = rr[i] - r0;  // rebased like split_coo (gcn_distr.py:406)
        out_col[pos] = cc[i] - c0;
        if (val) out_val[pos] = val[base + (int64_t)i * kWave + lane];
      }
    }
  }
}

// ---- blocks side by side ------------------------------------------------------------------------
// [A_0 | A_1 | ...]: the blocks of one block row of a partitioned matrix as one matrix, so that the stage loop
// sum_k A_k H_k (gcn_distr.py:221-244, gcn_distr_2d.py:333-417) becomes one product with the stacked H_k.
constexpr int kStackMax = 16;  // blocks of one call
struct StackArgs {
  const int32_t *rowptr[kStackMax];
  const int32_t *colind[kStackMax];
  const float *val[kStackMax];
  int32_t coloff[kStackMax];
  int32_t count;
};

// counts[i] = entries of row i over all blocks (counts[n] = 0: the place of the scan's total)
__global__ __launch_bounds__(kPrepThreads) void stack_count_kernel(const StackArgs a, int32_t n, uint32_t *__restrict__ counts) {
  const int64_t i = (int64_t)blockIdx.x * kPrepThreads + threadIdx.x;
  if (i > n) return;
  uint32_t c = 0;
  if (i < n)
    for (int k = 0; k < a.count; ++k) c += (uint32_t)(a.rowptr[k][i + 1] - a.rowptr[k][i]);
  counts[i] = c;
}

// One wave per row: the row's entries of block 0, then of block 1, ... with the blocks' column offsets added;
// the (row, column) order of the blocks is kept.
__global__ __launch_bounds__(kPrepThreads) void stack_rows_kernel(const StackArgs a, int32_t n,
                                                                  const uint32_t *__restrict__ rowptr_out,
                                                                  int32_t *__restrict__ row_out, int32_t *__restrict__ col_out,
                                                                  float *__restrict__ val_out) {
  const int64_t i = ((int64_t)blockIdx.x * kPrepThreads + threadIdx.x) / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (i >= n) return;
  int64_t at = rowptr_out[i];
  for (int k = 0; k < a.count; ++k) {
    const int32_t s = a.rowptr[k][i], e = a.rowptr[k][i + 1];
    for (int32_t j = s + lane; j < e; j += kWave) {
      const int64_t o = at + (j - s);
      row_out[o] = (int32_t)i;
      col_out[o] = a.colind[k][j] + a.coloff[k];
      val_out[o] = a.val[k][j];
    }
    at += e - s;
  }
}

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
  // degrees and their inverse roots live in the stream's scratch: no allocation, no synchronisation
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, (size_t)n * (sizeof(uint32_t) + sizeof(float)), &p));
  uint32_t *deg = (uint32_t *)p;
  float *dinv = d_dinv ? d_dinv : (float *)(deg + n);
  fill_zero_u32_kernel<<<grid_for(n), kPrepThreads, 0, stream>>>(deg, n);
  CG_LAUNCH_CHECK();
  prep_degree_kernel<<<grid_for(nnz), kPrepThreads, 0, stream>>>(d_row, nnz, n, deg);
  CG_LAUNCH_CHECK();
  prep_dinv_kernel<<<grid_for(n), kPrepThreads, 0, stream>>>(deg, n, dinv);
  CG_LAUNCH_CHECK();
  prep_scale_kernel<<<grid_for(nnz), kPrepThreads, 0, stream>>>(d_row, d_col, nnz, n, dinv, d_val);
  CG_LAUNCH_CHECK();
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
  // per-row tables in the stream's scratch: rowptr[n+1], below[n], obase[n+2], diag[n]
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, (size_t)(3 * (int64_t)n + 3) * sizeof(int32_t) + (size_t)n, &p));
  int32_t *rowptr = (int32_t *)p, *below = rowptr + n + 1;
  uint32_t *obase = (uint32_t *)(below + n), *d_total = obase + n + 1;
  uint8_t *diag = (uint8_t *)(obase + n + 2);
  CG_TRY(launch_rowptr(d_row, nnz, n, rowptr, stream));
  loops_rows_kernel<<<grid_for((int64_t)n + 1), kPrepThreads, 0, stream>>>(rowptr, d_col, n, obase, below, diag);
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
  if (nnz > 0) {
    int64_t blocks = ceil_div64(nnz, kPrepThreads);
    if (blocks > 256 * 64) blocks = 256 * 64;
    loops_entries_kernel<<<(unsigned)blocks, kPrepThreads, 0, stream>>>(d_row, d_col, nnz, rowptr, obase, diag,
                                                                        d_out_row, d_out_col);
    CG_LAUNCH_CHECK();
  }
  loops_diag_kernel<<<grid_for(n), kPrepThreads, 0, stream>>>(obase, below, n, d_out_row, d_out_col);
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
  // tile counts live in the stream's scratch: the call allocates nothing
  const int64_t tiles = ceil_div64(nnz, kBlockTile);
  void *p = nullptr;
  CG_TRY(scratch_get(stream, kSlotB, (size_t)(tiles + 2) * sizeof(uint32_t), &p));
  uint32_t *tile_count = (uint32_t *)p, *d_total = tile_count + tiles + 1;
  block_count_kernel<<<(unsigned)(tiles + 1), kPrepThreads, 0, stream>>>(d_row, d_col, nnz, r0, r1, c0, c1, tiles,
                                                                      tile_count);
  CG_LAUNCH_CHECK();
  CG_TRY(exclusive_scan_u32(tile_count, tile_count, tiles + 1, d_total, stream));
  uint32_t total = 0;
  CG_HIP(hipMemcpyAsync(&total, d_total, sizeof(total), hipMemcpyDeviceToHost, stream));
  CG_HIP(hipStreamSynchronize(stream));
  *out_nnz = total;
  if (total == 0 || (!d_out_row && !d_out_col && !d_out_val)) return CG_OK;  // empty block, or counting call
  if ((int64_t)total > capacity)
    CG_FAIL(CG_ERR_SIZE, "cg_coo_block: block has %u entries, capacity is %lld", total, (long long)capacity);
  if (!d_out_row || !d_out_col || (d_val && !d_out_val)) CG_FAIL(CG_ERR_NULL, "cg_coo_block: null output");
  block_compact_kernel<<<(unsigned)tiles, kPrepThreads, 0, stream>>>(d_row, d_col, d_val, nnz, r0, r1, c0, c1,
                                                                    tile_count, capacity, d_out_row, d_out_col,
                                                                    d_out_val);
  CG_LAUNCH_CHECK();
  CG_HIP(hipStreamSynchronize(stream));
  return CG_OK;
}

int cg_csr_hstack(cg_csr_t **out, cg_csr_t *const *blocks, int32_t count, uint32_t flags, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  if (!out) CG_FAIL(CG_ERR_NULL, "cg_csr_hstack: out is NULL");
  *out = nullptr;
  if (!blocks) CG_FAIL(CG_ERR_NULL, "cg_csr_hstack: blocks is NULL");
  if (count < 1 || count > kStackMax) CG_FAIL(CG_ERR_SIZE, "cg_csr_hstack: %d blocks (1 .. %d are supported)", count, kStackMax);
  StackArgs a{};
  a.count = count;
  int64_t n = -1, m = 0, nnz = 0;
  for (int k = 0; k < count; ++k) {
    if (!blocks[k]) CG_FAIL(CG_ERR_NULL, "cg_csr_hstack: block %d is NULL", k);
    int64_t info[8];
    CG_TRY(cg_csr_info(blocks[k], info));
    CG_TRY(cg_csr_arrays(blocks[k], 0, &a.rowptr[k], &a.colind[k], &a.val[k]));
    if (n >= 0 && info[0] != n) CG_FAIL(CG_ERR_SIZE, "cg_csr_hstack: block %d has %lld rows, block 0 has %lld", k, (long long)info[0], (long long)n);
    n = info[0];
    a.coloff[k] = (int32_t)m;
    m += info[1];
    nnz += info[2];
  }
  if (m >= 0x7fffffffLL || nnz >= 0x7fffffffLL)
    CG_FAIL(CG_ERR_OVERFLOW, "cg_csr_hstack: %lld columns and %lld entries are outside the int32 contract", (long long)m, (long long)nnz);
  CG_TRY(refuse_under_capture(stream, "stacking blocks"));
  uint32_t *counts = nullptr;
  int32_t *d_row = nullptr, *d_col = nullptr;
  float *d_val = nullptr;
  int st = CG_OK;
  do {
    const size_t eb = (size_t)(nnz > 0 ? nnz : 1) * 4;
    if (hipMalloc((void **)&counts, (size_t)(n + 1) * 4) != hipSuccess || hipMalloc((void **)&d_row, eb) != hipSuccess ||
        hipMalloc((void **)&d_col, eb) != hipSuccess || hipMalloc((void **)&d_val, eb) != hipSuccess) {
      (void)hipGetLastError();
      set_error("cg_csr_hstack: device allocation failed");
      st = CG_ERR_ALLOC;
      break;
    }
    stack_count_kernel<<<grid_for(n + 1), kPrepThreads, 0, stream>>>(a, (int32_t)n, counts);
    if (hipGetLastError() != hipSuccess) { st = CG_ERR_HIP; break; }
    if ((st = exclusive_scan_u32(counts, counts, n + 1, nullptr, stream)) != CG_OK) break;
    if (n > 0) {
      stack_rows_kernel<<<grid_for(n * kWave), kPrepThreads, 0, stream>>>(a, (int32_t)n, counts, d_row, d_col, d_val);
      if (hipGetLastError() != hipSuccess) { st = CG_ERR_HIP; break; }
    }
    st = cg_csr_create(out, d_row, d_col, d_val, nnz, (int32_t)n, (int32_t)m,
                       CG_CSR_SORTED | (flags & CG_CSR_TRANSPOSE), stream);
  } while (0);
  if (st == CG_ERR_HIP) set_error("cg_csr_hstack: kernel launch failed");
  (void)hipStreamSynchronize(stream);
  if (counts) (void)hipFree(counts);
  if (d_row) (void)hipFree(d_row);
  if (d_col) (void)hipFree(d_col);
  if (d_val) (void)hipFree(d_val);
  return st;
}

}  // extern "C"
