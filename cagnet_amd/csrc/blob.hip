// A sparse block as one contiguous byte string: what a rank would read from disk or receive from a
// peer.  The reference keeps its adjacency matrix as a pickled int64 COO tensor (gcn_distr.py:747)
// and ships blocks between ranks as three float32 arrays, indices included
// (gcn_distr_2d.py:369-374), which loses index bits above 2^24.  This format carries int32 CSR
// with fp32 values, checked on the way in.
//
// Layout, little endian, every array starting on a 64-byte boundary:
//   0   char[8]  magic "CGNTCSR\0"
//   8   uint32   version (1)
//   12  uint32   flags   (bit 0: the writer's handle carried the transpose; a reader rebuilds it)
//   16  int64    n, m, nnz
//   40  uint64   offset of rowptr  (int32[n + 1])
//   48  uint64   offset of colind  (int32[nnz])
//   56  uint64   offset of values  (float[nnz])
//   64  uint64   total bytes
//   72  uint64   checksum of bytes [128, total): FNV-1a over 64-bit words
//   80..127      zero
#include "common.h"
#include <string.h>
#include <vector>

namespace cg {

constexpr uint64_t kBlobHeader = 128;
constexpr uint64_t kBlobAlign = 64;
static const char kBlobMagic[8] = {'C', 'G', 'N', 'T', 'C', 'S', 'R', '\0'};

struct BlobHeader {
  char magic[8];
  uint32_t version, flags;
  int64_t n, m, nnz;
  uint64_t off_rowptr, off_colind, off_values, total, checksum;
  uint8_t reserved[48];
};
static_assert(sizeof(BlobHeader) == kBlobHeader, "blob header is 128 bytes");

static uint64_t align_up(uint64_t v) { return (v + kBlobAlign - 1) / kBlobAlign * kBlobAlign; }

static void blob_layout(int64_t n, int64_t nnz, BlobHeader &h) {
  h.off_rowptr = kBlobHeader;
  h.off_colind = align_up(h.off_rowptr + (uint64_t)(n + 1) * 4);
  h.off_values = align_up(h.off_colind + (uint64_t)nnz * 4);
  h.total = align_up(h.off_values + (uint64_t)nnz * 4);
}

static uint64_t blob_checksum(const uint8_t *p, uint64_t bytes) {  // bytes is a multiple of 8
  uint64_t hsh = 1469598103934665603ull;
  for (uint64_t i = 0; i < bytes; i += 8) {
    uint64_t w;
    memcpy(&w, p + i, 8);
    hsh = (hsh ^ w) * 1099511628211ull;
  }
  return hsh;
}

}  // namespace cg

extern "C" {

int cg_csr_blob_size(const cg_csr_t *h, int64_t *bytes) {
  using namespace cg;
  if (!h || !bytes) CG_FAIL(CG_ERR_NULL, "cg_csr_blob_size: null pointer");
  int64_t info[8];
  CG_TRY(cg_csr_info(h, info));
  BlobHeader hd;
  blob_layout(info[0], info[2], hd);
  *bytes = (int64_t)hd.total;
  return CG_OK;
}

int cg_csr_blob_write(const cg_csr_t *h, void *host_buf, int64_t capacity, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  if (!h || !host_buf) CG_FAIL(CG_ERR_NULL, "cg_csr_blob_write: null pointer");
  int64_t info[8];
  CG_TRY(cg_csr_info(h, info));
  BlobHeader hd;
  memset(&hd, 0, sizeof(hd));
  memcpy(hd.magic, kBlobMagic, 8);
  hd.version = 1;
  hd.flags = info[3] ? 1u : 0u;
  hd.n = info[0];
  hd.m = info[1];
  hd.nnz = info[2];
  blob_layout(hd.n, hd.nnz, hd);
  if (capacity < (int64_t)hd.total)
    CG_FAIL(CG_ERR_SIZE, "cg_csr_blob_write: buffer of %lld bytes, %llu needed", (long long)capacity,
            (unsigned long long)hd.total);
  const int32_t *d_rowptr = nullptr, *d_colind = nullptr;
  const float *d_val = nullptr;
  CG_TRY(cg_csr_arrays(h, 0, &d_rowptr, &d_colind, &d_val));
  uint8_t *out = (uint8_t *)host_buf;
  memset(out + kBlobHeader, 0, hd.total - kBlobHeader);  // padding bytes are part of the checksum
  CG_HIP(hipMemcpyAsync(out + hd.off_rowptr, d_rowptr, (size_t)(hd.n + 1) * 4, hipMemcpyDeviceToHost, stream));
  if (hd.nnz > 0) {
    CG_HIP(hipMemcpyAsync(out + hd.off_colind, d_colind, (size_t)hd.nnz * 4, hipMemcpyDeviceToHost, stream));
    CG_HIP(hipMemcpyAsync(out + hd.off_values, d_val, (size_t)hd.nnz * 4, hipMemcpyDeviceToHost, stream));
  }
  CG_HIP(hipStreamSynchronize(stream));
  hd.checksum = blob_checksum(out + kBlobHeader, hd.total - kBlobHeader);
  memcpy(out, &hd, sizeof(hd));
  return CG_OK;
}

int cg_csr_blob_read(cg_csr_t **out, const void *host_buf, int64_t bytes, uint32_t flags, cg_stream_t stream_) {
  using namespace cg;
  hipStream_t stream = (hipStream_t)stream_;
  if (!out) CG_FAIL(CG_ERR_NULL, "cg_csr_blob_read: out is NULL");
  *out = nullptr;
  if (!host_buf) CG_FAIL(CG_ERR_NULL, "cg_csr_blob_read: buffer is NULL");
  if (bytes < (int64_t)kBlobHeader) CG_FAIL(CG_ERR_SIZE, "cg_csr_blob_read: %lld bytes hold no header", (long long)bytes);
  const uint8_t *in = (const uint8_t *)host_buf;
  BlobHeader hd;
  memcpy(&hd, in, sizeof(hd));
  if (memcmp(hd.magic, kBlobMagic, 8) != 0) CG_FAIL(CG_ERR_UNSUPPORTED, "cg_csr_blob_read: not a CSR blob (bad magic)");
  if (hd.version != 1) CG_FAIL(CG_ERR_UNSUPPORTED, "cg_csr_blob_read: version %u is not supported", hd.version);
  if (hd.n < 0 || hd.m < 0 || hd.nnz < 0 || hd.n >= 0x7fffffffLL || hd.m >= 0x7fffffffLL || hd.nnz >= 0x7fffffffLL)
    CG_FAIL(CG_ERR_OVERFLOW, "cg_csr_blob_read: sizes n=%lld m=%lld nnz=%lld outside the int32 contract", (long long)hd.n,
            (long long)hd.m, (long long)hd.nnz);
  BlobHeader want;
  blob_layout(hd.n, hd.nnz, want);
  if (hd.off_rowptr != want.off_rowptr || hd.off_colind != want.off_colind || hd.off_values != want.off_values ||
      hd.total != want.total)
    CG_FAIL(CG_ERR_SIZE, "cg_csr_blob_read: array offsets do not match the sizes in the header");
  if ((uint64_t)bytes < hd.total)
    CG_FAIL(CG_ERR_SIZE, "cg_csr_blob_read: truncated, %lld of %llu bytes", (long long)bytes, (unsigned long long)hd.total);
  if (blob_checksum(in + kBlobHeader, hd.total - kBlobHeader) != hd.checksum)
    CG_FAIL(CG_ERR_INDEX, "cg_csr_blob_read: checksum mismatch");
  // rowptr is checked on the host, the column range by cg_csr_create on the device
  std::vector<int32_t> rowptr((size_t)hd.n + 1);
  memcpy(rowptr.data(), in + hd.off_rowptr, rowptr.size() * 4);
  if (rowptr[0] != 0 || rowptr[(size_t)hd.n] != (int32_t)hd.nnz)
    CG_FAIL(CG_ERR_INDEX, "cg_csr_blob_read: rowptr does not span [0, nnz]");
  for (int64_t i = 0; i < hd.n; ++i)
    if (rowptr[(size_t)i + 1] < rowptr[(size_t)i]) CG_FAIL(CG_ERR_UNSORTED, "cg_csr_blob_read: rowptr descends at row %lld", (long long)i);
  if (hd.nnz > 0 && (hd.n == 0 || hd.m == 0)) CG_FAIL(CG_ERR_SIZE, "cg_csr_blob_read: entries in an empty matrix");

  int32_t *d_rowptr = nullptr, *d_row = nullptr, *d_col = nullptr;
  float *d_val = nullptr;
  int st = CG_OK;
  do {
    const size_t eb = (size_t)(hd.nnz > 0 ? hd.nnz : 1) * 4;
    if (hipMalloc((void **)&d_rowptr, rowptr.size() * 4) != hipSuccess || hipMalloc((void **)&d_row, eb) != hipSuccess ||
        hipMalloc((void **)&d_col, eb) != hipSuccess || hipMalloc((void **)&d_val, eb) != hipSuccess) {
      (void)hipGetLastError();
      set_error("cg_csr_blob_read: device allocation failed");
      st = CG_ERR_ALLOC;
      break;
    }
    if (hipMemcpyAsync(d_rowptr, rowptr.data(), rowptr.size() * 4, hipMemcpyHostToDevice, stream) != hipSuccess) { st = CG_ERR_HIP; break; }
    if (hd.nnz > 0) {
      if (hipMemcpyAsync(d_col, in + hd.off_colind, (size_t)hd.nnz * 4, hipMemcpyHostToDevice, stream) != hipSuccess ||
          hipMemcpyAsync(d_val, in + hd.off_values, (size_t)hd.nnz * 4, hipMemcpyHostToDevice, stream) != hipSuccess) { st = CG_ERR_HIP; break; }
    }
    if ((st = expand_rows(d_rowptr, (int32_t)hd.n, d_row, stream)) != CG_OK) break;
    const uint32_t cflags = CG_CSR_SORTED | (((hd.flags & 1u) || (flags & CG_CSR_TRANSPOSE)) ? CG_CSR_TRANSPOSE : 0u);
    st = cg_csr_create(out, d_row, d_col, d_val, hd.nnz, (int32_t)hd.n, (int32_t)hd.m, cflags, stream);
  } while (0);
  if (st == CG_ERR_HIP) set_error("cg_csr_blob_read: host to device copy failed");
  (void)hipStreamSynchronize(stream);
  if (d_rowptr) (void)hipFree(d_rowptr);
  if (d_row) (void)hipFree(d_row);
  if (d_col) (void)hipFree(d_col);
  if (d_val) (void)hipFree(d_val);
  return st;
}

}  // extern "C"
