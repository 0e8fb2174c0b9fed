// Shared host/device helpers of libcagnet_amd (gfx950 only: 64-wide wavefronts).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/cagnet_amd.h"

namespace cg {

constexpr int kWave = 64;

// ---- error plumbing -----------------------------------------------------------------------
void set_error(const char *fmt, ...);
int hip_fail(hipError_t e, const char *what, const char *file, int line);

#define CG_HIP(call)                                                        \
  do {                                                                      \
    hipError_t e_ = (call);                                                 \
    if (e_ != hipSuccess) return cg::hip_fail(e_, #call, __FILE__, __LINE__); \
  } while (0)

#define CG_TRY(call)              \
  do {                            \
    int s_ = (call);              \
    if (s_ != CG_OK) return s_;   \
  } while (0)

#define CG_FAIL(code, ...)        \
  do {                            \
    cg::set_error(__VA_ARGS__);   \
    return (code);                \
  } while (0)

// Launch check: kernel launches report configuration errors through hipGetLastError.
#define CG_LAUNCH_CHECK() CG_HIP(hipGetLastError())

// ---- per (device, stream) grow-only scratch ------------------------------------------------
// slot: independent buffers that must be alive at the same time use different slots.
enum ScratchSlot { kSlotA = 0, kSlotB = 1, kSlotC = 2, kSlotD = 3, kSlotE = 4, kNumSlots = 5 };
int scratch_get(hipStream_t stream, int slot, size_t bytes, void **out);

// Frees every scratch buffer of (current device, stream), parked ones included, after the stream has drained.
int scratch_release(hipStream_t stream, int64_t *released_bytes);

// ---- memory that a captured graph may still name -------------------------------------------------
// A HIP graph captured from calls of this library keeps the raw addresses of the scratch buffers and
// of the handle's tables those calls used.  A buffer or table that was used under capture is therefore
// never freed by later calls: when it has to be replaced (scratch growth, plan eviction, schedule
// recycling, a changed tuning value) the old memory is parked and only the owner's release frees it.
bool stream_capturing(hipStream_t stream);
// Free `p`, or park it when the calling thread is inside a product on a pinned handle (ParkScope).
void table_free(void *p);
struct ParkScope {  // tables released inside the scope go to `sink` instead of hipFree (sink == nullptr: no change)
  void *prev;
  bool set;
  explicit ParkScope(void *sink_vector);
  ~ParkScope();
};
// CG_ERR_CAPTURE unless `stream` is not being captured: for steps that allocate, synchronise or read back.
int refuse_under_capture(hipStream_t stream, const char *what);

// ---- optional kernel timing with HIP events on the launch stream (runtime.hip) -------------------
bool prof_on();
void prof_begin(const char *name, int tag, hipStream_t stream);  // tag < 0: no "/f=" suffix
void prof_end(hipStream_t stream);
struct ProfScope {
  hipStream_t s;
  bool on;
  ProfScope(const char *name, int tag, hipStream_t stream) : s(stream), on(prof_on()) {
    if (on) prof_begin(name, tag, stream);
  }
  ~ProfScope() {
    if (on) prof_end(s);
  }
};

// ---- integer helpers ------------------------------------------------------------------------
static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline int bits_for(int32_t count) {  // number of bits needed to represent values in [0, count)
  int b = 0;
  uint32_t v = count > 1 ? (uint32_t)(count - 1) : 0u;
  while (v) { ++b; v >>= 1; }
  return b;
}

// ---- device-side scan / sort building blocks (scan.hip, sort.hip) ----------------------------
// Exclusive prefix sum of d_in[0..count) into d_out (may alias d_in); if d_total != nullptr the
// grand total is stored there.  Values and totals must fit uint32.
int exclusive_scan_u32(const uint32_t *d_in, uint32_t *d_out, int64_t count, uint32_t *d_total, hipStream_t stream);

// Stable LSD radix sort of `count` records (key_a, key_b, payload) by the low `bits` bits of
// the array selected per pass: first all digits of key_b (minor key), then those of key_a
// (major key).  Arrays are ping-ponged between buffer set 0 and 1; returns which set holds the
// result in *result_set.  Either bit count may be 0 (that key is then not sorted on).
struct SortBuffers {
  int32_t *key_a[2];
  int32_t *key_b[2];
  int32_t *payload[2];
};
int radix_sort_pairs(SortBuffers &buf, int64_t count, int bits_a, int bits_b, int *result_set, hipStream_t stream);

// The same sort from caller-owned inputs to caller-owned outputs: the first pass reads `in_*`, the
// last writes `out_*`, the passes between ping-pong through `tmp` (both sets are needed from three
// passes on).  in_p == nullptr: the payload is the record's position in the input (the result is
// the sorting permutation).  payload == false: none is carried.  Outputs that are nullptr are
// dropped.  The inputs are never written.
struct SortIo {
  const int32_t *in_a, *in_b, *in_p;
  int32_t *out_a, *out_b, *out_p;
  bool payload;
};
int radix_sort_records(const SortIo &io, SortBuffers &tmp, int64_t count, int bits_a, int bits_b, hipStream_t stream);

// coo2csr.hip
int launch_rowptr(const int32_t *d_row, int64_t nnz, int32_t n, int32_t *d_rowptr, hipStream_t stream);
// row index of every stored entry of a CSR matrix
int expand_rows(const int32_t *d_rowptr, int32_t n, int32_t *d_row, hipStream_t stream);
int coo_check(const int32_t *d_row, const int32_t *d_col, int64_t nnz, int32_t n, int32_t m, int require_sorted,
              hipStream_t stream);
int coo2csr_general(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n,
                    int32_t m, int32_t *d_rowptr, int32_t *d_colind, float *d_values, int32_t *d_perm,
                    hipStream_t stream);
int csr_transpose(const int32_t *d_rowptr, const int32_t *d_colind, const float *d_values, int64_t nnz, int32_t n,
                  int32_t m, int32_t *d_colptr, int32_t *d_rowind, float *d_values_t, int32_t *d_perm,
                  hipStream_t stream);

}  // namespace cg
