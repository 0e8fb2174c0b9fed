// Error reporting and the per (device, stream) scratch arena of libcagnet_amd.
#include "common.h"
#include <atomic>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

namespace cg {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char *what, const char *file, int line) {
  set_error("HIP error %d (%s) at %s:%d in %s", (int)e, hipGetErrorString(e), file, line, what);
  return CG_ERR_HIP;
}

struct ScratchBuf {
  void *ptr = nullptr;
  size_t bytes = 0;
};

static std::mutex g_scratch_mu;
static std::map<std::tuple<int, hipStream_t, int>, ScratchBuf> g_scratch;

// Grow-only.  Growing frees the old buffer after the stream has drained, so work already
// enqueued on `stream` that still reads it stays valid.
int scratch_get(hipStream_t stream, int slot, size_t bytes, void **out) {
  int dev = 0;
  CG_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  ScratchBuf &b = g_scratch[std::make_tuple(dev, stream, slot)];
  if (bytes > b.bytes) {
    if (b.ptr) {
      CG_HIP(hipStreamSynchronize(stream));
      CG_HIP(hipFree(b.ptr));
      b.ptr = nullptr;
      b.bytes = 0;
    }
    size_t want = bytes + bytes / 4;  // headroom so slowly growing requests do not reallocate each time
    want = (want + 255) & ~(size_t)255;
    hipError_t e = hipMalloc(&b.ptr, want);
    if (e != hipSuccess) {
      b.ptr = nullptr;
      set_error("scratch hipMalloc of %zu bytes failed: %s", want, hipGetErrorString(e));
      (void)hipGetLastError();
      return CG_ERR_ALLOC;
    }
    b.bytes = want;
  }
  *out = b.ptr;
  return CG_OK;
}

// ---- event recorder ------------------------------------------------------------------------
struct ProfRecord {
  std::string name;
  hipEvent_t start, stop;
};
static std::mutex g_prof_mu;
static std::vector<ProfRecord> g_prof;
static std::atomic<bool> g_prof_on{false};
static thread_local int g_prof_open = -1;
constexpr size_t kProfMaxRecords = 1 << 16;

bool prof_on() { return g_prof_on.load(std::memory_order_relaxed); }

void prof_begin(const char *name, int tag, hipStream_t stream) {
  g_prof_open = -1;
  ProfRecord r;
  r.name = name;
  if (tag >= 0) r.name += "/f=" + std::to_string(tag);
  if (hipEventCreate(&r.start) != hipSuccess) return;
  if (hipEventCreate(&r.stop) != hipSuccess) {
    (void)hipEventDestroy(r.start);
    return;
  }
  (void)hipEventRecord(r.start, stream);
  std::lock_guard<std::mutex> lock(g_prof_mu);
  if (g_prof.size() >= kProfMaxRecords) {  // full: drop this record rather than grow without bound
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
    return;
  }
  g_prof.push_back(r);
  g_prof_open = (int)g_prof.size() - 1;
}

void prof_end(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_prof_mu);
  if (g_prof_open >= 0 && g_prof_open < (int)g_prof.size()) (void)hipEventRecord(g_prof[g_prof_open].stop, stream);
  g_prof_open = -1;
}

}  // namespace cg

extern "C" {

int cg_prof_enable(int on) {
  cg::g_prof_on.store(on != 0);
  return CG_OK;
}

int cg_prof_read(const char *name, double *total_ms, int64_t *launches) {
  using namespace cg;
  if (!name || !total_ms || !launches) CG_FAIL(CG_ERR_NULL, "cg_prof_read: null pointer");
  std::lock_guard<std::mutex> lock(g_prof_mu);
  double total = 0.0;
  int64_t count = 0;
  std::vector<ProfRecord> keep;
  for (auto &r : g_prof) {
    if (r.name != name) {
      keep.push_back(r);
      continue;
    }
    float ms = 0.f;
    if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
      total += ms;
      ++count;
    } else {
      (void)hipGetLastError();
    }
    (void)hipEventDestroy(r.start);
    (void)hipEventDestroy(r.stop);
  }
  g_prof.swap(keep);
  *total_ms = total;
  *launches = count;
  return CG_OK;
}

int cg_abi_version(void) { return CG_ABI_VERSION; }

const char *cg_status_string(int status) {
  switch (status) {
    case CG_OK: return "ok";
    case CG_ERR_NULL: return "null pointer";
    case CG_ERR_SIZE: return "bad size";
    case CG_ERR_OVERFLOW: return "size overflows the int32 index contract";
    case CG_ERR_UNSORTED: return "rows not sorted";
    case CG_ERR_INDEX: return "index out of range";
    case CG_ERR_HIP: return "HIP runtime error";
    case CG_ERR_ALLOC: return "allocation failed";
    case CG_ERR_UNSUPPORTED: return "unsupported arguments";
    case CG_ERR_NO_TRANSPOSE: return "handle has no transpose";
    case CG_ERR_ALIAS: return "output aliases an input";
    default: return "unknown status";
  }
}

const char *cg_last_error(void) { return cg::g_err; }

}  // extern "C"
