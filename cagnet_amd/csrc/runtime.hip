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
  bool pinned = false;  // handed out while its stream was being captured: a graph may name it
};

static std::mutex g_scratch_mu;
static std::map<std::tuple<int, hipStream_t, int>, ScratchBuf> g_scratch;
static std::map<std::pair<int, hipStream_t>, std::vector<ScratchBuf>> g_scratch_parked;

bool stream_capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st == hipStreamCaptureStatusActive;
}

int refuse_under_capture(hipStream_t stream, const char *what) {
  if (stream_capturing(stream))
    CG_FAIL(CG_ERR_CAPTURE, "%s cannot run while its stream is being captured: run the same call once before the capture",
            what);
  return CG_OK;
}

static thread_local std::vector<void *> *g_park_sink = nullptr;

void table_free(void *p) {
  if (!p) return;
  if (g_park_sink)
    g_park_sink->push_back(p);
  else
    (void)hipFree(p);
}

ParkScope::ParkScope(void *sink_vector) : prev(g_park_sink), set(sink_vector != nullptr) {
  if (set) g_park_sink = static_cast<std::vector<void *> *>(sink_vector);
}
ParkScope::~ParkScope() {
  if (set) g_park_sink = static_cast<std::vector<void *> *>(prev);
}

// Grow-only.  Growing frees the old buffer after the stream has drained, so work already enqueued on
// `stream` that still reads it stays valid; a buffer that was handed out under capture is parked
// instead (a graph replays with its address) until scratch_release.
int scratch_get(hipStream_t stream, int slot, size_t bytes, void **out) {
  int dev = 0;
  CG_HIP(hipGetDevice(&dev));
  const bool capturing = stream_capturing(stream);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  ScratchBuf &b = g_scratch[std::make_tuple(dev, stream, slot)];
  if (bytes > b.bytes) {
    if (capturing)
      CG_FAIL(CG_ERR_CAPTURE,
              "scratch slot %d would grow from %zu to %zu bytes while its stream is being captured: run the same call "
              "once before the capture",
              slot, b.bytes, bytes);
    if (b.ptr) {
      if (b.pinned) {
        g_scratch_parked[std::make_pair(dev, stream)].push_back(b);
      } else {
        CG_HIP(hipStreamSynchronize(stream));
        CG_HIP(hipFree(b.ptr));
      }
      b = ScratchBuf();
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
  if (capturing) b.pinned = true;
  *out = b.ptr;
  return CG_OK;
}

int scratch_release(hipStream_t stream, int64_t *released_bytes) {
  int dev = 0;
  CG_HIP(hipGetDevice(&dev));
  CG_TRY(refuse_under_capture(stream, "cg_scratch_release"));
  CG_HIP(hipStreamSynchronize(stream));
  int64_t total = 0;
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  for (int slot = 0; slot < kNumSlots; ++slot) {
    auto it = g_scratch.find(std::make_tuple(dev, stream, slot));
    if (it == g_scratch.end()) continue;
    if (it->second.ptr) (void)hipFree(it->second.ptr);
    total += (int64_t)it->second.bytes;
    g_scratch.erase(it);
  }
  auto pit = g_scratch_parked.find(std::make_pair(dev, stream));
  if (pit != g_scratch_parked.end()) {
    for (ScratchBuf &b : pit->second) {
      if (b.ptr) (void)hipFree(b.ptr);
      total += (int64_t)b.bytes;
    }
    g_scratch_parked.erase(pit);
  }
  if (released_bytes) *released_bytes = total;
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

int cg_scratch_release(cg_stream_t stream, int64_t *released_bytes) {
  return cg::scratch_release((hipStream_t)stream, released_bytes);
}

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
    case CG_ERR_CAPTURE: return "not possible while the stream is being captured";
    default: return "unknown status";
  }
}

const char *cg_last_error(void) { return cg::g_err; }

}  // extern "C"
