// Host-sanitizer driver of the C ABI: a plain C++ program linked against the ASan + UBSan build of the
// library's host code (cagnet_amd/build.py --host-sanitize).  Without arguments it walks the argument
// checks and host-only paths, which need no GPU.  With "gpu" it also runs real products on device 0
// through the parts of the host code that hold the most state: handle creation, forced hub and panel
// plans at several widths (plan eviction, schedule recycling), the block cache with eviction, failed plan
// builds, parked tables and scratch release; every product is checked against a loop on the host.
// Exit code 0 and no sanitizer report = pass.
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>
#include <algorithm>
#include <cmath>
#include <vector>
#include "cagnet_amd.h"

static int g_fail = 0;
#define EXPECT(cond)                                                     \
  do {                                                                   \
    if (!(cond)) {                                                       \
      fprintf(stderr, "FAILED %s:%d: %s (last error: %s)\n", __FILE__, __LINE__, #cond, cg_last_error()); \
      ++g_fail;                                                          \
    }                                                                    \
  } while (0)

static void host_only() {
  void *one = (void *)16;  // never dereferenced: validation comes first
  EXPECT(cg_abi_version() == CG_ABI_VERSION);
  for (int code = 0; code <= 11; ++code) EXPECT(strcmp(cg_status_string(code), "unknown status") != 0);
  EXPECT(strcmp(cg_status_string(99), "unknown status") == 0);
  const float *fone = (const float *)one;
  const int32_t *ione = (const int32_t *)one;
  EXPECT(cg_spmm_coo(nullptr, nullptr, nullptr, -1, 4, 4, fone, 4, (float *)32, 4, 4, 1.f, nullptr) == CG_ERR_SIZE);
  EXPECT(cg_spmm_coo(nullptr, nullptr, nullptr, (int64_t)1 << 31, 4, 4, fone, 4, (float *)32, 4, 4, 1.f, nullptr) == CG_ERR_OVERFLOW);
  EXPECT(cg_spmm_coo(nullptr, nullptr, nullptr, 5, 4, 4, fone, 4, (float *)32, 4, 4, 1.f, nullptr) == CG_ERR_NULL);
  EXPECT(cg_spmm_coo(ione, ione, fone, 5, 4, 4, fone, 3, (float *)32, 4, 4, 1.f, nullptr) == CG_ERR_SIZE);
  EXPECT(cg_spmm_coo(ione, ione, fone, 5, 4, 4, fone, 4, (float *)one, 4, 4, 1.f, nullptr) == CG_ERR_ALIAS);
  EXPECT(strstr(cg_last_error(), "alias") != nullptr);
  EXPECT(cg_spmm_coo_cached(nullptr, nullptr, nullptr, -1, 4, 4, fone, 4, (float *)32, 4, 4, 1.f, nullptr) == CG_ERR_SIZE);
  EXPECT(cg_spmm_coo_cached(ione, ione, fone, 5, 4, 4, fone, 3, (float *)32, 4, 4, 1.f, nullptr) == CG_ERR_SIZE);
  EXPECT(cg_coo_cache_info(nullptr) == CG_ERR_NULL);
  int64_t info[12] = {0};
  EXPECT(cg_coo_cache_info(info) == CG_OK);
  EXPECT(cg_coo_cache_clear() == CG_OK);
  cg_csr_t *h = nullptr;
  EXPECT(cg_csr_create(&h, nullptr, nullptr, nullptr, 3, 4, 4, CG_CSR_SORTED, nullptr) == CG_ERR_NULL);
  EXPECT(cg_csr_create(nullptr, ione, ione, fone, 3, 4, 4, CG_CSR_SORTED, nullptr) == CG_ERR_NULL);
  EXPECT(cg_csr_create(&h, ione, ione, fone, ((int64_t)1 << 31) - 1, 4, 4, CG_CSR_SORTED, nullptr) == CG_ERR_OVERFLOW);
  EXPECT(cg_csr_create(&h, ione, ione, fone, 3, 0, 4, CG_CSR_SORTED, nullptr) == CG_ERR_SIZE);
  EXPECT(cg_csr_spmm(nullptr, 0, fone, 4, (float *)32, 4, 4, 0.f, nullptr) == CG_ERR_NULL);
  EXPECT(cg_csr_destroy(nullptr) == CG_OK);
  EXPECT(cg_csr_unpin(nullptr, nullptr) == CG_ERR_NULL);
  EXPECT(cg_csr_info(nullptr, info) == CG_ERR_NULL);
  EXPECT(cg_csr_panel_info(nullptr, 0, info) == CG_ERR_NULL);
  EXPECT(cg_dense_xw(fone, 4, fone, 4, (float *)32, 4, 10, 0, 4, 0, nullptr) == CG_ERR_SIZE);
  EXPECT(cg_dense_gwt(nullptr, 4, fone, 4, (float *)32, 4, 10, 4, 4, nullptr) == CG_ERR_NULL);
  EXPECT(cg_relu_fwd(fone, (float *)32, -1, nullptr) == CG_ERR_SIZE);
  EXPECT(cg_log_softmax_fwd(fone, 3, (float *)32, 4, 10, 4, nullptr) == CG_ERR_SIZE);
  uint8_t junk[256] = {0};
  cg_csr_t *h2 = nullptr;
  EXPECT(cg_csr_blob_read(&h2, junk, 256, 0, nullptr) == CG_ERR_UNSUPPORTED);
  EXPECT(cg_csr_blob_read(&h2, junk, 64, 0, nullptr) == CG_ERR_SIZE);
  EXPECT(cg_csr_blob_read(&h2, nullptr, 256, 0, nullptr) == CG_ERR_NULL);
  EXPECT(cg_tune_set("no_such_knob", 1) == CG_ERR_UNSUPPORTED);
  EXPECT(cg_tune_set(nullptr, 1) == CG_ERR_NULL);
  const char *keys[] = {"spmm_seg", "spmm_win", "spmm_vec", "spmm_hub", "spmm_hub_kb", "spmm_hub_groups", "spmm_hub_tiers",
                        "spmm_hub_row", "spmm_panel", "spmm_panel_emin", "spmm_panel_cols", "spmm_panel_unit", "dense_mfma",
                        "coo_cache_blocks", "coo_cache_mib", "test_alloc_fail"};
  for (const char *k : keys) {
    EXPECT(cg_tune_set(k, 3) == CG_OK);
    EXPECT(cg_tune_set(k, 0) == CG_OK);
  }
  EXPECT(cg_prof_enable(1) == CG_OK);
  double ms = -1.0;
  int64_t launches = -1;
  EXPECT(cg_prof_read("spmm_rowseg/f=16", &ms, &launches) == CG_OK && launches == 0);
  EXPECT(cg_prof_read(nullptr, &ms, &launches) == CG_ERR_NULL);
  EXPECT(cg_prof_enable(0) == CG_OK);
}

// ---- with a GPU --------------------------------------------------------------------------------
#define HIP_OK(call)                                                             \
  do {                                                                           \
    hipError_t e_ = (call);                                                      \
    if (e_ != hipSuccess) {                                                      \
      fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      exit(3);                                                                   \
    }                                                                            \
  } while (0)

struct Lcg {  // small deterministic generator: the driver depends on nothing but libc
  uint64_t s;
  uint32_t next() {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return (uint32_t)(s >> 33);
  }
  float unit() { return (float)(next() & 0xffffff) / (float)0x1000000 - 0.5f; }
};

struct Coo {
  int32_t n, m;
  std::vector<int32_t> row, col;
  std::vector<float> val;
};

// power-law-ish pattern, rows sorted, no duplicates inside a row
static Coo make_coo(int32_t n, int32_t m, int per_row, uint64_t seed) {
  Coo a{n, m, {}, {}, {}};
  Lcg g{seed};
  std::vector<uint8_t> seen((size_t)m);
  for (int32_t r = 0; r < n; ++r) {
    std::fill(seen.begin(), seen.end(), 0);
    const int k = 1 + (int)(g.next() % (uint32_t)(2 * per_row));
    std::vector<int32_t> cols;
    for (int j = 0; j < k; ++j) {
      uint32_t c = g.next() % (uint32_t)m;
      if (g.next() & 1) c = c % (uint32_t)(m / 16 + 1);  // popular columns
      if (!seen[c]) {
        seen[c] = 1;
        cols.push_back((int32_t)c);
      }
    }
    std::sort(cols.begin(), cols.end());
    for (int32_t c : cols) {
      a.row.push_back(r);
      a.col.push_back(c);
      a.val.push_back(g.unit());
    }
  }
  return a;
}

template <typename T>
static T *to_device(const std::vector<T> &v) {
  T *d = nullptr;
  HIP_OK(hipMalloc((void **)&d, v.size() * sizeof(T) + 16));
  HIP_OK(hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return d;
}

static double product_error(const Coo &a, const std::vector<float> &B, int f, const std::vector<float> &C) {
  std::vector<double> ref((size_t)a.n * f, 0.0), mag((size_t)a.n * f, 0.0);
  for (size_t k = 0; k < a.row.size(); ++k)
    for (int j = 0; j < f; ++j) {
      const double t = (double)a.val[k] * (double)B[(size_t)a.col[k] * f + j];
      ref[(size_t)a.row[k] * f + j] += t;
      mag[(size_t)a.row[k] * f + j] += std::fabs(t);
    }
  double worst = 0.0;
  for (size_t i = 0; i < ref.size(); ++i) {
    const double e = std::fabs((double)C[i] - ref[i]) / (mag[i] > 1e-30 ? mag[i] : 1e-30);
    if (mag[i] > 0 && e > worst) worst = e;
    if (mag[i] == 0 && C[i] != 0.f) worst = 1.0;
  }
  return worst;
}

static void with_gpu() {
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count < 1) {
    fprintf(stderr, "no GPU visible\n");
    exit(4);
  }
  HIP_OK(hipSetDevice(0));
  hipStream_t stream = nullptr;
  HIP_OK(hipStreamCreate(&stream));
  const int32_t n = 1500, m = 1300;
  Coo a = make_coo(n, m, 40, 7);
  const int64_t nnz = (int64_t)a.row.size();
  int32_t *d_row = to_device(a.row), *d_col = to_device(a.col);
  float *d_val = to_device(a.val);
  const int widths[] = {16, 41, 258, 300, 384, 602, 636};
  cg_csr_t *h = nullptr;
  EXPECT(cg_csr_create(&h, d_row, d_col, d_val, nnz, n, m, CG_CSR_SORTED | CG_CSR_TRANSPOSE | CG_CSR_VALIDATE, stream) == CG_OK);
  int64_t info[12] = {0};
  EXPECT(cg_csr_info(h, info) == CG_OK && info[0] == n && info[1] == m && info[2] == nnz);
  for (int pass = 0; pass < 4; ++pass) {
    // pass 0: built-in choices; 1: hub plans forced (7 widths through 2 plan slots and 4 schedule slots);
    // 2: panel plans forced as well, with small tiles; 3: with dense tiles from 48 entries on, three workgroups
    EXPECT(cg_tune_set("spmm_hub", pass >= 1 ? 1 : 0) == CG_OK);
    EXPECT(cg_tune_set("spmm_hub_kb", pass >= 1 ? 64 : 0) == CG_OK);
    EXPECT(cg_tune_set("spmm_panel", pass >= 2 ? 1 : 0) == CG_OK);
    EXPECT(cg_tune_set("spmm_panel_emin", pass >= 2 ? 8 : 0) == CG_OK);
    EXPECT(cg_tune_set("spmm_panel_dmin", pass == 3 ? 48 : 0) == CG_OK);
    EXPECT(cg_tune_set("spmm_panel_dwg", pass == 3 ? 3 : 0) == CG_OK);
    EXPECT(cg_tune_set("spmm_panel_narrow", pass == 3 ? 1 : 0) == CG_OK);  // the narrow widths take dense tiles too
    EXPECT(cg_tune_set("spmm_panel_narrow_dmin", pass == 3 ? 48 : 0) == CG_OK);
    for (int f : widths) {
      Lcg g{(uint64_t)f * 31 + pass};
      std::vector<float> B((size_t)m * f), C((size_t)n * f, 0.f);
      for (float &x : B) x = g.unit();
      float *d_B = to_device(B), *d_C = to_device(C);
      EXPECT(cg_csr_spmm(h, 0, d_B, f, d_C, f, f, 0.f, stream) == CG_OK);
      HIP_OK(hipStreamSynchronize(stream));
      HIP_OK(hipMemcpy(C.data(), d_C, C.size() * sizeof(float), hipMemcpyDeviceToHost));
      const double err = product_error(a, B, f, C);
      if (!(err <= 1e-5)) {
        fprintf(stderr, "pass %d f %d: relative error %.3e\n", pass, f, err);
        ++g_fail;
      }
      EXPECT(cg_csr_panel_info(h, 0, info) == CG_OK);
      if (pass == 3 && f >= 258) EXPECT(info[0] == 1 && info[9] > 0 && info[1] + info[8] + info[5] == nnz);
      if (pass == 3 && f <= 64) {
        EXPECT(cg_csr_panel_info(h, 2, info) == CG_OK);
        EXPECT(info[0] == 1 && info[9] > 0 && info[1] == 0 && info[8] + info[5] == nnz);
      }
      HIP_OK(hipFree(d_B));
      HIP_OK(hipFree(d_C));
    }
  }
  // a plan build that runs out of memory: the product still succeeds, on the plain schedule
  {
    const int f = 320;
    std::vector<float> B((size_t)m * f, 0.25f), C((size_t)n * f, 0.f);
    float *d_B = to_device(B), *d_C = to_device(C);
    EXPECT(cg_tune_set("spmm_panel", 0) == CG_OK);
    EXPECT(cg_tune_set("test_alloc_fail", 3) == CG_OK);
    EXPECT(cg_csr_spmm(h, 0, d_B, f, d_C, f, f, 0.f, stream) == CG_OK);
    EXPECT(cg_tune_set("test_alloc_fail", 0) == CG_OK);
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(C.data(), d_C, C.size() * sizeof(float), hipMemcpyDeviceToHost));
    EXPECT(product_error(a, B, f, C) <= 1e-5);
    HIP_OK(hipFree(d_B));
    HIP_OK(hipFree(d_C));
  }
  // block cache: three blocks through two slots, hits and evictions, then clear
  {
    EXPECT(cg_tune_set("coo_cache_blocks", 2) == CG_OK);
    EXPECT(cg_coo_cache_clear() == CG_OK);
    const int f = 128;
    std::vector<float> B((size_t)m * f), C((size_t)n * f);
    Lcg g{99};
    for (float &x : B) x = g.unit();
    float *d_B = to_device(B), *d_C = to_device(C);
    std::vector<float *> vals;
    for (int k = 0; k < 3; ++k) {
      std::vector<float> v = a.val;
      v[(size_t)k] += 1.f;
      vals.push_back(to_device(v));
    }
    const int order[] = {0, 1, 0, 2, 1, 0};
    for (int k : order) {
      EXPECT(cg_spmm_coo_cached(d_row, d_col, vals[(size_t)k], nnz, n, m, d_B, f, d_C, f, f, 0.f, stream) == CG_OK);
      HIP_OK(hipStreamSynchronize(stream));
      HIP_OK(hipMemcpy(C.data(), d_C, C.size() * sizeof(float), hipMemcpyDeviceToHost));
      Coo ak = a;
      ak.val[(size_t)k] += 1.f;
      EXPECT(product_error(ak, B, f, C) <= 1e-5);
    }
    EXPECT(cg_coo_cache_info(info) == CG_OK && info[0] == 2 && info[3] >= 2);
    EXPECT(cg_coo_cache_clear() == CG_OK);
    EXPECT(cg_tune_set("coo_cache_blocks", 0) == CG_OK);
    for (float *p : vals) HIP_OK(hipFree(p));
    HIP_OK(hipFree(d_B));
    HIP_OK(hipFree(d_C));
  }
  for (const char *k : {"spmm_hub", "spmm_hub_kb", "spmm_panel", "spmm_panel_emin", "spmm_panel_dmin", "spmm_panel_dwg",
                        "spmm_panel_narrow", "spmm_panel_narrow_dmin"})
    EXPECT(cg_tune_set(k, 0) == CG_OK);
  int64_t released = -1;
  EXPECT(cg_csr_unpin(h, &released) == CG_OK && released == 0);  // nothing was captured: nothing was parked
  EXPECT(cg_csr_destroy(h) == CG_OK);
  EXPECT(cg_scratch_release(stream, &released) == CG_OK && released > 0);
  HIP_OK(hipFree(d_row));
  HIP_OK(hipFree(d_col));
  HIP_OK(hipFree(d_val));
  HIP_OK(hipStreamDestroy(stream));
}

int main(int argc, char **argv) {
  host_only();
  if (argc > 1 && !strcmp(argv[1], "gpu")) with_gpu();
  if (g_fail) {
    fprintf(stderr, "%d check(s) failed\n", g_fail);
    return 1;
  }
  printf("abi_host_driver: ok\n");
  // Leave without running exit handlers: the HIP runtime's own teardown frees, after its device layer is
  // gone, memory that the sanitizer's allocator tracks as device memory, which the sanitizer aborts on.
  fflush(stdout);
  fflush(stderr);
  _exit(0);
}
