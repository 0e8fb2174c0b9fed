/* Plain C restatement of the sparse kernels of CAGNET's per-rank compute path.
 * TEST INFRASTRUCTURE ONLY: used by tests/ as a second, independently written checker next to
 * oracle/gcn_oracle.py (which leans on torch/scipy).  Nothing under cagnet_amd/ links it.
 *
 *   ref_coo2csr_rowptr  cusparseXcoo2csr semantics    sparse-extension/sparse_coo_tensor.cu:136-142
 *   ref_csr_spmm        C = beta*C + A*B, A in CSR    sparse-extension/sparse_coo_tensor.cu:215-226
 *                       (the reference fixes alpha = beta = 1, :149-150)
 *   ref_csr_transpose   counting sort by column (the reference has no transpose; it reuses A,
 *                       gcn_distr.py:326)
 * Sequential loops in index order; the SpMM accumulates each output in double when wide != 0.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* rowptr[i] = first position k with row[k] >= i, for ascending row[]; rowptr[n] = nnz */
int ref_coo2csr_rowptr(const int32_t *row, int64_t nnz, int32_t n, int32_t *rowptr) {
  int64_t k = 0;
  for (int32_t i = 0; i <= n; ++i) {
    while (k < nnz && row[k] < i) ++k;
    rowptr[i] = (int32_t)k;
  }
  return 0;
}

int ref_csr_spmm(const int32_t *rowptr, const int32_t *colind, const float *val, int32_t n, int32_t m,
                 const float *B, int64_t ldb, float *C, int64_t ldc, int32_t f, float beta, int wide) {
  (void)m;
  if (wide) {
    double *acc = (double *)malloc(sizeof(double) * (size_t)f);
    if (!acc) return 1;
    for (int32_t i = 0; i < n; ++i) {
      for (int32_t x = 0; x < f; ++x) acc[x] = 0.0;
      for (int32_t k = rowptr[i]; k < rowptr[i + 1]; ++k) {
        const double a = val[k];
        const float *b = B + (int64_t)colind[k] * ldb;
        for (int32_t x = 0; x < f; ++x) acc[x] += a * (double)b[x];
      }
      float *c = C + (int64_t)i * ldc;
      for (int32_t x = 0; x < f; ++x) c[x] = (float)((beta != 0.f ? (double)beta * (double)c[x] : 0.0) + acc[x]);
    }
    free(acc);
  } else {
    float *acc = (float *)malloc(sizeof(float) * (size_t)f);
    if (!acc) return 1;
    for (int32_t i = 0; i < n; ++i) {
      for (int32_t x = 0; x < f; ++x) acc[x] = 0.f;
      for (int32_t k = rowptr[i]; k < rowptr[i + 1]; ++k) {
        const float a = val[k];
        const float *b = B + (int64_t)colind[k] * ldb;
        for (int32_t x = 0; x < f; ++x) acc[x] += a * b[x];
      }
      float *c = C + (int64_t)i * ldc;
      for (int32_t x = 0; x < f; ++x) c[x] = (beta != 0.f ? beta * c[x] : 0.f) + acc[x];
    }
    free(acc);
  }
  return 0;
}

/* CSR (n x m) -> CSR of the transpose (m x n); perm[k] = CSR position of transposed entry k */
int ref_csr_transpose(const int32_t *rowptr, const int32_t *colind, const float *val, int32_t n, int32_t m,
                      int32_t *colptr, int32_t *rowind, float *val_t, int32_t *perm) {
  const int64_t nnz = rowptr[n];
  int64_t *next = (int64_t *)calloc((size_t)m + 1, sizeof(int64_t));
  if (!next) return 1;
  for (int64_t k = 0; k < nnz; ++k) next[colind[k] + 1]++;
  for (int32_t j = 0; j < m; ++j) next[j + 1] += next[j];
  for (int32_t j = 0; j <= m; ++j) colptr[j] = (int32_t)next[j];
  for (int32_t i = 0; i < n; ++i) {
    for (int32_t k = rowptr[i]; k < rowptr[i + 1]; ++k) {
      const int64_t p = next[colind[k]]++;
      rowind[p] = i;
      if (val && val_t) val_t[p] = val[k];
      if (perm) perm[p] = k;
    }
  }
  free(next);
  return 0;
}
