/*
 * cagnet_amd.h -- C ABI of libcagnet_amd.so: the per-rank GCN compute path of
 * CAGNET (local coo2csr + accumulate-SpMM + H*W + ReLU / log_softmax+NLL,
 * forward and backward) as hand-written gfx950 HIP kernels.
 *
 * Conventions
 *   - Every pointer named d_* or documented "device" is a device pointer on the
 *     current HIP device.  Dense matrices are fp32 row-major with an explicit
 *     leading dimension in ELEMENTS (ld >= number of columns).  Sparse indices
 *     are int32 (the reference's contract); dense offsets are 64-bit inside.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  All
 *     work is enqueued on it; no entry point synchronises the device unless its
 *     comment says so.
 *   - Every entry point returns a cg_status (0 = success).  cg_last_error()
 *     returns a thread-local human-readable detail for the last failure.
 *     (The reference prints cuSPARSE/CUDA errors and continues,
 *     sparse-extension/sparse_coo_tensor.cu:20-30; a status code is strictly
 *     stronger and needs no change at the call sites.)
 *   - Summation orders are fixed by the schedule (no floating-point atomics):
 *     two calls with the same arguments give bit-identical results.
 *   - Library scratch memory is kept per (device, stream); calls that share a
 *     stream are ordered by it.  Calls on different streams use different
 *     scratch and may overlap.  A cg_csr_t handle is used by one host thread
 *     at a time (its schedule and plan caches are not re-entrant).
 *   - Stream capture (hipStreamBeginCapture): cg_csr_spmm, cg_csr_spmm_xw,
 *     cg_spmm_coo, the dense and the elementwise entry points may be captured
 *     once the same call has run eagerly on that stream (the first call of a
 *     shape builds tables and grows scratch, which a capture cannot hold; such
 *     a step returns CG_ERR_CAPTURE and leaves the capture usable for nothing).
 *     A captured graph keeps the addresses of the scratch buffers and handle
 *     tables its calls used.  The library therefore never frees those while
 *     the handle lives: a scratch buffer handed out under capture, and every
 *     table of a handle that ran a product under capture, is parked instead of
 *     freed when a later call has to replace it (growth, plan eviction, new
 *     tuning values).  cg_csr_unpin / cg_csr_destroy and cg_scratch_release
 *     free parked memory; call them only when no graph that used the handle or
 *     the stream will be replayed again.
 */
#ifndef CAGNET_AMD_H
#define CAGNET_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CG_ABI_VERSION 1

typedef void *cg_stream_t;       /* hipStream_t */
typedef struct cg_csr cg_csr_t;  /* opaque: device-resident CSR (+ optional transpose) and its schedules */

enum cg_status {
  CG_OK = 0,
  CG_ERR_NULL = 1,         /* a required pointer is NULL */
  CG_ERR_SIZE = 2,         /* negative size, ld < columns, f <= 0, ... */
  CG_ERR_OVERFLOW = 3,     /* nnz >= 2^31, n + 1 overflows int32, ... */
  CG_ERR_UNSORTED = 4,     /* validation: rows not ascending on the sorted path */
  CG_ERR_INDEX = 5,        /* validation: row >= n or col >= m or negative index */
  CG_ERR_HIP = 6,          /* a HIP runtime call failed (detail in cg_last_error) */
  CG_ERR_ALLOC = 7,        /* device or host allocation failed */
  CG_ERR_UNSUPPORTED = 8,  /* argument combination not implemented */
  CG_ERR_NO_TRANSPOSE = 9, /* transpose product asked of a handle built without CG_CSR_TRANSPOSE */
  CG_ERR_ALIAS = 10,       /* output aliases an input where that is not allowed */
  CG_ERR_CAPTURE = 11      /* the call would allocate, build tables or read back while its stream is being captured */
};

/* flags of cg_csr_create */
#define CG_CSR_SORTED 1u    /* trust: input is sorted by (row, col) (torch .coalesce() order) */
#define CG_CSR_TRANSPOSE 2u /* also build the transpose (CSC of A = CSR of A^T) for A^T * G */
#define CG_CSR_VALIDATE 4u  /* check index ranges (and sortedness if CG_CSR_SORTED); synchronises */

int cg_abi_version(void);
const char *cg_status_string(int status);
const char *cg_last_error(void);
/* Frees the library's scratch buffers of (current device, stream), including buffers parked because a
 * captured graph used them (see Conventions), after synchronising the stream; the next call on the
 * stream allocates afresh.  *released_bytes is nullable.  CG_ERR_CAPTURE while the stream is capturing.
 * No counterpart in the reference (torch's caching allocator owns cuSPARSE's workspace there). */
int cg_scratch_release(cg_stream_t stream, int64_t *released_bytes);

/* ------------------------------------------------------------------------------------------
 * coo2csr.  Replaces the cusparseXcoo2csr step that the reference runs inside every spmm_gpu
 * call (sparse-extension/sparse_coo_tensor.cu:136-142): compress ascending int32 row indices
 * into rowptr[n+1], base 0.  rowptr[i] = #{k : row[k] < i}.  d_row must be ascending; indices
 * outside [0, n) are clamped into the table instead of faulting.  nnz == 0 is legal.
 */
int cg_coo2csr_rowptr(const int32_t *d_row, int64_t nnz, int32_t n, int32_t *d_rowptr, cg_stream_t stream);

/* Validating companion (debug mode of the same boundary: the reference never checks its
 * inputs, sparse_coo_tensor.cu:113-142).  Synchronises `stream`.  Returns CG_ERR_INDEX if any
 * row is outside [0,n) or col outside [0,m); CG_ERR_UNSORTED if require_sorted and rows
 * descend somewhere (or cols do not strictly ascend inside a row when require_sorted == 2). */
int cg_coo_check(const int32_t *d_row, const int32_t *d_col, int64_t nnz, int32_t n, int32_t m,
                 int require_sorted, cg_stream_t stream);

/* General COO -> CSR for input in ANY order: stable LSD radix sort of (row, col) keys in LDS,
 * then the row compression above.  Duplicates are kept (not summed), in input order.  Outputs:
 * d_rowptr[n+1], d_colind[nnz], d_values[nnz] (may be NULL when d_val is NULL) and, when
 * d_perm != NULL, d_perm[k] = input position of output entry k.  Result order equals
 * scipy.sparse.coo_matrix(...).tocsr() with sorted indices / torch .coalesce() on
 * duplicate-free input (what the reference's callers feed spmm_gpu: gcn_distr.py:546).
 * d_colind may be d_col and d_values may be d_val (conversion in place; the inputs are otherwise
 * left untouched); with d_perm the values are gathered by it, so d_values must then differ from d_val.
 * Allocates temporaries and synchronises `stream` before returning. */
int cg_coo2csr(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n, int32_t m,
               int32_t *d_rowptr, int32_t *d_colind, float *d_values, int32_t *d_perm, cg_stream_t stream);

/* CSR of A (n x m) -> CSR of A^T (m x n) == CSC of A: the precomputed operand of the A^T*G
 * backward product (the reference reuses A itself and so assumes symmetry, gcn_distr.py:326,
 * gcn_distr_2d.py:683).  Stable radix sort by column, so rows ascend inside each column.
 * d_perm (nullable): d_perm[k] = CSR position of transposed entry k.  d_rowind may be d_colind
 * and, without d_perm, d_values_t may be d_values.  Allocates temporaries and synchronises `stream`. */
int cg_csr_transpose(const int32_t *d_rowptr, const int32_t *d_colind, const float *d_values, int64_t nnz,
                     int32_t n, int32_t m, int32_t *d_colptr, int32_t *d_rowind, float *d_values_t,
                     int32_t *d_perm, cg_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * spmm_gpu, one shot.  Same operands and meaning as the reference operator
 *   spmm_gpu(A_rowindices, A_colindices, A_values, n, m, B, C)
 * (sparse-extension/sparse_coo_tensor.cu:113-240, called at gcn_distr.py:238-240):
 * C[n,f] = beta*C + A[n,m] * B[m,f] with A as row-sorted COO; the reference fixes beta = 1
 * (sparse_coo_tensor.cu:149-150).  Like the reference it rebuilds everything from the COO arrays
 * on every call (row compression, row-segment schedule), but as device work on `stream`: no
 * allocation after the scratch has grown to size, no device synchronisation.  B and C stay
 * row-major and keep their storage (the reference transposes both and replaces their storage,
 * :166-168,:183-185,:234-239).  Rows must ascend; input that violates this gives wrong sums, as it
 * does in the reference, but never an access outside the operands (indices are clamped).
 */
int cg_spmm_coo(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n, int32_t m,
                const float *d_B, int64_t ldb, float *d_C, int64_t ldc, int32_t f, float beta, cg_stream_t stream);

/* Same product and checks as cg_spmm_coo, for the way the reference's callers use spmm_gpu: the same
 * block at every stage of every epoch, through fresh `.indices()[k].int()` temporaries
 * (gcn_distr.py:238-240), so neither addresses nor tensor identities tell whether a block was seen
 * before.  Products that cg_csr_spmm would run with a column-popularity plan (wide, over a dense
 * power-law block: the plan is far too costly to build per call) are handled here; every other
 * product is passed to cg_spmm_coo, which rebuilds its plain schedule for less than a digest costs.
 * A handled call computes a 128-bit digest of (row, col, val) on the device (one pass over
 * 12 nnz bytes) and reads it back, which synchronises `stream` once; a block whose digest, nnz, n
 * and m were seen before on this device reuses the handle built at its first sighting (a private
 * copy of the arrays as CSR, the schedules and the column-popularity plans of cg_csr_spmm), and the
 * result is bit-identical to cg_csr_spmm on such a handle.  A first sighting builds the handle
 * as cg_csr_create(CG_CSR_SORTED) does: index ranges and row order are checked and reported
 * (CG_ERR_INDEX, CG_ERR_UNSORTED).  Two different blocks with equal digests (probability about
 * 2^-128 per pair) would be taken for one another.  The least recently used block is dropped
 * beyond cg_tune_set("coo_cache_blocks", k) blocks (default 8; negative: keep none and behave as
 * cg_spmm_coo) or beyond "coo_cache_mib" MiB of kept device memory (default 32 GiB).
 * Input that is not row-sorted or out of range is therefore reported on this path only; the products
 * passed on to cg_spmm_coo have that entry point's precondition (see there) and report nothing.
 * A caller whose values change on every call pays the digest, the handle and the plan build (about
 * 40 ms at 114.6 M entries) each time and should call cg_spmm_coo instead.
 * May be called from several host threads at once, also on different streams (the table of blocks is
 * locked, products on one block are serialised); cannot be captured into a HIP graph (CG_ERR_CAPTURE:
 * it reads the digest back). */
int cg_spmm_coo_cached(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t n,
                       int32_t m, const float *d_B, int64_t ldb, float *d_C, int64_t ldc, int32_t f, float beta,
                       cg_stream_t stream);
/* Drops every block cg_spmm_coo_cached keeps (device memory is freed once queued products finish). */
int cg_coo_cache_clear(void);
/* info = {blocks kept, hits, misses, evictions} since the library was loaded. */
int cg_coo_cache_info(int64_t info[4]);

/* ------------------------------------------------------------------------------------------
 * Cached handle: what the reference rebuilds on every call (index casts gcn_distr.py:238,
 * coo2csr, workspace malloc/free, sparse_coo_tensor.cu:136-231) is built once here.
 * cg_csr_create copies the operands (the caller may free its arrays afterwards), builds the CSR,
 * the transpose if asked, and synchronises `stream`.
 */
int cg_csr_create(cg_csr_t **out, const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz,
                  int32_t n, int32_t m, uint32_t flags, cg_stream_t stream);
int cg_csr_destroy(cg_csr_t *h);
/* [A_0 | A_1 | ... | A_{count-1}] as one handle: the blocks of one block row of a partitioned matrix (equal row
 * counts; at most 16), side by side in the order given, block k's columns behind those of the blocks before it.
 * One product of the new handle with the dense blocks H_k stacked in the same order (rows of H_0, then of H_1, ...)
 * is the whole stage loop z = sum_k A_k H_k that the reference runs as one spmm_gpu call per stage
 * (gcn_distr.py:221-244, gcn_distr_2d.py:333-417): Z is written once instead of once per stage.  The entries are
 * copied (the blocks stay as they are and may be destroyed afterwards); CG_CSR_TRANSPOSE in `flags` also builds
 * the transpose of the stacked matrix.  Synchronises `stream`. */
int cg_csr_hstack(cg_csr_t **out, cg_csr_t *const *blocks, int32_t count, uint32_t flags, cg_stream_t stream);
/* Frees the tables parked on a handle since one of its products was captured into a HIP graph (see
 * Conventions) and lets later replacements free at once again.  Synchronises the device.  *released
 * (nullable) receives the number of device allocations freed.  Only for callers that have dropped every
 * graph captured over this handle.  No counterpart in the reference, which captures no graphs. */
int cg_csr_unpin(cg_csr_t *h, int64_t *released);

/* C[rows,f] = beta*C + op(A) * B, op(A) = A (transpose == 0: rows = n, B is m x f) or A^T
 * (transpose != 0: rows = m, B is n x f).  The first call for a given width class builds its
 * schedule (row segments, windows of tasks; for wide products over dense power-law matrices a
 * plan that regroups the entries by column popularity) and synchronises once; later calls are
 * stream ordered.  Results are bit-identical from call to call.  Scratch memory is kept per
 * (device, stream); a handle may be used from one host thread at a time. */
int cg_csr_spmm(cg_csr_t *h, int transpose, const float *d_B, int64_t ldb, float *d_C, int64_t ldc, int32_t f,
                float beta, cg_stream_t stream);

/* Fused layer product Z[rows,fo] = act((beta*C + op(A) * B) * W): the two steps of GCNFunc.forward,
 * z = spmm(A, H) then torch.mm(z, weight) (gcn_distr.py:271-275), without writing the rows x f
 * intermediate; relu != 0 applies max(., 0) (gcn_distr.py:284-288).  C is an input here (the sum of
 * earlier stages, read when beta != 0, never written; NULL with beta == 0).  W is f x fo, fo <= 64.
 * Returns CG_ERR_UNSUPPORTED, before any work, for widths that have no fused form (f below 128 or
 * so, f * fo beyond the LDS budget): the caller then runs cg_csr_spmm and cg_dense_xw. */
int cg_csr_spmm_xw(cg_csr_t *h, int transpose, const float *d_B, int64_t ldb, const float *d_C, int64_t ldc, float beta,
                   const float *d_W, int64_t ldw, float *d_Z, int64_t ldz, int32_t f, int32_t fo, int relu,
                   cg_stream_t stream);

/* info[0..7] = { n, m, nnz, has_transpose, max row degree, max column degree (or -1),
 *                column-popularity plan last looked up by a wide product of A, of A^T:
 *                tiers in use, -1 when the column counts declined it, 0 when none was considered } */
int cg_csr_info(const cg_csr_t *h, int64_t info[8]);
/* Panel plan a wide product of A (bit 0 of `transpose` set: of A^T) last looked up; with bit 1 of `transpose` set the
 * plan of the narrow products (f <= 64), which has dense tiles only; with bits 2..3 holding 1, 2 or 3 the tile plan
 * with panels of 256, 512 or 1024 rows: info[0..11] =
 * { 1 in use / -1 declined (the tiles hold too few of the entries) / 0 none considered yet,
 *   entries multiplied out of LDS by the vector ALUs, their (active) tiles, their units (workgroups),
 *   row panels with several units of either kind, entries left to the row-wise kernels, entries a tile
 *   needs, column ranks per panel, entries in dense tiles (multiplied on the fp32 matrix cores), dense tiles, their
 *   units, entries from which a tile is dense (0: no dense tiles were allowed) }.  No counterpart in the
 * reference, which hands the whole product to cusparseSpMM (sparse-extension/sparse_coo_tensor.cu:215-226). */
int cg_csr_panel_info(const cg_csr_t *h, int transpose, int64_t info[12]);
/* Device pointers of the arrays the handle owns (transpose != 0: those of A^T). */
int cg_csr_arrays(const cg_csr_t *h, int transpose, const int32_t **d_rowptr, const int32_t **d_colind,
                  const float **d_values);

/* ------------------------------------------------------------------------------------------
 * Dense products of GCNFunc (torch.mm at gcn_distr.py:275, :330, :187).
 *   cg_dense_xw : Z[n,fo]  = X[n,k] * W[k,fo]           (optionally fused ReLU: relu != 0)
 *   cg_dense_gwt: dX[n,k]  = G[n,fo] * W[k,fo]^T
 *   cg_dense_xtg: dW[k,fo] = X[n,k]^T * G[n,fo]         (split over n, fixed-order second pass)
 */
int cg_dense_xw(const float *d_X, int64_t ldx, const float *d_W, int64_t ldw, float *d_Z, int64_t ldz, int64_t n,
                int32_t k, int32_t fo, int relu, cg_stream_t stream);
int cg_dense_gwt(const float *d_G, int64_t ldg, const float *d_W, int64_t ldw, float *d_dX, int64_t lddx,
                 int64_t n, int32_t k, int32_t fo, cg_stream_t stream);
int cg_dense_xtg(const float *d_X, int64_t ldx, const float *d_G, int64_t ldg, float *d_dW, int64_t lddw,
                 int64_t n, int32_t k, int32_t fo, cg_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Activations and loss of GCNFunc / train (gcn_distr.py:284-294, :312-322, :349-362).
 *   relu_fwd        : h = max(z, 0)
 *   relu_bwd        : dz = g * [h > 0]   (h is the ReLU OUTPUT; [h > 0] == [z > 0])
 *   log_softmax_fwd : out[i,:] = z[i,:] - logsumexp(z[i,:])
 *   log_softmax_bwd : dz[i,:] = g[i,:] - exp(out[i,:]) * sum_c g[i,c]
 *   nll_loss_fwd    : *d_loss = -(1/|mask|) * sum_{i in mask} logp[i, y_i]; |mask| == 0 gives 0
 *                     (the reference's fake_loss branch, gcn_distr.py:359-362)
 *   nll_loss_bwd    : dlogp[i,c] = -gscale * mask_i / |mask| * [c == y_i]   (zero elsewhere)
 *   log_softmax_nll_bwd : fused dz = gscale * mask_i/|mask| * (exp(logp[i,c]) - [c == y_i])
 *   log_softmax_nll_fwd : log_softmax_fwd and nll_loss_fwd in one pass over z (the reference's
 *                         train ends in exactly this pair, gcn_distr.py:344 and :356); the loss is
 *                         the same float nll_loss_fwd returns for the log-probabilities written
 * y is int64 (torch labels); mask is one byte per row (torch.bool / uint8), NULL = all rows.
 * In these formulas "mask" means the rows that are in the mask AND carry a label in [0, c): a row with any
 * other label (torch's ignore_index = -100 among them) adds nothing to the sum, does not count in |mask|
 * and gets a zero gradient, which is what F.nll_loss does with ignore_index rows (for other labels outside
 * the range torch raises; here they are ignored the same way).  d_count receives |mask| as int64
 * (device).  Both reductions run in a fixed order.
 */
int cg_relu_fwd(const float *d_z, float *d_h, int64_t count, cg_stream_t stream);
int cg_relu_bwd(const float *d_g, const float *d_h, float *d_dz, int64_t count, cg_stream_t stream);
int cg_log_softmax_fwd(const float *d_z, int64_t ldz, float *d_out, int64_t ldo, int64_t n, int32_t c,
                       cg_stream_t stream);
int cg_log_softmax_bwd(const float *d_g, int64_t ldg, const float *d_out, int64_t ldo, float *d_dz, int64_t lddz,
                       int64_t n, int32_t c, cg_stream_t stream);
int cg_nll_loss_fwd(const float *d_logp, int64_t ld, const int64_t *d_y, const uint8_t *d_mask, int64_t n,
                    int32_t c, float *d_loss, int64_t *d_count, cg_stream_t stream);
/* cg_nll_loss_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same
 * kernels, same order of additions and therefore the same float as cg_nll_loss_fwd, but the
 * per-workgroup partial sums live in a device array that is part of the library image (about 768 KiB
 * on every GPU the library runs on, held until the process ends) instead of the grow-only scratch:
 * the call allocates and frees nothing.  n may be at most 16,777,216 rows (CG_ERR_SIZE beyond).
 * The first call on a device looks the array's address up (once; make that call outside a capture).
 * All calls on one GPU share the array: calls that overlap on one GPU, on any streams, race. */
int cg_nll_loss_fwd_static(const float *d_logp, int64_t ld, const int64_t *d_y, const uint8_t *d_mask, int64_t n,
                           int32_t c, float *d_loss, int64_t *d_count, cg_stream_t stream);
int cg_nll_loss_bwd(const int64_t *d_y, const uint8_t *d_mask, const int64_t *d_count, const float *d_gscale,
                    float *d_dlogp, int64_t ld, int64_t n, int32_t c, cg_stream_t stream);
int cg_log_softmax_nll_bwd(const float *d_logp, int64_t ld, const int64_t *d_y, const uint8_t *d_mask,
                           const int64_t *d_count, const float *d_gscale, float *d_dz, int64_t lddz, int64_t n,
                           int32_t c, cg_stream_t stream);
int cg_log_softmax_nll_fwd(const float *d_z, int64_t ldz, const int64_t *d_y, const uint8_t *d_mask, float *d_out,
                           int64_t ldo, int64_t n, int32_t c, float *d_loss, int64_t *d_count, cg_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * A sparse block as one byte string in host memory, for files and for transfers between ranks.
 * The reference loads its adjacency matrix from a pickled int64 COO tensor (gcn_distr.py:747)
 * and sends blocks as three float32 arrays, indices included (gcn_distr_2d.py:369-374), which is
 * lossy above 2^24.  The blob holds a 128-byte header (magic "CGNTCSR", version 1, flags, n, m,
 * nnz, array offsets, total size, FNV-1a checksum of the payload) followed by int32 rowptr[n+1],
 * int32 colind[nnz] and float values[nnz], each on a 64-byte boundary, little endian.
 *
 * cg_csr_blob_size: bytes a handle needs.  cg_csr_blob_write: fills host_buf (>= that size).
 * cg_csr_blob_read: checks magic, version, sizes, offsets, checksum, rowptr monotonicity and the
 * column range, then builds a handle; the transpose is rebuilt when the writer's handle had one
 * or when `flags` holds CG_CSR_TRANSPOSE.  A malformed blob is rejected with CG_ERR_UNSUPPORTED
 * (magic, version), CG_ERR_SIZE (truncated, inconsistent offsets), CG_ERR_INDEX (checksum, column
 * range, rowptr ends) or CG_ERR_UNSORTED.  All three synchronise `stream`. */
int cg_csr_blob_size(const cg_csr_t *h, int64_t *bytes);
int cg_csr_blob_write(const cg_csr_t *h, void *host_buf, int64_t capacity, cg_stream_t stream);
int cg_csr_blob_read(cg_csr_t **out, const void *host_buf, int64_t bytes, uint32_t flags, cg_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Input preparation on the device.  The reference prepares its adjacency matrix on the host:
 * add_remaining_self_loops (gcn_distr.py:791), scale_elements (gcn_distr.py:412-470) and
 * split_coo (gcn_distr.py:398-409).  These three entry points do the same work on int32 COO
 * arrays that are already in device memory.  Temporaries come from the scratch memory the library
 * keeps per (device, stream).  cg_add_self_loops and cg_coo_block return a count, so they
 * synchronise `stream`; cg_gcn_normalize is stream ordered and does not.
 *
 * cg_add_self_loops: (row, col) strictly ascending COO of an n x n pattern -> the same pattern
 * with every diagonal entry present exactly once, still ascending.  *out_nnz receives the size of
 * the result; with both outputs NULL the call only counts.  CG_ERR_SIZE if capacity is too small,
 * CG_ERR_UNSORTED / CG_ERR_INDEX for input that is not strictly ascending or out of range. */
int cg_add_self_loops(const int32_t *d_row, const int32_t *d_col, int64_t nnz, int32_t n, int32_t *d_out_row,
                      int32_t *d_out_col, int64_t capacity, int64_t *out_nnz, cg_stream_t stream);

/* cg_gcn_normalize: values of D^-1/2 A D^-1/2 for a pattern that already holds its self-loops, in
 * the arithmetic of scale_elements: deg_i = stored entries of row i, dinv_i = fl32(deg_i^-1/2)
 * with the power in fp64 (gcn_distr.py:440-448), val = fl32(dinv_row * fl32(1 * dinv_col))
 * (gcn_distr.py:458-464).  Any entry order.  d_dinv (nullable, n floats) receives dinv. */
int cg_gcn_normalize(const int32_t *d_row, const int32_t *d_col, int64_t nnz, int32_t n, float *d_val,
                     float *d_dinv, cg_stream_t stream);

/* cg_coo_block: the entries with r0 <= row < r1 and c0 <= col < c1, in input order, rebased to
 * the block's origin (gcn_distr.py:404-406; the 2D variant gcn_distr_2d.py:1040-1047).  d_val
 * and d_out_val may both be NULL (pattern only).  *out_nnz receives the block's size; with all
 * outputs NULL the call only counts. */
int cg_coo_block(const int32_t *d_row, const int32_t *d_col, const float *d_val, int64_t nnz, int32_t r0, int32_t r1,
                 int32_t c0, int32_t c1, int32_t *d_out_row, int32_t *d_out_col, float *d_out_val, int64_t capacity,
                 int64_t *out_nnz, cg_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Kernel timing (the reference brackets phases with wall clocks and device synchronisation,
 * gcn_distr.py:66-94; here HIP events are recorded on the launch stream around single kernels).
 * cg_prof_enable(1) starts recording, cg_prof_enable(0) stops.  cg_prof_read waits for the
 * recorded events of `name`, returns their summed duration in milliseconds and their number, and
 * forgets them.  A record's name ends in "/f=<number>": the width of an SpMM product
 * ("spmm_rowseg/f=602"), the reduction length k of a dense product ("dense_xw/f=602"), the number
 * of classes of a row-wise kernel.  Names: "spmm_rowseg" (the main kernel of a
 * product, or the cold class of a hub plan), "spmm_hub_hot" (all hot tiers of a hub plan as one
 * record), "spmm_reduce" (rows split into segments), "spmm_hub_reduce" (partial rows of a hub plan
 * with narrow teams), "spmm_panel" (staged tiles of a panel plan and the sum of a panel's blocks of
 * partial rows), "spmm_panel_dense" (its dense tiles on the matrix cores), "spmm_panel_add" (partial rows added to a narrow
 * product), "dense_xw", "dense_gwt", "dense_xtg" (partial products and their sum),
 * "relu_fwd", "relu_bwd" (no suffix), "log_softmax_fwd", "log_softmax_bwd", "nll_fwd", "nll_bwd",
 * "log_softmax_nll_bwd".
 * Recording is off by default and costs nothing then.
 */
int cg_prof_enable(int on);
/* Tuning knobs, 0 = built-in choice (no counterpart in the reference, which hands every choice to
 * cuSPARSE).  Results stay deterministic for a given setting; different settings change the
 * summation order of split rows.
 *   "spmm_seg"        stored entries per row segment (>= 64; narrow teams cap it at 512)
 *   "spmm_win"        stored entries after which a new window of tasks starts (64..512)
 *   "spmm_vec"        cap on the floats a lane moves per access (1, 2; otherwise 4)
 *   "spmm_hub"        hub plan: -1 never, 1 always, 0 by width and density
 *   "spmm_hub_kb"     KiB of hot B rows per XCD group and tier
 *   "spmm_hub_groups" XCD groups the hot columns are dealt to (1, 2, 4, 8)
 *   "spmm_hub_tiers"  tiers of hot columns (0: chosen from the column counts; groups * tiers <= 64)
 *   "spmm_hub_row"    rows with fewer entries keep all of them in the cold class (0: 64)
 *   "spmm_panel"      panel plan (dense row-panel x column-block tiles multiplied out of LDS; even widths
 *                     258..636): -1 never, 1 always, 0 when the product has at least 8e8 multiply-adds, rows hold at
 *                     least 8 entries on average and at least half of the entries share their column with another
 *                     entry of the same panel of 128 rows
 *   "spmm_panel_emin" entries a 128 x 32 tile needs to be staged (0: 1, every tile; tiles below it leave their
 *                     entries to the row-wise kernels)
 *   "spmm_panel_cols" column ranks inside a row panel that can be part of a tile (0: all)
 *   "spmm_panel_unit" entries after which the tiles of a row panel go to another workgroup (0: 65536)
 *   "spmm_panel_dmin" entries from which a 128 x 32 tile is stored whole and multiplied on the fp32 matrix
 *                     cores (0: 768; negative: never).  Such a tile multiplies its zeros too:
 *                     a row of B with an infinity or a NaN then reaches all 128 rows of the tile
 *   "spmm_panel_dwg"  workgroups that share the dense tiles equally (0: four per compute unit)
 *   "spmm_panel_share" 0: the columns a row panel stages keep the order of their entry counts in the whole matrix, and
 *                     units whose panels start at the same place of that order are queued for one XCD together
 *                     (one copy from memory then serves them all out of that XCD's L2); -1: every panel orders its
 *                     columns by their entries in the panel, costliest units first
 *   "spmm_panel_narrow" the same plan with dense tiles only for narrow products (f <= 64; the other entries go to the
 *                     row-wise kernels and the partial rows are added in afterwards): -1 never, 1 always, 0 when rows
 *                     hold at least 64 entries on average, the product has at least 1e9 multiply-adds and the dense
 *                     tiles hold at least a quarter of the entries
 *   "spmm_panel_narrow_dmin" entries from which a tile is dense for narrow products (0: 512)
 *   "spmm_panel_legacy" 1: the staged tiles of the panel plan go through the older kernel, which keeps a panel's rows
 *                     in named registers and takes the records of a (tile, wave, row) run in pairs, padded; 0: through
 *                     the tile kernel (accumulators addressed through the register index, records as they are).  A B
 *                     that is not 8-byte aligned or has an odd leading dimension goes to the older kernel whatever
 *                     this says (the tile kernel's copies need 8-byte aligned rows), and so do the widths 634 and 636,
 *                     two of whose tiles the tile kernel's LDS layout has no room for
 *   "spmm_tile"       tile plans (every entry multiplied out of LDS by the tile kernel; panels of 256 rows and
 *                     column slices of up to 316 columns for widths above 128, 512 rows for 65..128, 1024 rows up
 *                     to 64): -1 never, 1 always, 0 by width and matrix: widths from 65 on except the even widths
 *                     318..636 where the panel plan is in use, and 48..64 on matrices of under 64 entries per row,
 *                     on products of at least 8e8 multiply-adds with at least 8 entries per row
 *   "spmm_strict_nonfinite" 1: no plan that multiplies stored zeros (the dense tiles of the panel plans) or padding
 *                     records: a row of B with an infinity or a NaN then reaches exactly the rows of C that have an
 *                     entry in that column, as in a product entry by entry (cusparseSpMM in the reference)
 *   "spmm_panel_qskip", "spmm_panel_qcap" measuring aids for the older staged-tile kernel ("spmm_panel_legacy" 1):
 *                     a launch takes only the units from position qskip on, or before position qcap, of each of its
 *                     eight unit queues; the product is then incomplete
 *   "dense_mfma"      -1: dense products on the vector ALU tile kernel only
 *   "coo_cache_blocks" blocks cg_spmm_coo_cached keeps (0: 8; negative: none)
 *   "coo_cache_mib"   device memory those blocks may hold together, in MiB (0: 32768); a block counts as four
 *                     copies of its entries (the CSR and its plans); the newest block always stays
 *   "test_alloc_fail" test hook: k > 0 makes the k-th device allocation for handle tables from now on fail
 *                     once with CG_ERR_ALLOC (a plan whose build fails that way is given up for good and the
 *                     product runs on the plain schedule)
 * An unknown key returns CG_ERR_UNSUPPORTED. */
int cg_tune_set(const char *key, int value);
int cg_prof_read(const char *name, double *total_ms, int64_t *launches);


#ifdef __cplusplus
}
#endif
#endif /* CAGNET_AMD_H */
