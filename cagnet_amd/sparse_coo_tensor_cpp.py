"""The reference's native module, name for name.

CAGNET's drivers do `from sparse_coo_tensor_cpp import sparse_coo_tensor_gpu, spmm_gpu`
(gcn_distr.py:27, gcn_distr_15d.py:27, gcn_distr_2d.py:38, gcn_distr_3d.py:36); the module is
registered at sparse-extension/sparse_coo_tensor.cu:242-245.  This module exports the same two
names with the same positional signatures, plus `coo2csr`, which the reference only runs
internally (sparse_coo_tensor.cu:136-142).

Differences a caller can observe, all deliberate:
  * errors raise (CagnetError) instead of being printed and ignored (sparse_coo_tensor.cu:20-30);
  * B and C keep their storage and their row-major layout; the reference hands both back as
    column-major strided views of fresh storage (sparse_coo_tensor.cu:166-168, :183-185, :233-239);
  * the call is ordered on torch's current stream; with `cache_blocks` (the default) it
    synchronises that stream once per call to read back a 16-byte digest, without it not at all
    (the reference synchronises the whole device on every call, sparse_coo_tensor.cu:231).

`cache_blocks`: the reference's callers pass the same block at every stage of every epoch, as
fresh `.int()` temporaries.  When True, spmm_gpu recognises a block by a digest of its arrays and
reuses the CSR, schedules and plans built when it first saw it (cg_spmm_coo_cached); when False
every call rebuilds them on the device (cg_spmm_coo).  Kept blocks hold device memory (about four
copies of a block's entries each, at most 8 blocks or 32 GiB, least recently used dropped first;
`ops.coo_cache_clear()` hands it back).  A caller whose values change on every call should set it to
False: every call would otherwise build a handle and a plan for a block that is never seen again.

Precondition, as in the reference (cusparseXcoo2csr needs sorted rows, sparse_coo_tensor.cu:137-142):
rows ascending, 0 <= row < n, 0 <= col < m.  What happens when it does not hold depends on the path:
  * wide products over dense blocks (f >= 64, at least 8 entries per row, nnz * f >= 3e9) with
    `cache_blocks`: checked when a block is first seen; CagnetError (CG_ERR_UNSORTED, CG_ERR_INDEX);
  * every other product: not checked.  Indices are clamped, so nothing outside the operands is
    touched, but C is then as meaningless as in the reference.  Set `validate_inputs = True` to
    check every call first (one more pass over the indices and one stream synchronisation per call).
"""
from __future__ import annotations

from typing import Sequence

import torch

from . import ops

__all__ = ["spmm_gpu", "sparse_coo_tensor_gpu", "coo2csr", "cache_blocks", "validate_inputs"]

cache_blocks = True
validate_inputs = False


def spmm_gpu(A_rowindices: torch.Tensor, A_colindices: torch.Tensor, A_values: torch.Tensor, n: int, m: int,
             B: torch.Tensor, C: torch.Tensor) -> None:
    """C += A @ B.  A is n x m, given as row-sorted COO with int32 indices and fp32 values
    (the callers pass `.indices()[k].int()` of a coalesced tensor, gcn_distr.py:238-240);
    B is m x f and C is n x f, both fp32.  Returns None, like the reference."""
    if validate_inputs:
        ops.coo_check(A_rowindices, A_colindices, int(n), int(m), require_sorted=True)
    B = ops.aligned_rows(B)   # a B registered with ops.keep_aligned: read through its kept copy with line-aligned rows
    if C.dim() == 2 and C.numel() > 0 and C.stride(1) != 1:
        # a transposed view, e.g. a C that an earlier reference-style call left column-major
        tmp = C.contiguous()
        ops.spmm_coo(A_rowindices, A_colindices, A_values, int(n), int(m), B, tmp, beta=1.0, cached=cache_blocks)
        C.copy_(tmp)
        return None
    ops.spmm_coo(A_rowindices, A_colindices, A_values, int(n), int(m), B, C, beta=1.0, cached=cache_blocks)
    return None


def sparse_coo_tensor_gpu(indices: torch.Tensor, values: torch.Tensor, size: Sequence[int]) -> torch.Tensor:
    """COO constructor that skips index validation (and its device synchronisation), like
    sparse_coo_tensor_gpu at sparse-extension/sparse_coo_tensor.cu:43-54.  No kernel is involved."""
    if indices.dim() != 2:
        raise ValueError("indices must be 2-D (sparse_dim x nnz)")
    return torch.sparse_coo_tensor(indices, values, tuple(size), check_invariants=False)


def coo2csr(A_rowindices: torch.Tensor, A_colindices: torch.Tensor, A_values: torch.Tensor, n: int, m: int,
            transpose: bool = False):
    """(rowptr[n+1], colind[nnz], values[nnz]) in (row, col) order, from COO in any order.
    The reference performs only the row compression, on sorted input, inside spmm_gpu
    (cusparseXcoo2csr, sparse_coo_tensor.cu:137-142).

    transpose=True appends the CSR of A^T, which the backward products A^T G read
    (gcn_distr.py:306, :326 pass `adj_matrix.t()` blocks): the result is then
    (rowptr, colind, values, colptr[m+1], rowind[nnz], values_t[nnz], perm[nnz]) with
    values_t[k] == values[perm[k]], entry k of A^T being entry perm[k] of A."""
    rowptr, colind, values = ops.coo2csr(A_rowindices, A_colindices, A_values, int(n), int(m))
    if not transpose:
        return rowptr, colind, values
    colptr, rowind, values_t, perm = ops.csr_transpose(rowptr, colind, values, int(n), int(m), return_perm=True)
    return rowptr, colind, values, colptr, rowind, values_t, perm
