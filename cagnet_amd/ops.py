"""Tensor-level wrappers over the C ABI: torch supplies device memory and the current stream,
every computation happens in libcagnet_amd.so.

Dense operands are fp32 CUDA(HIP) tensors, row-major with unit column stride (a row stride larger
than the column count is passed on as the leading dimension).  Sparse indices are int32.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int64, c_void_p
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import CG_CSR_SORTED, CG_CSR_TRANSPOSE, CG_CSR_VALIDATE, CagnetError, check, lib

__all__ = [
    "CagnetError", "CsrMatrix", "coo2csr_rowptr", "coo2csr", "csr_transpose", "coo_check", "spmm_coo",
    "dense_xw", "dense_gwt", "dense_xtg", "relu_fwd", "relu_bwd", "log_softmax_fwd", "log_softmax_bwd",
    "nll_loss_fwd", "nll_loss_bwd", "log_softmax_nll_bwd",
]


def _stream() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def scratch_release(stream: "torch.cuda.Stream | None" = None) -> int:
    """Free the library's scratch buffers of `stream` (default: the current stream), including
    buffers kept alive because a captured HIP graph used them (cg_scratch_release).  Synchronises
    the stream.  Returns the number of bytes freed."""
    released = ctypes.c_int64(0)
    handle = c_void_p(stream.cuda_stream) if stream is not None else _stream()
    check(lib.cg_scratch_release(handle, ctypes.byref(released)), "cg_scratch_release")
    return int(released.value)


def _ptr(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else c_void_p(0)


def _need(t: torch.Tensor, name: str, dtype: torch.dtype, dim: Optional[int] = None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a torch.Tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise ValueError(f"{name}: must live on the GPU (got device {t.device}); there is no CPU path")
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if dim is not None and t.dim() != dim:
        raise ValueError(f"{name}: expected {dim} dimensions, got {t.dim()}")
    return t


def _index(t: torch.Tensor, name: str) -> torch.Tensor:
    t = _need(t, name, torch.int32, 1)
    return t if t.is_contiguous() else t.contiguous()


def _values(t: torch.Tensor, name: str) -> torch.Tensor:
    t = _need(t, name, torch.float32, 1)
    return t if t.is_contiguous() else t.contiguous()


def _rowmajor(t: torch.Tensor, name: str) -> Tuple[torch.Tensor, int]:
    """Return (tensor, leading dimension).  Copies only when the column stride is not 1."""
    t = _need(t, name, torch.float32, 2)
    rows, cols = t.shape
    if cols > 0 and t.stride(1) != 1 or (rows > 1 and t.stride(0) < cols):
        t = t.contiguous()
    ld = t.stride(0) if rows > 1 else max(cols, 1)
    return t, max(ld, cols, 1)


def _out_rowmajor(t: torch.Tensor, name: str) -> int:
    _need(t, name, torch.float32, 2)
    rows, cols = t.shape
    if (cols > 1 and t.stride(1) != 1) or (rows > 1 and t.stride(0) < cols):
        raise ValueError(f"{name}: output must be row-major with unit column stride (strides {t.stride()})")
    # the library is about to write into t behind torch's back: say so, for everything that goes by a tensor's
    # version (autograd's saved tensors, the copies aligned_rows keeps)
    torch.autograd.graph.increment_version(t)
    return max(t.stride(0) if rows > 1 else cols, cols, 1)


# ------------------------------------------------------------------------------------------------
# coo2csr family
# ------------------------------------------------------------------------------------------------
def coo2csr_rowptr(row: torch.Tensor, n: int) -> torch.Tensor:
    """rowptr[n+1] of ascending int32 row indices (cusparseXcoo2csr of the reference,
    sparse-extension/sparse_coo_tensor.cu:136-142)."""
    row = _index(row, "row")
    rowptr = torch.empty(n + 1, dtype=torch.int32, device=row.device)
    check(lib.cg_coo2csr_rowptr(_ptr(row), row.numel(), n, _ptr(rowptr), _stream()), "cg_coo2csr_rowptr")
    return rowptr


def coo_check(row: torch.Tensor, col: torch.Tensor, n: int, m: int, require_sorted: int = 1) -> None:
    row, col = _index(row, "row"), _index(col, "col")
    if row.numel() != col.numel():
        raise ValueError("row and col differ in length")
    check(lib.cg_coo_check(_ptr(row), _ptr(col), row.numel(), n, m, require_sorted, _stream()), "cg_coo_check")


def coo2csr(row: torch.Tensor, col: torch.Tensor, val: Optional[torch.Tensor], n: int, m: int,
            return_perm: bool = False):
    """COO in any order -> (rowptr, colind, values[, perm]) sorted by (row, col), stable."""
    row, col = _index(row, "row"), _index(col, "col")
    nnz = row.numel()
    if col.numel() != nnz or (val is not None and val.numel() != nnz):
        raise ValueError("row, col and val differ in length")
    if val is not None:
        val = _values(val, "val")
    dev = row.device
    rowptr = torch.empty(n + 1, dtype=torch.int32, device=dev)
    colind = torch.empty(nnz, dtype=torch.int32, device=dev)
    values = torch.empty(nnz, dtype=torch.float32, device=dev) if val is not None else None
    perm = torch.empty(nnz, dtype=torch.int32, device=dev) if return_perm else None
    check(lib.cg_coo2csr(_ptr(row), _ptr(col), _ptr(val), nnz, n, m, _ptr(rowptr), _ptr(colind), _ptr(values),
                         _ptr(perm), _stream()), "cg_coo2csr")
    return (rowptr, colind, values, perm) if return_perm else (rowptr, colind, values)


# ------------------------------------------------------------------------------------------------
# input preparation (host code in the reference: gcn_distr.py:791, :412-470, :398-409)
# ------------------------------------------------------------------------------------------------
def add_self_loops(row: torch.Tensor, col: torch.Tensor, n: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Strictly ascending int32 COO pattern of an n x n matrix -> the same pattern with every
    diagonal entry present exactly once (add_remaining_self_loops, gcn_distr.py:791)."""
    row, col = _index(row, "row"), _index(col, "col")
    if row.numel() != col.numel():
        raise ValueError("row and col differ in length")
    count = ctypes.c_int64(0)
    check(lib.cg_add_self_loops(_ptr(row), _ptr(col), row.numel(), n, None, None, 0, ctypes.byref(count), _stream()),
          "cg_add_self_loops")
    out_row = torch.empty(count.value, dtype=torch.int32, device=row.device)
    out_col = torch.empty(count.value, dtype=torch.int32, device=row.device)
    check(lib.cg_add_self_loops(_ptr(row), _ptr(col), row.numel(), n, _ptr(out_row), _ptr(out_col), count.value,
                                ctypes.byref(count), _stream()), "cg_add_self_loops")
    return out_row, out_col


def gcn_normalize(row: torch.Tensor, col: torch.Tensor, n: int, return_dinv: bool = False):
    """fp32 values of D^-1/2 A D^-1/2 for a pattern that already holds its self-loops, in the
    arithmetic of scale_elements (gcn_distr.py:439-468).  Bit-identical to the host computation."""
    row, col = _index(row, "row"), _index(col, "col")
    if row.numel() != col.numel():
        raise ValueError("row and col differ in length")
    val = torch.empty(row.numel(), dtype=torch.float32, device=row.device)
    dinv = torch.empty(n, dtype=torch.float32, device=row.device) if return_dinv else None
    check(lib.cg_gcn_normalize(_ptr(row), _ptr(col), row.numel(), n, _ptr(val), _ptr(dinv), _stream()),
          "cg_gcn_normalize")
    return (val, dinv) if return_dinv else val


def coo_block(row: torch.Tensor, col: torch.Tensor, val: Optional[torch.Tensor], r0: int, r1: int, c0: int, c1: int):
    """Entries inside [r0, r1) x [c0, c1) in input order, rebased to the block (split_coo,
    gcn_distr.py:398-409): (row, col, val)."""
    row, col = _index(row, "row"), _index(col, "col")
    nnz = row.numel()
    if col.numel() != nnz or (val is not None and val.numel() != nnz):
        raise ValueError("row, col and val differ in length")
    if val is not None:
        val = _values(val, "val")
    count = ctypes.c_int64(0)
    check(lib.cg_coo_block(_ptr(row), _ptr(col), _ptr(val), nnz, r0, r1, c0, c1, None, None, None, 0,
                           ctypes.byref(count), _stream()), "cg_coo_block")
    dev = row.device
    out_row = torch.empty(count.value, dtype=torch.int32, device=dev)
    out_col = torch.empty(count.value, dtype=torch.int32, device=dev)
    out_val = torch.empty(count.value, dtype=torch.float32, device=dev) if val is not None else None
    if count.value:
        check(lib.cg_coo_block(_ptr(row), _ptr(col), _ptr(val), nnz, r0, r1, c0, c1, _ptr(out_row), _ptr(out_col),
                               _ptr(out_val), count.value, ctypes.byref(count), _stream()), "cg_coo_block")
    return out_row, out_col, out_val


def csr_transpose(rowptr: torch.Tensor, colind: torch.Tensor, values: Optional[torch.Tensor], n: int, m: int,
                  return_perm: bool = False):
    """CSR of A (n x m) -> CSR of A^T (m x n): (colptr, rowind, values_t[, perm])."""
    rowptr, colind = _index(rowptr, "rowptr"), _index(colind, "colind")
    if rowptr.numel() != n + 1:
        raise ValueError(f"rowptr has {rowptr.numel()} entries, expected n + 1 = {n + 1}")
    nnz = colind.numel()
    if values is not None:
        values = _values(values, "values")
        if values.numel() != nnz:
            raise ValueError("colind and values differ in length")
    dev = rowptr.device
    colptr = torch.empty(m + 1, dtype=torch.int32, device=dev)
    rowind = torch.empty(nnz, dtype=torch.int32, device=dev)
    values_t = torch.empty(nnz, dtype=torch.float32, device=dev) if values is not None else None
    perm = torch.empty(nnz, dtype=torch.int32, device=dev) if return_perm else None
    check(lib.cg_csr_transpose(_ptr(rowptr), _ptr(colind), _ptr(values), nnz, n, m, _ptr(colptr), _ptr(rowind),
                               _ptr(values_t), _ptr(perm), _stream()), "cg_csr_transpose")
    return (colptr, rowind, values_t, perm) if return_perm else (colptr, rowind, values_t)


# ------------------------------------------------------------------------------------------------
# SpMM
# ------------------------------------------------------------------------------------------------
def spmm_coo(row: torch.Tensor, col: torch.Tensor, val: torch.Tensor, n: int, m: int, B: torch.Tensor,
             C: torch.Tensor, beta: float = 1.0, cached: bool = False) -> None:
    """C[n,f] = beta*C + A*B with A as row-sorted COO; the one-shot form of the reference operator
    (sparse-extension/sparse_coo_tensor.cu:113-240).  cached=True recognises a block it has seen
    before by a digest of its arrays and reuses the CSR, schedules and plans built then (one stream
    synchronisation per call); cached=False rebuilds them as asynchronous device work."""
    row, col, val = _index(row, "row"), _index(col, "col"), _values(val, "val")
    if not (row.numel() == col.numel() == val.numel()):
        raise ValueError("row, col and val differ in length")
    B, ldb = _rowmajor(B, "B")
    ldc = _out_rowmajor(C, "C")
    if B.shape[0] != m or C.shape[0] != n or B.shape[1] != C.shape[1]:
        raise ValueError(f"shape mismatch: A is {n}x{m}, B is {tuple(B.shape)}, C is {tuple(C.shape)}")
    fn, name = (lib.cg_spmm_coo_cached, "cg_spmm_coo_cached") if cached else (lib.cg_spmm_coo, "cg_spmm_coo")
    check(fn(_ptr(row), _ptr(col), _ptr(val), val.numel(), n, m, _ptr(B), ldb, _ptr(C), ldc, B.shape[1],
             float(beta), _stream()), name)


def coo_cache_info() -> dict:
    """Blocks spmm_coo(cached=True) keeps, and its hits / misses / evictions so far."""
    info = (ctypes.c_int64 * 4)()
    check(lib.cg_coo_cache_info(info), "cg_coo_cache_info")
    return {"blocks": info[0], "hits": info[1], "misses": info[2], "evictions": info[3]}


def coo_cache_clear() -> None:
    """Drop every block spmm_coo(cached=True) keeps."""
    check(lib.cg_coo_cache_clear(), "cg_coo_cache_clear")


class _DeviceArray:
    """Zero-copy view of handle-owned device memory for torch.as_tensor."""

    def __init__(self, ptr: int, count: int, typestr: str):
        self.__cuda_array_interface__ = {
            "shape": (count,), "typestr": typestr, "data": (ptr, False), "version": 2, "strides": None,
        }


class CsrMatrix:
    """Device-resident CSR of one sparse block (and optionally of its transpose) with cached
    schedules: what the reference rebuilds inside every spmm_gpu call is built once here."""

    def __init__(self, row: torch.Tensor, col: torch.Tensor, val: torch.Tensor, n: int, m: int, *,
                 is_sorted: bool = True, transpose: bool = False, validate: bool = False):
        row, col, val = _index(row, "row"), _index(col, "col"), _values(val, "val")
        if not (row.numel() == col.numel() == val.numel()):
            raise ValueError("row, col and val differ in length")
        flags = (CG_CSR_SORTED if is_sorted else 0) | (CG_CSR_TRANSPOSE if transpose else 0) | (
            CG_CSR_VALIDATE if validate else 0)
        handle = c_void_p(0)
        self._handle = None
        self.device = row.device
        with torch.cuda.device(self.device):
            check(lib.cg_csr_create(ctypes.byref(handle), _ptr(row), _ptr(col), _ptr(val), val.numel(), n, m, flags,
                                    _stream()), "cg_csr_create")
        self._handle = handle
        self.n, self.m, self.nnz = int(n), int(m), int(val.numel())
        self.has_transpose = bool(transpose)

    @classmethod
    def from_torch_coo(cls, a: torch.Tensor, **kw) -> "CsrMatrix":
        """From a coalesced torch.sparse_coo tensor (the type the reference keeps its blocks in,
        gcn_distr.py:493-512, :546)."""
        a = a.coalesce()
        idx = a.indices()
        return cls(idx[0].int(), idx[1].int(), a.values().float(), a.shape[0], a.shape[1], is_sorted=True, **kw)

    @classmethod
    def hstack(cls, blocks: Sequence["CsrMatrix"], transpose: bool = False) -> "CsrMatrix":
        """[A_0 | A_1 | ...]: the blocks of one block row side by side as one matrix (cg_csr_hstack).  One product
        with the stacked dense blocks is the whole stage loop sum_k A_k H_k (gcn_distr.py:221-244).  The entries
        are copied; `col_offsets[k]` is the first column of block k in the result."""
        blocks = list(blocks)
        if not blocks:
            raise ValueError("hstack of no blocks")
        self = cls.__new__(cls)
        self._handle = None
        self.device = blocks[0].device
        arr = (c_void_p * len(blocks))(*[b._handle for b in blocks])
        handle = c_void_p(0)
        with torch.cuda.device(self.device):
            check(lib.cg_csr_hstack(ctypes.byref(handle), arr, len(blocks), CG_CSR_TRANSPOSE if transpose else 0, _stream()),
                  "cg_csr_hstack")
        self._handle = handle
        self.n, self.m, self.nnz = blocks[0].n, sum(b.m for b in blocks), sum(b.nnz for b in blocks)
        self.has_transpose = bool(transpose)
        self.col_offsets = [sum(b.m for b in blocks[:k]) for k in range(len(blocks) + 1)]
        return self

    def __del__(self):
        h = getattr(self, "_handle", None)
        if h is not None and lib is not None:
            try:
                lib.cg_csr_destroy(h)
            except Exception:
                pass
            self._handle = None

    # ---- one byte string per block: files and transfers (the reference pickles int64 COO,
    # gcn_distr.py:747, and sends indices as float32, gcn_distr_2d.py:369-374) ----------------------
    def to_blob(self):
        """The block as a numpy uint8 array: 128-byte header, int32 rowptr / colind, fp32 values."""
        import numpy as np
        size = c_int64(0)
        check(lib.cg_csr_blob_size(self._handle, ctypes.byref(size)), "cg_csr_blob_size")
        buf = np.empty(size.value, dtype=np.uint8)
        with torch.cuda.device(self.device):
            check(lib.cg_csr_blob_write(self._handle, c_void_p(buf.ctypes.data), size.value, _stream()),
                  "cg_csr_blob_write")
        return buf

    @classmethod
    def from_blob(cls, blob, device="cuda:0", transpose: bool = False) -> "CsrMatrix":
        """Rebuild a block from `to_blob` bytes (numpy uint8 array, bytes or a memory map).  The
        content is checked (header, checksum, rowptr, column range) before anything is launched on it."""
        import numpy as np
        buf = np.frombuffer(blob, dtype=np.uint8) if not isinstance(blob, np.ndarray) else blob
        if buf.dtype != np.uint8 or buf.ndim != 1 or not buf.flags["C_CONTIGUOUS"]:
            raise ValueError("blob must be a contiguous 1-D uint8 buffer")
        self = cls.__new__(cls)
        self._handle = None
        self.device = torch.device(device)
        handle = c_void_p(0)
        with torch.cuda.device(self.device):
            check(lib.cg_csr_blob_read(ctypes.byref(handle), c_void_p(buf.ctypes.data), buf.size,
                                       CG_CSR_TRANSPOSE if transpose else 0, _stream()), "cg_csr_blob_read")
        self._handle = handle
        info = self.info()
        self.n, self.m, self.nnz = int(info["n"]), int(info["m"]), int(info["nnz"])
        self.has_transpose = bool(info["has_transpose"])
        return self

    def save(self, path) -> None:
        self.to_blob().tofile(path)

    @classmethod
    def load(cls, path, device="cuda:0", transpose: bool = False) -> "CsrMatrix":
        import numpy as np
        return cls.from_blob(np.memmap(path, dtype=np.uint8, mode="r"), device=device, transpose=transpose)

    @property
    def shape(self) -> Tuple[int, int]:
        return (self.n, self.m)

    def graph_retain(self) -> None:
        """A captured graph that multiplies with this matrix now exists (`gcn.GraphedTrain` calls this)."""
        self._graph_refs = getattr(self, "_graph_refs", 0) + 1

    def graph_release(self) -> int:
        """One of the graphs counted by `graph_retain` is gone.  The tables the library parked for captured
        graphs are freed (`unpin`) only when the last one is: a graph that is still alive replays with their
        addresses.  Returns the number of device allocations freed."""
        refs = getattr(self, "_graph_refs", 0)
        if refs <= 0:
            return 0
        self._graph_refs = refs - 1
        return self.unpin() if self._graph_refs == 0 else 0

    def unpin(self) -> int:
        """Free the tables this matrix has kept alive for HIP graphs captured over its products
        (cg_csr_unpin): call it only when none of those graphs will be replayed again.  Returns the
        number of device allocations freed."""
        released = ctypes.c_int64(0)
        check(lib.cg_csr_unpin(self._handle, ctypes.byref(released)), "cg_csr_unpin")
        return int(released.value)

    def info(self) -> dict:
        buf = (c_int64 * 8)()
        check(lib.cg_csr_info(self._handle, buf), "cg_csr_info")
        return {"n": buf[0], "m": buf[1], "nnz": buf[2], "has_transpose": bool(buf[3]),
                "max_row_degree": buf[4], "max_col_degree": buf[5],
                # column-popularity plan the last wide product looked up: tiers, -1 declined, 0 none
                "plan_tiers": buf[6], "plan_tiers_transpose": buf[7]}

    def panel_info(self, transpose: bool = False, narrow: bool = False, tile: int = 0) -> dict:
        """Panel plan the last wide (narrow=True: narrow, f <= 64) product of A (transpose=True: of A^T) looked up, or
        with tile = 1, 2, 3 the tile plan with panels of 256, 512, 1024 rows:
        state 1 in use / -1 declined / 0 none considered; entries multiplied out of LDS, in dense tiles on the matrix
        cores, left to the row-wise kernels; tile and unit counts; the thresholds the plan was built with."""
        buf = (c_int64 * 12)()
        which = int(transpose) | (2 if narrow else 0) | ((int(tile) & 3) << 2)
        check(lib.cg_csr_panel_info(self._handle, which, buf), "cg_csr_panel_info")
        return {"state": buf[0], "staged_entries": buf[1], "staged_tiles": buf[2], "staged_units": buf[3],
                "split_panels": buf[4], "rest_entries": buf[5], "tile_min_entries": buf[6], "column_ranks": buf[7],
                "dense_entries": buf[8], "dense_tiles": buf[9], "dense_units": buf[10], "dense_min_entries": buf[11]}

    def plan_signature(self, f: int, launched, transpose: bool = False) -> str:
        """What decides the memory traffic of a product of width f besides the kernels it launched (`launched`: their
        profiling names): the parameters and sizes of the plan it ran on - the tile plan of the width's panel height,
        else the panel plan, else the narrow plan's dense tiles - and the tiers of a hub plan."""
        parts = []
        if "spmm_panel" in launched or "spmm_panel_dense" in launched:
            tile = ("tile", dict(tile=1 if f > 128 else 2 if f > 64 else 3))
            # tiles on the matrix cores: only the panel plan (wide products) and the narrow plan have them
            order = ((("narrow", dict(narrow=True)),) if f <= 64 else (("panel", dict()),)) if "spmm_panel_dense" in launched \
                else (tile, ("panel", dict()))
            for name, kw in order:
                i = self.panel_info(transpose=transpose, **kw)
                if i["state"] == 1:
                    parts.append("%s:e%d.c%d.d%d.t%d.u%d.dt%d.r%d" % (
                        name, i["tile_min_entries"], i["column_ranks"], i["dense_min_entries"], i["staged_tiles"],
                        i["staged_units"], i["dense_tiles"], i["rest_entries"]))
                    break
        if "spmm_hub_hot" in launched:
            parts.append("hub:%d" % self.info()["plan_tiers_transpose" if transpose else "plan_tiers"])
        return ",".join(parts) if parts else "rowwise"

    def arrays(self, transpose: bool = False):
        """(rowptr, colind, values) of A, or of A^T, as tensors that alias the handle's memory."""
        p = [c_void_p(0), c_void_p(0), c_void_p(0)]
        check(lib.cg_csr_arrays(self._handle, int(transpose), ctypes.byref(p[0]), ctypes.byref(p[1]),
                                ctypes.byref(p[2])), "cg_csr_arrays")
        rows = self.m if transpose else self.n
        out = [torch.as_tensor(_DeviceArray(p[0].value, rows + 1, "<i4"), device=self.device)]
        if self.nnz > 0:
            out.append(torch.as_tensor(_DeviceArray(p[1].value, self.nnz, "<i4"), device=self.device))
            out.append(torch.as_tensor(_DeviceArray(p[2].value, self.nnz, "<f4"), device=self.device))
        else:
            out.append(torch.empty(0, dtype=torch.int32, device=self.device))
            out.append(torch.empty(0, dtype=torch.float32, device=self.device))
        return tuple(out)

    def spmm(self, B: torch.Tensor, out: Optional[torch.Tensor] = None, beta: float = 0.0,
             transpose: bool = False) -> torch.Tensor:
        """out = beta*out + op(A)*B.  A fresh output is allocated (and beta forced to 0) if none is given."""
        B, ldb = _rowmajor(B, "B")
        rows, inner = (self.m, self.n) if transpose else (self.n, self.m)
        if B.shape[0] != inner:
            raise ValueError(f"B has {B.shape[0]} rows, the sparse operand has {inner} columns")
        f = B.shape[1]
        if out is None:
            out = torch.empty(rows, f, dtype=torch.float32, device=B.device)
            beta = 0.0
        ldc = _out_rowmajor(out, "out")
        if tuple(out.shape) != (rows, f):
            raise ValueError(f"out has shape {tuple(out.shape)}, expected {(rows, f)}")
        check(lib.cg_csr_spmm(self._handle, int(transpose), _ptr(B), ldb, _ptr(out), ldc, f, float(beta), _stream()),
              "cg_csr_spmm")
        return out


    def spmm_xw(self, B: torch.Tensor, W: torch.Tensor, relu: bool = False, acc: Optional[torch.Tensor] = None,
                transpose: bool = False) -> Optional[torch.Tensor]:
        """Z = act((acc + op(A) @ B) @ W) in one pass, without the rows x f intermediate (the two
        steps of GCNFunc.forward, gcn_distr.py:271-275).  `acc` is the sum of earlier stages (read
        only).  Returns None when this width has no fused form; the caller then uses spmm + dense_xw."""
        B, ldb = _rowmajor(B, "B")
        W, ldw = _rowmajor(W, "W")
        rows, inner = (self.m, self.n) if transpose else (self.n, self.m)
        f, fo = B.shape[1], W.shape[1]
        if B.shape[0] != inner or W.shape[0] != f:
            raise ValueError(f"B is {tuple(B.shape)}, W is {tuple(W.shape)}, the sparse operand has {inner} columns")
        ldc = 0
        if acc is not None:
            acc, ldc = _rowmajor(acc, "acc")
            if tuple(acc.shape) != (rows, f):
                raise ValueError(f"acc has shape {tuple(acc.shape)}, expected {(rows, f)}")
        Z = torch.empty(rows, fo, dtype=torch.float32, device=B.device)
        st = lib.cg_csr_spmm_xw(self._handle, int(transpose), _ptr(B), ldb, _ptr(acc), ldc, 1.0 if acc is not None else 0.0,
                                _ptr(W), ldw, _ptr(Z), max(fo, 1), f, fo, int(relu), _stream())
        if st == _lib.CG_ERR_UNSUPPORTED:
            return None
        check(st, "cg_csr_spmm_xw")
        return Z


# ------------------------------------------------------------------------------------------------
# dense products
# ------------------------------------------------------------------------------------------------
def dense_xw(X: torch.Tensor, W: torch.Tensor, relu: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Z = X @ W (optionally ReLU fused into the store); torch.mm at gcn_distr.py:275."""
    X, ldx = _rowmajor(X, "X")
    W, ldw = _rowmajor(W, "W")
    n, k = X.shape
    if W.shape[0] != k:
        raise ValueError(f"X is {tuple(X.shape)}, W is {tuple(W.shape)}")
    fo = W.shape[1]
    if out is None:
        out = torch.empty(n, fo, dtype=torch.float32, device=X.device)
    ldz = _out_rowmajor(out, "out")
    check(lib.cg_dense_xw(_ptr(X), ldx, _ptr(W), ldw, _ptr(out), ldz, n, k, fo, int(relu), _stream()), "cg_dense_xw")
    return out


def dense_gwt(G: torch.Tensor, W: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """dX = G @ W.T; torch.mm(ag, weight.t()) at gcn_distr.py:330."""
    G, ldg = _rowmajor(G, "G")
    W, ldw = _rowmajor(W, "W")
    n, fo = G.shape
    k = W.shape[0]
    if W.shape[1] != fo:
        raise ValueError(f"G is {tuple(G.shape)}, W is {tuple(W.shape)}")
    if out is None:
        out = torch.empty(n, k, dtype=torch.float32, device=G.device)
    lddx = _out_rowmajor(out, "out")
    check(lib.cg_dense_gwt(_ptr(G), ldg, _ptr(W), ldw, _ptr(out), lddx, n, k, fo, _stream()), "cg_dense_gwt")
    return out


def dense_xtg(X: torch.Tensor, G: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """dW = X.T @ G; torch.mm(inputs.t(), ag) at gcn_distr.py:187."""
    X, ldx = _rowmajor(X, "X")
    G, ldg = _rowmajor(G, "G")
    n, k = X.shape
    if G.shape[0] != n:
        raise ValueError(f"X is {tuple(X.shape)}, G is {tuple(G.shape)}")
    fo = G.shape[1]
    if out is None:
        out = torch.empty(k, fo, dtype=torch.float32, device=X.device)
    lddw = _out_rowmajor(out, "out")
    check(lib.cg_dense_xtg(_ptr(X), ldx, _ptr(G), ldg, _ptr(out), lddw, n, k, fo, _stream()), "cg_dense_xtg")
    return out


# ------------------------------------------------------------------------------------------------
# activations and loss
# ------------------------------------------------------------------------------------------------
def _flat(t: torch.Tensor, name: str) -> torch.Tensor:
    t = _need(t, name, torch.float32)
    return t if t.is_contiguous() else t.contiguous()


def relu_fwd(z: torch.Tensor) -> torch.Tensor:
    z = _flat(z, "z")
    h = torch.empty_like(z)
    check(lib.cg_relu_fwd(_ptr(z), _ptr(h), z.numel(), _stream()), "cg_relu_fwd")
    return h


def relu_bwd(g: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
    g, h = _flat(g, "g"), _flat(h, "h")
    if g.shape != h.shape:
        raise ValueError("g and h differ in shape")
    dz = torch.empty_like(g)
    check(lib.cg_relu_bwd(_ptr(g), _ptr(h), _ptr(dz), g.numel(), _stream()), "cg_relu_bwd")
    return dz


def log_softmax_fwd(z: torch.Tensor) -> torch.Tensor:
    z, ldz = _rowmajor(z, "z")
    n, c = z.shape
    out = torch.empty(n, c, dtype=torch.float32, device=z.device)
    check(lib.cg_log_softmax_fwd(_ptr(z), ldz, _ptr(out), max(c, 1), n, c, _stream()), "cg_log_softmax_fwd")
    return out


def log_softmax_bwd(g: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    g, ldg = _rowmajor(g, "g")
    out, ldo = _rowmajor(out, "out")
    if g.shape != out.shape:
        raise ValueError("g and out differ in shape")
    n, c = g.shape
    dz = torch.empty(n, c, dtype=torch.float32, device=g.device)
    check(lib.cg_log_softmax_bwd(_ptr(g), ldg, _ptr(out), ldo, _ptr(dz), max(c, 1), n, c, _stream()),
          "cg_log_softmax_bwd")
    return dz


def _labels(y: torch.Tensor, n: int) -> torch.Tensor:
    y = _need(y, "y", torch.int64, 1)
    if y.numel() != n:
        raise ValueError(f"y has {y.numel()} labels for {n} rows")
    return y if y.is_contiguous() else y.contiguous()


def _mask(mask: Optional[torch.Tensor], n: int) -> Optional[torch.Tensor]:
    if mask is None:
        return None
    if mask.dtype not in (torch.bool, torch.uint8) or not mask.is_cuda or mask.dim() != 1 or mask.numel() != n:
        raise ValueError("mask must be a CUDA bool/uint8 vector with one entry per row")
    return mask if mask.is_contiguous() else mask.contiguous()


def nll_loss_fwd(logp: torch.Tensor, y: torch.Tensor, mask: Optional[torch.Tensor] = None):
    """(loss, count): loss = -mean over masked rows of logp[i, y_i] as a 0-d tensor; count = |mask| (int64, 0-d)."""
    logp, ld = _rowmajor(logp, "logp")
    n, c = logp.shape
    y, mask = _labels(y, n), _mask(mask, n)
    loss = torch.empty((), dtype=torch.float32, device=logp.device)
    count = torch.empty((), dtype=torch.int64, device=logp.device)
    check(lib.cg_nll_loss_fwd(_ptr(logp), ld, _ptr(y), _ptr(mask), n, c, c_void_p(loss.data_ptr()),
                              c_void_p(count.data_ptr()), _stream()), "cg_nll_loss_fwd")
    return loss, count


def log_softmax_nll_fwd(z: torch.Tensor, y: torch.Tensor, mask: Optional[torch.Tensor] = None):
    """(logp, loss, count) = log_softmax_fwd followed by nll_loss_fwd, in one pass over z; the loss is
    the same float the two separate calls give."""
    z, ldz = _rowmajor(z, "z")
    n, c = z.shape
    y, mask = _labels(y, n), _mask(mask, n)
    logp = torch.empty(n, c, dtype=torch.float32, device=z.device)
    loss = torch.empty((), dtype=torch.float32, device=z.device)
    count = torch.empty((), dtype=torch.int64, device=z.device)
    check(lib.cg_log_softmax_nll_fwd(_ptr(z), ldz, _ptr(y), _ptr(mask), _ptr(logp), max(c, 1), n, c,
                                     c_void_p(loss.data_ptr()), c_void_p(count.data_ptr()), _stream()),
          "cg_log_softmax_nll_fwd")
    return logp, loss, count


def nll_loss_bwd(y: torch.Tensor, mask: Optional[torch.Tensor], count: torch.Tensor, gscale: Optional[torch.Tensor],
                 n: int, c: int) -> torch.Tensor:
    y, mask = _labels(y, n), _mask(mask, n)
    d = torch.empty(n, c, dtype=torch.float32, device=y.device)
    gs = None if gscale is None else _need(gscale, "gscale", torch.float32).reshape(())
    check(lib.cg_nll_loss_bwd(_ptr(y), _ptr(mask), c_void_p(count.data_ptr()),
                              c_void_p(gs.data_ptr()) if gs is not None else c_void_p(0), _ptr(d), max(c, 1), n, c,
                              _stream()), "cg_nll_loss_bwd")
    return d


def log_softmax_nll_bwd(logp: torch.Tensor, y: torch.Tensor, mask: Optional[torch.Tensor], count: torch.Tensor,
                        gscale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """dz of mean-NLL(log_softmax(z)) given logp = log_softmax(z): gscale*mask/|mask|*(softmax - onehot)."""
    logp, ld = _rowmajor(logp, "logp")
    n, c = logp.shape
    y, mask = _labels(y, n), _mask(mask, n)
    dz = torch.empty(n, c, dtype=torch.float32, device=logp.device)
    gs = None if gscale is None else _need(gscale, "gscale", torch.float32).reshape(())
    check(lib.cg_log_softmax_nll_bwd(_ptr(logp), ld, _ptr(y), _ptr(mask), c_void_p(count.data_ptr()),
                                     c_void_p(gs.data_ptr()) if gs is not None else c_void_p(0), _ptr(dz), max(c, 1),
                                     n, c, _stream()), "cg_log_softmax_nll_bwd")
    return dz


# A wide dense operand whose rows are not a whole number of 128-byte lines long (602 floats = 2408 bytes) is read by the
# SpMM kernels through rows that start at every alignment and span 20 lines instead of 19: measured on a graph of
# 232,965 vertices with 492 entries per row, the f = 602 product takes 12.3 ms on X as it is, 12.2 ms with the rows 604
# floats apart and 11.9 ms with 608 or 640 (0.25 ms to make the copy).  A feature matrix is the same tensor in every epoch,
# so a caller can register it (`keep_aligned`): the stage loop and the drop-in `spmm_gpu` then read it through a kept copy
# with line-aligned rows.  Only registered tensors are ever copied.  The copy is remade when the tensor's version counter
# has moved; writes that do not move it (`x.data.copy_()`, DLPack or custom-kernel writers, direct calls of the C ABI)
# leave the copy stale: call `keep_aligned(x)` again or `aligned_cache_clear()` after such a write.  Tensors beyond 2 GiB
# are left alone (the copy would double them).
aligned_operands = True
_ALIGNED_MIN_COLS = 64
_ALIGNED_MAX_BYTES = 2 << 30
_aligned_cache: dict = {}   # id(tensor) -> [weakref, key, copy or None, event or None, stream the copy was made on]


def _aligned_key(t: torch.Tensor):
    return (t.data_ptr(), tuple(t.shape), tuple(t.stride()), t._version)


def _aligned_wanted(t: torch.Tensor) -> bool:
    return (aligned_operands and t.dim() == 2 and t.dtype == torch.float32 and t.is_cuda and t.shape[1] >= _ALIGNED_MIN_COLS
            and t.stride(1) == 1 and t.stride(0) % 32 != 0 and t.shape[0] > 0 and t.numel() * 4 <= _ALIGNED_MAX_BYTES)


def keep_aligned(t: torch.Tensor) -> torch.Tensor:
    """Register `t` (a dense operand that stays the same over many products, e.g. the input features) for a kept
    copy with line-aligned rows; registering again drops a copy made earlier.  Returns `t`.

    The copy is remade when `t`'s version counter, storage address, shape or strides change, i.e. after every
    in-place write through torch or this library.  A write that bypasses the version counter (`t.data`, a view of the
    storage taken under `torch.no_grad()` tricks, another process) is not seen: register only tensors you do not
    write that way, or call `keep_aligned(t)` again (or `aligned_cache_clear()`) after such a write."""
    import weakref

    _aligned_cache[id(t)] = [weakref.ref(t), None, None, None, None]
    for k in [k for k, e in _aligned_cache.items() if e[0]() is None]:
        del _aligned_cache[k]
    return t


def aligned_cache_clear() -> None:
    """Forget every registration and free the kept copies."""
    _aligned_cache.clear()


def aligned_rows(t: torch.Tensor) -> torch.Tensor:
    """`t`, or the kept copy of a registered `t` with the rows a multiple of 128 bytes apart (see `keep_aligned`)."""
    entry = _aligned_cache.get(id(t))
    if entry is None or entry[0]() is not t or not _aligned_wanted(t):
        return t
    key = _aligned_key(t)
    stream = torch.cuda.current_stream(t.device)
    if entry[1] != key or entry[2] is None:
        if torch.cuda.is_current_stream_capturing():
            return t  # no copy yet: the graph reads the caller's tensor
        ld = (t.shape[1] + 31) // 32 * 32
        with torch.no_grad():
            wide = torch.empty(t.shape[0], ld, dtype=t.dtype, device=t.device)
            wide[:, :t.shape[1]].copy_(t)
        event = torch.cuda.Event()
        event.record(stream)
        entry[1:] = [key, wide[:, :t.shape[1]], event, stream]
    elif entry[4] != stream and not torch.cuda.is_current_stream_capturing():
        stream.wait_event(entry[3])  # the copy was made on another stream
    return entry[2]
