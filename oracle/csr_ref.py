"""ctypes loader of oracle/_build/libcsr_ref.so (oracle/csr_ref.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import c_float, c_int, c_int32, c_int64, c_void_p
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
LIB_PATH = _DIR / "_build" / "libcsr_ref.so"


def build(force: bool = False) -> Path:
    if force or not LIB_PATH.exists() or LIB_PATH.stat().st_mtime < (_DIR / "csr_ref.c").stat().st_mtime:
        subprocess.run(["make", "-C", str(_DIR), "-B" if force else "-s", "all"], check=True, capture_output=True)
    return LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(str(LIB_PATH))
        _lib.ref_coo2csr_rowptr.argtypes = [c_void_p, c_int64, c_int32, c_void_p]
        _lib.ref_csr_spmm.argtypes = [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_int64, c_void_p,
                                      c_int64, c_int32, c_float, c_int]
        _lib.ref_csr_transpose.argtypes = [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p,
                                           c_void_p, c_void_p]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(c_void_p)


def coo2csr_rowptr(row: np.ndarray, n: int) -> np.ndarray:
    row = np.ascontiguousarray(row, dtype=np.int32)
    out = np.empty(n + 1, dtype=np.int32)
    lib().ref_coo2csr_rowptr(_p(row), row.size, n, _p(out))
    return out


def csr_spmm(rowptr, colind, val, n: int, m: int, B: np.ndarray, C: np.ndarray, beta: float = 1.0,
             wide: bool = False) -> np.ndarray:
    rowptr = np.ascontiguousarray(rowptr, dtype=np.int32)
    colind = np.ascontiguousarray(colind, dtype=np.int32)
    val = np.ascontiguousarray(val, dtype=np.float32)
    B = np.ascontiguousarray(B, dtype=np.float32)
    out = np.array(C, dtype=np.float32, order="C", copy=True)
    f = B.shape[1]
    rc = lib().ref_csr_spmm(_p(rowptr), _p(colind), _p(val), n, m, _p(B), f, _p(out), f, f, float(beta), int(wide))
    if rc:
        raise MemoryError("ref_csr_spmm")
    return out


def csr_transpose(rowptr, colind, val, n: int, m: int):
    rowptr = np.ascontiguousarray(rowptr, dtype=np.int32)
    colind = np.ascontiguousarray(colind, dtype=np.int32)
    nnz = int(rowptr[n])
    valc = None if val is None else np.ascontiguousarray(val, dtype=np.float32)
    colptr = np.empty(m + 1, dtype=np.int32)
    rowind = np.empty(nnz, dtype=np.int32)
    val_t = None if val is None else np.empty(nnz, dtype=np.float32)
    perm = np.empty(nnz, dtype=np.int32)
    rc = lib().ref_csr_transpose(_p(rowptr), _p(colind), _p(valc), n, m, _p(colptr), _p(rowind), _p(val_t), _p(perm))
    if rc:
        raise MemoryError("ref_csr_transpose")
    return colptr, rowind, val_t, perm
