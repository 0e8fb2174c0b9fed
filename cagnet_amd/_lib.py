"""ctypes binding of libcagnet_amd.so (the C ABI declared in include/cagnet_amd.h).

There is exactly one implementation behind these calls: the HIP library.  If it has not been built
the import of this module raises; nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_uint32, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libcagnet_amd.so"

CG_OK = 0
CG_CSR_SORTED = 1
CG_CSR_TRANSPOSE = 2
CG_CSR_VALIDATE = 4

CG_ERR_UNSUPPORTED = 8
STATUS_NAMES = {
    0: "CG_OK", 1: "CG_ERR_NULL", 2: "CG_ERR_SIZE", 3: "CG_ERR_OVERFLOW", 4: "CG_ERR_UNSORTED",
    5: "CG_ERR_INDEX", 6: "CG_ERR_HIP", 7: "CG_ERR_ALLOC", 8: "CG_ERR_UNSUPPORTED",
    9: "CG_ERR_NO_TRANSPOSE", 10: "CG_ERR_ALIAS", 11: "CG_ERR_CAPTURE",
}


class CagnetError(RuntimeError):
    """A non-zero cg_status.  The reference prints such errors and continues
    (sparse-extension/sparse_coo_tensor.cu:20-30); here they raise."""

    def __init__(self, status: int, detail: str, where: str):
        self.status = status
        name = STATUS_NAMES.get(status, str(status))
        super().__init__(f"{where}: {name}: {detail}")


P = c_void_p  # every device pointer travels as void*

# name -> (argtypes); every entry point returns int unless listed in _RESTYPES
_SIGNATURES = {
    "cg_abi_version": [],
    "cg_status_string": [c_int],
    "cg_last_error": [],
    "cg_coo2csr_rowptr": [P, c_int64, c_int32, P, P],
    "cg_coo_check": [P, P, c_int64, c_int32, c_int32, c_int, P],
    "cg_coo2csr": [P, P, P, c_int64, c_int32, c_int32, P, P, P, P, P],
    "cg_csr_transpose": [P, P, P, c_int64, c_int32, c_int32, P, P, P, P, P],
    "cg_spmm_coo": [P, P, P, c_int64, c_int32, c_int32, P, c_int64, P, c_int64, c_int32, c_float, P],
    "cg_spmm_coo_cached": [P, P, P, c_int64, c_int32, c_int32, P, c_int64, P, c_int64, c_int32, c_float, P],
    "cg_coo_cache_clear": [],
    "cg_coo_cache_info": [POINTER(c_int64)],
    "cg_csr_create": [POINTER(c_void_p), P, P, P, c_int64, c_int32, c_int32, c_uint32, P],
    "cg_csr_destroy": [P],
    "cg_csr_unpin": [P, POINTER(c_int64)],
    "cg_csr_hstack": [POINTER(P), POINTER(P), c_int32, c_uint32, P],
    "cg_scratch_release": [P, POINTER(c_int64)],
    "cg_csr_spmm": [P, c_int, P, c_int64, P, c_int64, c_int32, c_float, P],
    "cg_csr_spmm_xw": [P, c_int, P, c_int64, P, c_int64, c_float, P, c_int64, P, c_int64, c_int32, c_int32, c_int, P],
    "cg_csr_info": [P, POINTER(c_int64)],
    "cg_csr_panel_info": [P, c_int, POINTER(c_int64)],
    "cg_csr_arrays": [P, c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p)],
    "cg_dense_xw": [P, c_int64, P, c_int64, P, c_int64, c_int64, c_int32, c_int32, c_int, P],
    "cg_dense_gwt": [P, c_int64, P, c_int64, P, c_int64, c_int64, c_int32, c_int32, P],
    "cg_dense_xtg": [P, c_int64, P, c_int64, P, c_int64, c_int64, c_int32, c_int32, P],
    "cg_relu_fwd": [P, P, c_int64, P],
    "cg_relu_bwd": [P, P, P, c_int64, P],
    "cg_log_softmax_fwd": [P, c_int64, P, c_int64, c_int64, c_int32, P],
    "cg_log_softmax_bwd": [P, c_int64, P, c_int64, P, c_int64, c_int64, c_int32, P],
    "cg_nll_loss_fwd": [P, c_int64, P, P, c_int64, c_int32, P, P, P],
    "cg_nll_loss_fwd_static": [P, c_int64, P, P, c_int64, c_int32, P, P, P],
    "cg_nll_loss_bwd": [P, P, P, P, P, c_int64, c_int64, c_int32, P],
    "cg_log_softmax_nll_bwd": [P, c_int64, P, P, P, P, P, c_int64, c_int64, c_int32, P],
    "cg_log_softmax_nll_fwd": [P, c_int64, P, P, P, c_int64, c_int64, c_int32, P, P, P],
    "cg_csr_blob_size": [P, POINTER(c_int64)],
    "cg_csr_blob_write": [P, P, c_int64, P],
    "cg_csr_blob_read": [POINTER(c_void_p), P, c_int64, c_uint32, P],
    "cg_add_self_loops": [P, P, c_int64, c_int32, P, P, c_int64, POINTER(c_int64), P],
    "cg_gcn_normalize": [P, P, c_int64, c_int32, P, P, P],
    "cg_coo_block": [P, P, P, c_int64, c_int32, c_int32, c_int32, c_int32, P, P, P, c_int64, POINTER(c_int64), P],
    "cg_prof_enable": [c_int],
    "cg_tune_set": [c_char_p, c_int],
    "cg_prof_read": [c_char_p, POINTER(ctypes.c_double), POINTER(c_int64)],
}
_RESTYPES = {"cg_status_string": c_char_p, "cg_last_error": c_char_p}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def _load() -> ctypes.CDLL:
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m cagnet_amd.build` (hipcc, gfx950). "
            "cagnet_amd has no other backend."
        )
    # One HIP runtime per process: torch ships its own libamdhip64.so.7, and the device pointers and
    # streams handed to the library come from it.  Importing torch first makes the dynamic linker
    # resolve the library's libamdhip64.so.7 dependency to that already loaded copy.
    import torch  # noqa: F401

    lib = ctypes.CDLL(str(LIB_PATH))
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, c_int)
    return lib


lib = _load()


def check(status: int, where: str) -> None:
    if status != CG_OK:
        detail = lib.cg_last_error().decode("utf-8", "replace")
        raise CagnetError(status, detail, where)
