"""The C ABI without a GPU: the library loads, exports every symbol the header declares, the
Python binding covers the same set, and argument validation answers with distinct status codes
before any device work."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "cagnet_amd.h"


def _declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(cg_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from cagnet_amd import _lib
    names = _declared()
    assert len(names) >= 25
    raw = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in names:
        assert hasattr(raw, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == names, "binding and header disagree"
    assert _lib.lib.cg_abi_version() == 1


def test_every_declaration_cites_the_reference_or_says_it_has_no_counterpart():
    text = HEADER.read_text()
    assert "sparse-extension/sparse_coo_tensor.cu:113-240" in text     # spmm_gpu
    assert "sparse_coo_tensor.cu:136-142" in text                      # coo2csr
    assert "gcn_distr.py:275" in text and "gcn_distr.py:284-294" in text  # dense products, activations and loss
    assert "gcn_distr.py:791" in text and "gcn_distr.py:412-470" in text and "gcn_distr.py:398-409" in text  # preparation
    assert "gcn_distr.py:747" in text and "gcn_distr_2d.py:369-374" in text  # block format


def test_header_is_plain_c_and_cplusplus(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 and as C++11 with nothing but <stdint.h>."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("gcc not available")
    src = tmp_path / "use.c"
    src.write_text('#include "cagnet_amd.h"\nint main(void) { return cg_abi_version() == CG_ABI_VERSION ? 0 : 1; }\n')
    inc = str(HEADER.parent)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-I", inc, str(src)],
                   check=True)
    subprocess.run(["g++", "-std=c++11", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", "-I", inc, str(src)], check=True)


def test_status_codes_without_a_gpu():
    from cagnet_amd._lib import lib
    null = None
    one = ctypes.c_void_p(16)  # never dereferenced: validation comes first
    E = {"null": 1, "size": 2, "overflow": 3, "unsupported": 8}
    assert lib.cg_spmm_coo(null, null, null, -1, 4, 4, one, 4, one, 4, 4, 1.0, null) == E["size"]
    assert lib.cg_spmm_coo(null, null, null, 1 << 31, 4, 4, one, 4, one, 4, 4, 1.0, null) == E["overflow"]
    assert lib.cg_spmm_coo(null, null, null, 5, 4, 4, one, 4, one, 4, 4, 1.0, null) == E["null"]
    assert lib.cg_spmm_coo(one, one, one, 5, 4, 4, one, 3, one, 4, 4, 1.0, null) == E["size"]      # ldb < f
    assert lib.cg_spmm_coo(one, one, one, 5, 4, 4, one, 4, one, 4, 0, 1.0, null) == E["size"]      # f == 0
    assert lib.cg_spmm_coo(one, one, one, 5, 4, 4, one, 4, one, 4, 4, 1.0, null) == 10             # C aliases B
    # the block-cache form checks the same things before it touches the device
    assert lib.cg_spmm_coo_cached(null, null, null, -1, 4, 4, one, 4, one, 4, 4, 1.0, null) == E["size"]
    assert lib.cg_spmm_coo_cached(null, null, null, 1 << 31, 4, 4, one, 4, one, 4, 4, 1.0, null) == E["overflow"]
    assert lib.cg_spmm_coo_cached(null, null, null, 5, 4, 4, one, 4, one, 4, 4, 1.0, null) == E["null"]
    assert lib.cg_spmm_coo_cached(one, one, one, 5, 4, 4, one, 3, one, 4, 4, 1.0, null) == E["size"]
    assert lib.cg_coo_cache_info(None) == E["null"]
    assert lib.cg_coo_cache_clear() == 0
    assert lib.cg_spmm_coo_cached(one, one, one, 5, 4, 4, one, 4, one, 4, 4, 1.0, null) == 10
    assert b"alias" in lib.cg_last_error()
    h = ctypes.c_void_p(0)
    assert lib.cg_csr_create(ctypes.byref(h), null, null, null, 3, 4, 4, 1, null) == E["null"]
    assert lib.cg_csr_create(None, one, one, one, 3, 4, 4, 1, null) == E["null"]
    assert lib.cg_csr_create(ctypes.byref(h), one, one, one, (1 << 31) - 1, 4, 4, 1, null) == E["overflow"]
    assert lib.cg_csr_create(ctypes.byref(h), one, one, one, 3, 0x7fffffff, 4, 1, null) == E["overflow"]
    assert lib.cg_csr_create(ctypes.byref(h), one, one, one, 3, 0, 4, 1, null) == E["size"]
    assert lib.cg_csr_spmm(null, 0, one, 4, one, 4, 4, 0.0, null) == E["null"]
    assert lib.cg_csr_destroy(null) == 0
    assert lib.cg_coo2csr_rowptr(null, 3, 4, one, null) == E["null"]
    assert lib.cg_coo2csr_rowptr(one, -3, 4, one, null) == E["size"]
    assert lib.cg_coo2csr(one, one, one, 3, 4, 4, one, one, null, null, null) == E["null"]     # values without output
    assert lib.cg_dense_xw(one, 4, one, 4, one, 4, 10, 0, 4, 0, null) == E["size"]
    assert lib.cg_dense_xw(one, 3, one, 4, one, 4, 10, 4, 4, 0, null) == E["size"]              # ldx < k
    assert lib.cg_dense_gwt(null, 4, one, 4, one, 4, 10, 4, 4, null) == E["null"]
    assert lib.cg_dense_xtg(one, 4, one, 4, null, 4, 10, 4, 4, null) == E["null"]
    assert lib.cg_relu_fwd(one, one, -1, null) == E["size"]
    assert lib.cg_relu_fwd(null, one, 5, null) == E["null"]
    assert lib.cg_log_softmax_fwd(one, 3, one, 4, 10, 4, null) == E["size"]
    assert lib.cg_nll_loss_fwd(one, 4, one, null, 10, 4, null, one, null) == E["null"]
    count = ctypes.c_int64(-1)
    assert lib.cg_add_self_loops(null, null, 5, 4, null, null, 0, ctypes.byref(count), null) == E["null"]
    assert lib.cg_add_self_loops(one, one, 5, 4, null, null, 0, None, null) == E["null"]
    assert lib.cg_add_self_loops(one, one, -1, 4, null, null, 0, ctypes.byref(count), null) == E["size"]
    assert lib.cg_gcn_normalize(one, one, 1 << 31, 4, one, null, null) == E["overflow"]
    assert lib.cg_gcn_normalize(one, null, 5, 4, one, null, null) == E["null"]
    assert lib.cg_coo_block(one, one, null, 5, 3, 2, 0, 4, null, null, null, 0, ctypes.byref(count), null) == E["size"]
    assert lib.cg_coo_block(one, one, null, 0, 0, 2, 0, 4, null, null, null, 0, ctypes.byref(count), null) == 0
    assert count.value == 0
    h2 = ctypes.c_void_p(0)
    junk = (ctypes.c_uint8 * 256)()
    assert lib.cg_csr_blob_read(ctypes.byref(h2), junk, 256, 0, null) == E["unsupported"]        # bad magic
    assert lib.cg_csr_blob_read(ctypes.byref(h2), junk, 64, 0, null) == E["size"]                # no room for a header
    assert lib.cg_csr_blob_read(ctypes.byref(h2), null, 256, 0, null) == E["null"]
    assert lib.cg_csr_blob_size(null, ctypes.byref(count)) == E["null"]
    assert lib.cg_tune_set(b"no_such_knob", 1) == E["unsupported"]
    assert lib.cg_tune_set(b"spmm_seg", 0) == 0
    for key in (b"spmm_hub_row", b"coo_cache_blocks", b"dense_mfma"):
        assert lib.cg_tune_set(key, 0) == 0
    for code in range(0, 11):
        assert lib.cg_status_string(code) not in (None, b"unknown status")
    assert lib.cg_status_string(99) == b"unknown status"


def test_python_surface_rejects_cpu_tensors_and_wrong_types():
    import torch
    from cagnet_amd import ops
    from cagnet_amd.sparse_coo_tensor_cpp import sparse_coo_tensor_gpu, spmm_gpu
    i = torch.zeros(3, dtype=torch.int32)
    v = torch.zeros(3)
    with pytest.raises(ValueError, match="no CPU path"):
        spmm_gpu(i, i, v, 4, 4, torch.zeros(4, 2), torch.zeros(4, 2))
    with pytest.raises(ValueError, match="no CPU path"):
        ops.dense_xw(torch.zeros(4, 2), torch.zeros(2, 2))
    with pytest.raises(ValueError, match="no CPU path"):
        ops.CsrMatrix(i, i, v, 4, 4)
    t = sparse_coo_tensor_gpu(torch.tensor([[0, 1], [1, 0]]), torch.tensor([1.0, 2.0]), (2, 2))
    assert t.is_sparse and t.shape == (2, 2) and float(t.to_dense()[0, 1]) == 1.0
    import sparse_coo_tensor_cpp as shim  # the reference's module name resolves from the repo root
    assert shim.spmm_gpu is spmm_gpu
    from cagnet_amd import sparse_coo_tensor_cpp as mod
    assert mod.cache_blocks is True      # blocks seen before are recognised by default


def _host_driver():
    """The ASan + UBSan build of the library's host code and its driver (tests/abi_host_driver.cpp); built here
    only when nothing is there yet."""
    from cagnet_amd import build
    if not build.SAN_DRIVER_PATH.exists() or not build.SAN_LIB_PATH.exists():
        build.build_host_driver()
    return build.SAN_DRIVER_PATH


def run_host_driver(*args):
    import os
    import subprocess
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([str(_host_driver()), *args], capture_output=True, text=True, timeout=600, env=env)
    report = proc.stdout[-3000:] + proc.stderr[-6000:]
    assert proc.returncode == 0, report
    assert "AddressSanitizer" not in proc.stderr and "runtime error:" not in proc.stderr, report
    assert "abi_host_driver: ok" in proc.stdout


def test_host_code_under_address_and_ub_sanitizers():
    """Argument checks, status strings, tuning keys, blob header parsing and the recorder of the library,
    compiled with -fsanitize=address,undefined on the host side, driven by a sanitized C++ program: no GPU is
    needed for these paths.  (Leak checking is off: the HIP runtime keeps its own allocations until exit.)"""
    run_host_driver()
