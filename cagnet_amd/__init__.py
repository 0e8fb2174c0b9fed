"""cagnet_amd: the per-rank GCN compute path of CAGNET (local coo2csr + accumulate-SpMM + H*W +
ReLU / log_softmax+NLL, forward and backward) on one AMD Instinct MI355X (gfx950).

Submodules
    ops                    tensor-level wrappers over the C ABI of lib/libcagnet_amd.so
    sparse_coo_tensor_cpp  the reference's native module, name for name (spmm_gpu, ...)
    gcn                    broad_func / GCNFunc / train of the reference, restated for one GPU
    synth                  seeded synthetic graphs and the reference's input preparation (pure torch)
    build                  hipcc recipe of the library

`ops`, `gcn` and `sparse_coo_tensor_cpp` need the built library and raise ImportError without it;
there is no other backend.
"""
__version__ = "0.1.0"

_LAZY = ("ops", "gcn", "sparse_coo_tensor_cpp", "synth", "build", "_lib")


def __getattr__(name):
    if name in _LAZY:
        import importlib

        return importlib.import_module(f"{__name__}.{name}")
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
