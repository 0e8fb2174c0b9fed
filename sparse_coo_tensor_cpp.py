"""Import shim: lets CAGNET's drivers keep `from sparse_coo_tensor_cpp import spmm_gpu, ...`
(gcn_distr.py:27) when this directory is on sys.path."""
from cagnet_amd.sparse_coo_tensor_cpp import coo2csr, sparse_coo_tensor_gpu, spmm_gpu  # noqa: F401

__all__ = ["spmm_gpu", "sparse_coo_tensor_gpu", "coo2csr"]
