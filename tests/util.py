"""Helpers shared by the parity tests: seeded small problems and oracle-side conversions."""
from __future__ import annotations

import numpy as np
import torch

from cagnet_amd import synth
from oracle import gcn_oracle as orc

# north_star tolerance: max relative error 1e-5 in fp32, measured against the row-sum magnitude
REL_TOL = 1e-5
LOSS_TOL = 1e-4


def small_graph(scale: int, n_edges: int, seed: int):
    row, col, n = synth.rmat_graph(scale, n_edges, seed)
    val = synth.gcn_normalize(row, col, n)
    return row, col, val, n


def random_coo(n: int, m: int, nnz: int, seed: int, sort: bool = True):
    """Duplicate-free random COO with N(0,1) values (general, non-symmetric, rectangular)."""
    rng = np.random.default_rng(seed)
    nnz = min(nnz, n * m)
    key = rng.choice(n * m, size=nnz, replace=False) if n * m < (1 << 26) else np.unique(
        rng.integers(0, n * m, size=nnz))
    if sort:
        key = np.sort(key)
    row = torch.from_numpy((key // m).astype(np.int64))
    col = torch.from_numpy((key % m).astype(np.int64))
    val = torch.from_numpy(rng.standard_normal(key.size).astype(np.float32))
    return row, col, val


def spmm_error(got: torch.Tensor, row, col, val, n, m, B, C0=None) -> float:
    """max |got - ref64| / sum_j |a_ij||b_jk| with ref64 the fp64 oracle of C0 + A B."""
    B64 = B.detach().cpu().double()
    C64 = torch.zeros(n, B.shape[1], dtype=torch.float64) if C0 is None else C0.detach().cpu().double()
    ref = orc.spmm(row.cpu(), col.cpu(), val.cpu(), n, m, B64, C64, torch.float64)
    mag = orc.spmm_abs(row.cpu(), col.cpu(), val.cpu(), n, m, B64) + C64.abs()
    return orc.max_rel_error(got, ref, mag)


def gemm_error(got: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> float:
    a64, b64 = a.detach().cpu().double(), b.detach().cpu().double()
    return orc.max_rel_error(got, a64 @ b64, a64.abs() @ b64.abs())
