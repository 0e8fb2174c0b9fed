"""Seeded synthetic inputs of the GCN compute path, and the reference's input preparation.

The reference reads Reddit/Amazon/Protein from files (gcn_distr.py:717-785); here graphs are
R-MAT (a, b, c, d = .57, .19, .19, .05), de-duplicated, symmetrised, with self-loops, and
normalised as D^-1/2 (A + I) D^-1/2 in the reference's own arithmetic (`gcn_normalize`).
Everything runs in torch on the device it is asked for (CPU for tests and fixtures, the GPU for
the large benchmark graphs) from explicit seeds.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch

RMAT_ABCD = (0.57, 0.19, 0.19, 0.05)


def _gen(seed: int, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    return g


def rmat_edges(scale: int, n_edges: int, seed: int, device="cpu", abcd=RMAT_ABCD) -> Tuple[torch.Tensor, torch.Tensor]:
    """n_edges directed R-MAT edges on 2^scale vertices (duplicates and self-loops included)."""
    a, b, c, _ = abcd
    g = _gen(seed, device)
    src = torch.zeros(n_edges, dtype=torch.int64, device=device)
    dst = torch.zeros(n_edges, dtype=torch.int64, device=device)
    for _level in range(scale):
        r = torch.rand(n_edges, generator=g, device=device)
        down = r >= (a + b)                       # quadrants c, d: source bit set
        right = ((r >= a) & (r < a + b)) | (r >= a + b + c)  # quadrants b, d: destination bit set
        src = (src << 1) | down.to(torch.int64)
        dst = (dst << 1) | right.to(torch.int64)
    return src, dst


def symmetric_graph_from_edges(src: torch.Tensor, dst: torch.Tensor, n: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """De-duplicate, symmetrise and add every self-loop; returns (row, col) int64 sorted by
    (row, col) -- the order torch's .coalesce() gives (gcn_distr.py:546)."""
    keep = (src < n) & (dst < n)
    src, dst = src[keep], dst[keep]
    loops = torch.arange(n, dtype=torch.int64, device=src.device)
    key = torch.cat([src * n + dst, dst * n + src, loops * n + loops])
    key = torch.unique(key)  # sorted ascending
    return key // n, key % n


def rmat_graph(scale: int, n_edges: int, seed: int, device="cpu") -> Tuple[torch.Tensor, torch.Tensor, int]:
    """(row, col, n) of the symmetrised self-looped R-MAT graph on n = 2^scale vertices."""
    n = 1 << scale
    src, dst = rmat_edges(scale, n_edges, seed, device)
    row, col = symmetric_graph_from_edges(src, dst, n)
    return row, col, n


def rmat_graph_target_nnz(n: int, target_nnz: int, seed: int, device="cpu", batch: Optional[int] = None,
                          max_rounds: int = 256) -> Tuple[torch.Tensor, torch.Tensor]:
    """R-MAT on the next power of two, vertices >= n rejected, sampled until the symmetrised,
    self-looped graph has target_nnz stored entries (within one, by parity: nnz = 2*pairs + n).
    Surplus pairs are dropped by a seeded random choice."""
    if target_nnz < n:
        raise ValueError("target_nnz must be at least n (the self-loops)")
    scale = max(1, math.ceil(math.log2(n)))
    want_pairs = (target_nnz - n) // 2
    if want_pairs > n * (n - 1) // 2:
        raise ValueError("target_nnz exceeds the complete graph")
    if batch is None:
        batch = min(1 << 25, max(1 << 14, 2 * want_pairs))
    pairs = torch.empty(0, dtype=torch.int64, device=device)  # keys lo * n + hi with lo < hi
    for rnd in range(max_rounds):
        if pairs.numel() >= want_pairs:
            break
        src, dst = rmat_edges(scale, batch, seed * 1000003 + rnd, device)
        keep = (src < n) & (dst < n) & (src != dst)
        src, dst = src[keep], dst[keep]
        lo, hi = torch.minimum(src, dst), torch.maximum(src, dst)
        pairs = torch.unique(torch.cat([pairs, lo * n + hi]))
        del src, dst, lo, hi, keep
    if pairs.numel() < want_pairs:
        raise RuntimeError(f"only {pairs.numel()} distinct pairs after {max_rounds} rounds, wanted {want_pairs}")
    if pairs.numel() > want_pairs:
        g = _gen(seed + 7919, device)
        choose = torch.randperm(pairs.numel(), generator=g, device=device)[:want_pairs]
        pairs = pairs[choose]
    lo, hi = pairs // n, pairs % n
    loops = torch.arange(n, dtype=torch.int64, device=device)
    key = torch.cat([lo * n + hi, hi * n + lo, loops * n + loops])
    key = torch.sort(key).values
    return key // n, key % n


def gcn_normalize(row: torch.Tensor, col: torch.Tensor, n: int) -> torch.Tensor:
    """fp32 values of D^-1/2 (A + I) D^-1/2 for a pattern that already holds the self-loops, in
    the arithmetic of scale_elements (gcn_distr.py:439-468): deg = entries per row, counted in
    fp64 (`histc(row.double())`), `deg.pow(-0.5)` in fp64, cast to fp32, then the unit value is
    scaled on the right (by the column's factor) and then on the left (by the row's), each product
    rounded to fp32."""
    deg = torch.bincount(row, minlength=n).to(torch.float64)
    dinv = deg.pow(-0.5).to(torch.float32)
    ones = torch.ones(row.numel(), dtype=torch.float32, device=row.device)
    right = ones * dinv[col]
    return dinv[row] * right


def block_bounds_1d(node_count: int, parts: int) -> List[int]:
    """Vertex boundaries of the 1D / 1.5D split: blocks of ceil(n/parts), the last one smaller
    (split_coo with n_per_proc = ceil(n/size), gcn_distr.py:398-400, :474)."""
    n_per_proc = math.ceil(float(node_count) / parts)
    vtx = list(range(0, node_count, n_per_proc))
    vtx.append(node_count)
    return vtx


def block_bounds_2d(node_count: int, proc_dim: int) -> List[int]:
    """Vertex boundaries of the 2D split: blocks of n // sqrt(P), the remainder goes to the last
    block (gcn_distr_2d.py:1032-1038, :1102)."""
    n_per_proc = node_count // proc_dim
    vtx = list(range(0, node_count, n_per_proc))[:proc_dim]
    vtx.append(node_count)
    return vtx


def coo_block(row: torch.Tensor, col: torch.Tensor, val: torch.Tensor, r0: int, r1: int, c0: int, c1: int):
    """Entries with r0 <= row < r1 and c0 <= col < c1, rebased to the block (split_coo,
    gcn_distr.py:404-406).  Order is preserved, so a (row, col)-sorted input stays sorted."""
    keep = (row >= r0) & (row < r1) & (col >= c0) & (col < c1)
    return row[keep] - r0, col[keep] - c0, val[keep]


def glorot_uniform(fan_in: int, fan_out: int, seed: int, device="cpu") -> torch.Tensor:
    bound = math.sqrt(6.0 / (fan_in + fan_out))
    g = _gen(seed, device)
    return (torch.rand(fan_in, fan_out, generator=g, device=device, dtype=torch.float32) * 2.0 - 1.0) * bound


def normal_features(n: int, f: int, seed: int, device="cpu") -> torch.Tensor:
    return torch.randn(n, f, generator=_gen(seed, device), device=device, dtype=torch.float32)


def uniform_labels(n: int, classes: int, seed: int, device="cpu") -> torch.Tensor:
    return torch.randint(0, classes, (n,), generator=_gen(seed, device), device=device, dtype=torch.int64)


def random_mask(n: int, fraction: float, seed: int, device="cpu") -> torch.Tensor:
    return torch.rand(n, generator=_gen(seed, device), device=device) < fraction


@dataclass
class GcnProblem:
    """One seeded instance: normalised graph in sorted COO, features, labels, mask, Glorot weights."""
    n: int
    row: torch.Tensor   # int64, sorted by (row, col)
    col: torch.Tensor   # int64
    val: torch.Tensor   # fp32
    x: torch.Tensor
    y: torch.Tensor
    train_mask: torch.Tensor
    w1: torch.Tensor
    w2: torch.Tensor
    seeds: dict

    @property
    def nnz(self) -> int:
        return int(self.val.numel())


def make_problem(*, scale: Optional[int] = None, n_edges: Optional[int] = None, n: Optional[int] = None,
                 target_nnz: Optional[int] = None, features: int, hidden: int, classes: int,
                 mask_fraction: float = 1.0, seed: int = 0, device="cpu") -> GcnProblem:
    seeds = {"graph": seed * 10 + 1, "x": seed * 10 + 2, "y": seed * 10 + 3, "mask": seed * 10 + 4,
             "w1": seed * 10 + 5, "w2": seed * 10 + 6}
    if scale is not None:
        row, col, n = rmat_graph(scale, int(n_edges), seeds["graph"], device)
    else:
        row, col = rmat_graph_target_nnz(int(n), int(target_nnz), seeds["graph"], device)
    val = gcn_normalize(row, col, n)
    x = normal_features(n, features, seeds["x"], device)
    y = uniform_labels(n, classes, seeds["y"], device)
    if mask_fraction >= 1.0:
        mask = torch.ones(n, dtype=torch.bool, device=device)
    else:
        mask = random_mask(n, mask_fraction, seeds["mask"], device)
    w1 = glorot_uniform(features, hidden, seeds["w1"], device)
    w2 = glorot_uniform(hidden, classes, seeds["w2"], device)
    return GcnProblem(n, row, col, val, x, y, mask, w1, w2, seeds)
