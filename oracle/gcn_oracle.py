"""CPU oracle of CAGNET's per-rank GCN compute path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this module;
it is the checker, never the product: nothing under cagnet_amd/ imports it.

It restates, on stock PyTorch / NumPy / SciPy on the CPU, the arithmetic the reference performs
through cuSPARSE, PyTorch 1.3.1 and torch_sparse (none of which ships in the reference tree, and
the reference has no tests or golden vectors, so this is an independent restatement):

  coo2csr_rowptr   cusparseXcoo2csr            sparse-extension/sparse_coo_tensor.cu:136-142
  coo2csr          coalesced (row, col) order  gcn_distr.py:546 (+ the compression above)
  csr_transpose    (the A^T the reference never builds; it reuses A, gcn_distr.py:326)
  spmm             spmm_gpu, C += A B          sparse-extension/sparse_coo_tensor.cu:113-240
                   == the torch.sparse line the reference keeps commented, gcn_distr_3d.py:478
  stage_schedule_15d  stages of a rank         gcn_distr_15d.py:194-208
  stage_loop       broad_func                  gcn_distr.py:203-246 (1.5D: gcn_distr_15d.py:197-234,
                                               2D: gcn_distr_2d.py:333-417), broadcasts removed
  GCNFuncOracle    GCNFunc                     gcn_distr.py:248-339
  train_epoch      train                       gcn_distr.py:341-366
  gcn_normalize    scale_elements              gcn_distr.py:412-470
  add_self_loops   add_remaining_self_loops    gcn_distr.py:791 (+ coalesce, :546)
  block_bounds_*   split_coo / partitions      gcn_distr.py:398-409, gcn_distr_2d.py:1032-1047, :1102

How each function is pinned (tests/test_oracle.py): coo2csr/transpose against
scipy.sparse tocsr()/tocsc() and torch .coalesce()/.to_sparse_csr() and a lower_bound closed
form; spmm against scipy CSR @ dense, a dense matmul and hand-computed special cases (identity,
single row, empty rows); GCNFunc's hand-written backward against torch autograd over the same
forward and torch.autograd.gradcheck in fp64; the loss against F.nll_loss on gathered rows; the
normalisation against a dense D^-1/2 (A+I) D^-1/2 in fp64 and its symmetry; self-loops against
scipy's (A - diag(A) + I) pattern; block bounds and block extraction against brute-force
enumeration and scipy slicing.  No function of this oracle is "parity unpinned".

Every routine takes `dtype` (torch.float32 for the reference's arithmetic, torch.float64 for the
error yardstick both the GPU result and the fp32 CPU result are measured against).
"""
from __future__ import annotations

import math
import struct
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F


# ------------------------------------------------------------------------------------------------
# integer part: CSR construction
# ------------------------------------------------------------------------------------------------
def coo2csr_rowptr(row: np.ndarray, n: int) -> np.ndarray:
    """rowptr[i] = number of entries with row index < i (cusparseXcoo2csr, base 0), int32[n+1].
    Computed by counting (a histogram and a running sum), not by searching."""
    row = np.asarray(row)
    counts = np.bincount(row.astype(np.int64), minlength=n) if row.size else np.zeros(n, dtype=np.int64)
    if counts.size > n:
        raise ValueError("row index >= n")
    out = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(counts, out=out[1:])
    return out.astype(np.int32)


def coo2csr(row: np.ndarray, col: np.ndarray, val: Optional[np.ndarray], n: int, m: int):
    """(rowptr, colind, values, perm): entries ordered by (row, col), ties in input order;
    duplicates are kept.  perm[k] = input position of output entry k."""
    row, col = np.asarray(row, dtype=np.int64), np.asarray(col, dtype=np.int64)
    if row.size and (row.min() < 0 or row.max() >= n or col.min() < 0 or col.max() >= m):
        raise ValueError("index out of range")
    perm = np.lexsort((col, row)).astype(np.int32)  # stable; last key is the primary one
    rowptr = coo2csr_rowptr(row[perm], n)
    colind = col[perm].astype(np.int32)
    values = None if val is None else np.asarray(val)[perm]
    return rowptr, colind, values, perm


def csr_expand_rows(rowptr: np.ndarray) -> np.ndarray:
    rowptr = np.asarray(rowptr, dtype=np.int64)
    return np.repeat(np.arange(rowptr.size - 1, dtype=np.int64), np.diff(rowptr))


def csr_transpose(rowptr: np.ndarray, colind: np.ndarray, values: Optional[np.ndarray], n: int, m: int):
    """CSR of A^T (== CSC of A): (colptr, rowind, values_t, perm), rows ascending inside a column."""
    rows = csr_expand_rows(rowptr)
    colind = np.asarray(colind, dtype=np.int64)
    perm = np.argsort(colind, kind="stable").astype(np.int32)
    colptr = coo2csr_rowptr(colind[perm], m)
    rowind = rows[perm].astype(np.int32)
    values_t = None if values is None else np.asarray(values)[perm]
    return colptr, rowind, values_t, perm


# ------------------------------------------------------------------------------------------------
# SpMM and the stage loop
# ------------------------------------------------------------------------------------------------
def coo_tensor(row, col, val, n: int, m: int, dtype=torch.float32) -> torch.Tensor:
    """The tensor type the reference keeps a sparse block in (gcn_distr.py:493-512): coalesced COO."""
    idx = torch.stack([torch.as_tensor(row, dtype=torch.int64), torch.as_tensor(col, dtype=torch.int64)])
    v = torch.as_tensor(val).to(dtype)
    return torch.sparse_coo_tensor(idx, v, (n, m)).coalesce()


def spmm(row, col, val, n: int, m: int, B: torch.Tensor, C: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    """Returns C + A @ B (the reference operator accumulates into C: alpha = beta = 1,
    sparse_coo_tensor.cu:149-150), computed with torch.sparse.mm in `dtype`."""
    A = coo_tensor(row, col, val, n, m, dtype)
    return C.to(dtype) + torch.sparse.mm(A, B.to(dtype))


def spmm_abs(row, col, val, n: int, m: int, B: torch.Tensor) -> torch.Tensor:
    """Row-sum magnitude sum_j |a_ij| |b_jk| in fp64: the denominator of the SpMM error metric."""
    A = coo_tensor(row, col, np.abs(np.asarray(val, dtype=np.float64)), n, m, torch.float64)
    return torch.sparse.mm(A, B.to(torch.float64).abs())


def stage_loop(blocks: Sequence[torch.Tensor], dense: Sequence[torch.Tensor], dtype=torch.float32) -> torch.Tensor:
    """z_loc = sum_i blocks[i] @ dense[i]: z_loc starts at zero and every stage accumulates
    (gcn_distr.py:215, :221-244).  blocks are sparse COO tensors."""
    z = torch.zeros(blocks[0].shape[0], dense[0].shape[1], dtype=dtype)
    for a, h in zip(blocks, dense):
        z = z + torch.sparse.mm(a.to(dtype), h.to(dtype))
    return z


def stage_schedule_15d(rank: int, size: int, replication: int):
    """(source rank, block id) per stage of a rank in the 1.5D algorithm, restated from
    gcn_distr_15d.py:194-208: stages = P // c^2, the last replica column takes the remainder
    (:197-199); q = (rank_col * (P // c^2) + i) * c + rank_col (:204); block id = q // c (:208)."""
    rank_col = rank % replication
    stages = size // replication ** 2
    if rank_col == replication - 1:
        stages = size // replication - (replication - 1) * stages
    sched = []
    for i in range(stages):
        q = (rank_col * (size // replication ** 2) + i) * replication + rank_col
        sched.append((q, rank_col * (size // replication ** 2) + i))
    return sched


# ------------------------------------------------------------------------------------------------
# GCNFunc and train
# ------------------------------------------------------------------------------------------------
def _activation(z: torch.Tensor, kind: str) -> torch.Tensor:
    if kind == "relu":
        return F.relu(z)
    if kind == "log_softmax":
        return F.log_softmax(z, dim=1)
    return z


class GCNFuncOracle(torch.autograd.Function):
    """GCNFunc (gcn_distr.py:248-339) on CPU tensors.  forward: Z = (sum_i A_i H_i) W, h = func(Z).
    backward: G' = func'(Z) * G by re-running func under autograd (:312-322); AG = sum_i A'_i G'_i
    (:326; A'_i = blocks_bwd[i], which the reference takes to be the same blocks); dH = AG W^T
    (:330); dW = H^T AG (:337)."""

    @staticmethod
    def forward(ctx, inputs, weight, blocks_fwd, blocks_bwd, peers_fwd, peers_bwd, rank, kind):
        ctx.save_for_backward(inputs, weight)
        ctx.blocks_bwd, ctx.peers_bwd, ctx.rank, ctx.kind = blocks_bwd, peers_bwd, rank, kind
        dense = [inputs if i == rank else peers_fwd[i] for i in range(len(blocks_fwd))]
        z = stage_loop(blocks_fwd, dense, inputs.dtype)
        z = torch.mm(z, weight)
        ctx.z = z
        return _activation(z, kind)

    @staticmethod
    def backward(ctx, grad_output):
        inputs, weight = ctx.saved_tensors
        z = ctx.z.detach().requires_grad_(True)
        with torch.enable_grad():
            func_eval = _activation(z, ctx.kind)
            sigmap = torch.autograd.grad(outputs=func_eval, inputs=z, grad_outputs=grad_output)[0]
        dense = [sigmap if i == ctx.rank else ctx.peers_bwd[i] for i in range(len(ctx.blocks_bwd))]
        ag = stage_loop(ctx.blocks_bwd, dense, inputs.dtype)
        grad_input = torch.mm(ag, weight.t())
        grad_weight = torch.mm(inputs.t(), ag)
        return grad_input, grad_weight, None, None, None, None, None, None


def gcn_layer(inputs, weight, blocks_fwd, kind, blocks_bwd=None, peers_fwd=None, peers_bwd=None, rank=0):
    blocks_bwd = blocks_fwd if blocks_bwd is None else blocks_bwd
    return GCNFuncOracle.apply(inputs, weight, blocks_fwd, blocks_bwd, peers_fwd, peers_bwd, rank, kind)


def masked_nll(outputs: torch.Tensor, y: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    """F.nll_loss(outputs[mask], y[mask]) (gcn_distr.py:356); with an empty mask the reference
    back-propagates (outputs * 0).sum() instead (:359-362), i.e. loss 0 and zero gradients."""
    if mask is None:
        return F.nll_loss(outputs, y)
    if int(mask.sum()) == 0:
        return (outputs * torch.zeros_like(outputs)).sum()
    return F.nll_loss(outputs[mask], y[mask])


def forward_backward(x, w1, w2, blocks_fwd, y, mask, blocks_bwd=None, dtype=torch.float32,
                     peers1=(None, None), peers2=(None, None), rank=0, x_requires_grad=True):
    """One forward + backward of the 2-layer model of train (gcn_distr.py:342-358): returns
    dict(loss, outputs, hidden, dw1, dw2, dx)."""
    def cast(t):
        return None if t is None else [None if b is None else b.to(dtype) for b in t]

    x = x.to(dtype).clone().requires_grad_(x_requires_grad)
    w1 = w1.to(dtype).clone().requires_grad_(True)
    w2 = w2.to(dtype).clone().requires_grad_(True)
    bf = [b.to(dtype) for b in blocks_fwd]
    bb = bf if blocks_bwd is None else [b.to(dtype) for b in blocks_bwd]
    h = gcn_layer(x, w1, bf, "relu", bb, cast(peers1[0]), cast(peers1[1]), rank)
    out = gcn_layer(h, w2, bf, "log_softmax", bb, cast(peers2[0]), cast(peers2[1]), rank)
    loss = masked_nll(out, y, mask)
    loss.backward()
    return {"loss": loss.detach(), "outputs": out.detach(), "hidden": h.detach(), "dw1": w1.grad, "dw2": w2.grad,
            "dx": x.grad}


def train_epochs(x, w1, w2, blocks_fwd, y, mask, epochs: int, lr: float = 0.01, optimizer: str = "sgd",
                 blocks_bwd=None, dtype=torch.float32) -> Tuple[List[float], torch.Tensor, torch.Tensor]:
    """`epochs` calls of train (gcn_distr.py:341-366).  Returns (loss per epoch, w1, w2).
    optimizer: "sgd" (the CPU plumbing configuration) or "adam" (the reference, gcn_distr.py:562)."""
    x = x.to(dtype)
    w1 = w1.to(dtype).clone().requires_grad_(True)
    w2 = w2.to(dtype).clone().requires_grad_(True)
    bf = [b.to(dtype) for b in blocks_fwd]
    bb = bf if blocks_bwd is None else [b.to(dtype) for b in blocks_bwd]
    opt = torch.optim.SGD([w1, w2], lr=lr) if optimizer == "sgd" else torch.optim.Adam([w1, w2], lr=lr)
    losses = []
    for _ in range(epochs):
        h = gcn_layer(x, w1, bf, "relu", bb)
        out = gcn_layer(h, w2, bf, "log_softmax", bb)
        opt.zero_grad()
        loss = masked_nll(out, y, mask)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    return losses, w1.detach(), w2.detach()


# ------------------------------------------------------------------------------------------------
# input preparation
# ------------------------------------------------------------------------------------------------
def gcn_normalize(row: np.ndarray, col: np.ndarray, n: int) -> np.ndarray:
    """scale_elements (gcn_distr.py:439-468) in NumPy: deg counted per row in fp64, deg**-0.5 in
    fp64, cast to fp32; value = fl32(dinv[row] * fl32(1 * dinv[col]))."""
    row, col = np.asarray(row, dtype=np.int64), np.asarray(col, dtype=np.int64)
    deg = np.bincount(row, minlength=n).astype(np.float64)
    with np.errstate(divide="ignore"):
        dinv = np.power(deg, -0.5).astype(np.float32)
    right = (np.float32(1.0) * dinv[col]).astype(np.float32)
    return (dinv[row] * right).astype(np.float32)


def add_self_loops(row: np.ndarray, col: np.ndarray, n: int):
    """add_remaining_self_loops on an unweighted pattern (gcn_distr.py:791) followed by the
    coalesce the reference applies to its adjacency matrix (gcn_distr.py:546): the off-diagonal
    entries plus every (i, i) once, in (row, col) order."""
    row, col = np.asarray(row, dtype=np.int64), np.asarray(col, dtype=np.int64)
    off = row != col
    r = np.concatenate([row[off], np.arange(n, dtype=np.int64)])
    c = np.concatenate([col[off], np.arange(n, dtype=np.int64)])
    order = np.lexsort((c, r))
    return r[order], c[order]


def block_bounds_1d(node_count: int, parts: int) -> List[int]:
    """gcn_distr.py:398-400 with n_per_proc = ceil(n/parts) (:474)."""
    step = int(math.ceil(float(node_count) / parts))
    return list(range(0, node_count, step)) + [node_count]


def block_bounds_2d(node_count: int, proc_dim: int) -> List[int]:
    """gcn_distr_2d.py:1032-1038 with n_per_proc = n // sqrt(P) (:1102): remainder to the last block."""
    step = node_count // proc_dim
    return list(range(0, node_count, step))[:proc_dim] + [node_count]


def coo_block(row: np.ndarray, col: np.ndarray, val: np.ndarray, r0: int, r1: int, c0: int, c1: int):
    """Entries inside [r0, r1) x [c0, c1), rebased (gcn_distr.py:404-406)."""
    row, col = np.asarray(row), np.asarray(col)
    keep = (row >= r0) & (row < r1) & (col >= c0) & (col < c1)
    return row[keep] - r0, col[keep] - c0, np.asarray(val)[keep]


# ------------------------------------------------------------------------------------------------
# byte format of a sparse block (replaces the pickled int64 COO of gcn_distr.py:747 and the float32
# index payload of gcn_distr_2d.py:369-374); restated here from the format description alone
# ------------------------------------------------------------------------------------------------
BLOB_MAGIC = b"CGNTCSR\x00"
BLOB_HEADER = 128


def _blob_offsets(n: int, nnz: int):
    up = lambda v: (v + 63) // 64 * 64
    off_rowptr = BLOB_HEADER
    off_colind = up(off_rowptr + 4 * (n + 1))
    off_values = up(off_colind + 4 * nnz)
    return off_rowptr, off_colind, off_values, up(off_values + 4 * nnz)


def _fnv1a_words(payload: bytes) -> int:
    h = 1469598103934665603
    for (w,) in struct.iter_unpack("<Q", payload):
        h = ((h ^ w) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def blob_write(rowptr: np.ndarray, colind: np.ndarray, values: np.ndarray, n: int, m: int, has_transpose: bool) -> bytes:
    nnz = int(len(colind))
    o_r, o_c, o_v, total = _blob_offsets(n, nnz)
    buf = bytearray(total)
    buf[o_r:o_r + 4 * (n + 1)] = np.asarray(rowptr, dtype="<i4").tobytes()
    buf[o_c:o_c + 4 * nnz] = np.asarray(colind, dtype="<i4").tobytes()
    buf[o_v:o_v + 4 * nnz] = np.asarray(values, dtype="<f4").tobytes()
    head = struct.pack("<8sIIqqqQQQQQ", BLOB_MAGIC, 1, 1 if has_transpose else 0, n, m, nnz, o_r, o_c, o_v, total,
                       _fnv1a_words(bytes(buf[BLOB_HEADER:])))
    buf[:len(head)] = head
    return bytes(buf)


def blob_read(blob: bytes):
    """(rowptr, colind, values, n, m, has_transpose); raises ValueError on a malformed blob."""
    blob = bytes(blob)
    if len(blob) < BLOB_HEADER:
        raise ValueError("no header")
    magic, version, flags, n, m, nnz, o_r, o_c, o_v, total, checksum = struct.unpack_from("<8sIIqqqQQQQQ", blob, 0)
    if magic != BLOB_MAGIC or version != 1:
        raise ValueError("bad magic or version")
    if min(n, m, nnz) < 0 or (o_r, o_c, o_v, total) != _blob_offsets(n, nnz) or len(blob) < total:
        raise ValueError("inconsistent sizes")
    if _fnv1a_words(blob[BLOB_HEADER:total]) != checksum:
        raise ValueError("checksum mismatch")
    rowptr = np.frombuffer(blob, dtype="<i4", count=n + 1, offset=o_r)
    colind = np.frombuffer(blob, dtype="<i4", count=nnz, offset=o_c)
    values = np.frombuffer(blob, dtype="<f4", count=nnz, offset=o_v)
    if rowptr[0] != 0 or rowptr[-1] != nnz or np.any(np.diff(rowptr) < 0):
        raise ValueError("rowptr is not a monotone map onto [0, nnz]")
    if nnz and (colind.min() < 0 or colind.max() >= m):
        raise ValueError("column index out of range")
    return rowptr, colind, values, n, m, bool(flags & 1)


# ------------------------------------------------------------------------------------------------
# error metric of the parity tests
# ------------------------------------------------------------------------------------------------
def max_rel_error(got: torch.Tensor, ref64: torch.Tensor, magnitude64: torch.Tensor) -> float:
    """max |got - ref| / magnitude, entries with zero magnitude compared absolutely against 0."""
    got = got.detach().to("cpu", torch.float64)
    diff = (got - ref64).abs()
    mag = magnitude64.clamp_min(1e-300)
    rel = torch.where(magnitude64 > 0, diff / mag, diff)
    return float(rel.max()) if rel.numel() else 0.0
