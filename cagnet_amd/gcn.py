"""Host side of the per-rank GCN compute path: the stage loop, GCNFunc and train of the reference
(gcn_distr.py:203-246, :248-339, :341-366) restated for one GPU on top of the C ABI.

What changes against the reference, and why:
  * the broadcasts are gone: the dense blocks the other ranks would have sent are already resident
    (`ResidentBlocks`), so a stage is just `z_loc += A_k @ H_k`;
  * sparse blocks are `CsrMatrix` handles (CSR, optional transpose and schedules built once)
    instead of COO tensors that are cast and converted on every call (gcn_distr.py:238-240);
  * ReLU is fused into the store of `(A H) W`; backward derives the mask from the saved output
    instead of re-running the activation under autograd (gcn_distr.py:312-322);
  * with one block that carries its transpose, backward multiplies by A^T; the reference always
    reuses A and therefore needs a symmetric matrix (gcn_distr.py:326).
Names and argument order follow the reference so that its drivers read the same.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Union

import torch
import torch.nn.functional as F

from . import ops
from .ops import CsrMatrix

# the reference keeps these as module globals set from the command line (gcn_distr.py:57-58, :826-827)
activations = True

# Product order of a layer.  True (default) is the reference's: the SpMM runs first, at the input
# width, Z = (A H) W (gcn_distr.py:271, :275).  False is an opt-in reordering, Z = A (H W): the
# same mathematics with the SpMM at the output width (602 -> 16 for the first layer), different
# rounding; backward is unchanged because it already multiplies A by the output-width gradient.
spmm_first = True


# Fuse the layer's two forward products, Z = act((sum_i A_i H_i) W), into the last stage's SpMM when
# the width allows it: the n x f_in intermediate (gcn_distr.py:271) is then never written.  Same
# product order as the reference; only the summation order inside the small W product differs.
fused_forward = True
# ... but only where it pays: the epilogue costs a fixed f_in * f_out multiply-adds per row, the
# saving is one write and one read of the row.  Measured against the row-wise SpMM kernels: Amazon shape
# (16 entries per row) epoch 77.7 -> 71.4 ms, Reddit shape (492 entries per row) 24.3 -> 24.5 ms.  Where the
# library multiplies the block through a tile plan (rows of 8 entries and more, products from 8e8 multiply-adds
# and 65 columns on: cg_tune_set "spmm_tile"), the plain product wins - Amazon shape at f = 300: fused 39.5 ms,
# tile plan 33.0 ms + 3.4 ms for the product with W - and the fused form is left to the smaller products.
fused_forward_max_row_entries = 64


def _tile_plan_expected(block: CsrMatrix, width: int) -> bool:
    """The library's own rule for multiplying `block` at this width through a tile plan (spmm.hip: want_tile)."""
    return width >= 65 and block.nnz >= 8 * max(block.n, 1) and float(block.nnz) * width >= 8e8


# The stage loop reads a wide operand that the caller registered with ops.keep_aligned (the input features, say)
# through a kept copy with line-aligned rows when its own rows are not a whole number of 128-byte lines long
# (ops.aligned_rows; ops.aligned_operands = False turns that off).
_aligned_rows = ops.aligned_rows


# Backward of a layer that widens (16 -> 41 classes).  The reference multiplies A by the output-width gradient first,
# AG = A G, and takes dH = AG W^T and dW = H^T AG from it (gcn_distr.py:326-337).  With this flag such a layer keeps
# Z = A H from its forward pass and computes dW = Z^T G and dH = A^T (G W^T) instead: the same mathematics (for the
# symmetric A the reference assumes, or with the block's stored transpose), with the SpMM at the input width (16)
# instead of the output width (41, carried as 44); different rounding.  Single-block products only: with several
# stages the per-rank partial sums of dW would differ from the reference's before their all-reduce.
narrow_backward = True


# With every stage operand resident, the stage loop z = sum_k A_k H_k is one product of the blocks side by side,
# [A_0 | A_1 | ...], with the H_k stacked (one plan over the whole block row, Z written once instead of read and
# written again per stage); `fuse_stages = False` keeps the reference's one product per stage (gcn_distr.py:221-244).
# Same sums, other order of the additions.  The stacked matrix is a second copy of the blocks' entries (built at
# the first fused loop over a list of blocks and kept with it), and the stage operands are kept stacked in one
# buffer per direction: the peers' blocks are copied into it once, the rank's own block before every product.
fuse_stages = True


class StackedPeers(list):
    """The resident blocks of a stage loop (a list, None at the caller's own index), also kept stacked in one
    buffer so that the loop can run as one product."""

    def __init__(self, blocks: Sequence[Optional[torch.Tensor]]):
        super().__init__(blocks)
        self.buffer = None      # [sum of the blocks' rows, width], built on first use
        self.offsets = None     # first row of every stage's block in it
        self.filled_for = None  # rank whose peers have been copied in

    def stacked(self, rank: int, own: torch.Tensor, rows: Sequence[int]) -> torch.Tensor:
        """The buffer with the peers' blocks in place and `own` copied to the caller's slot."""
        width = own.shape[1]
        if self.buffer is None or self.buffer.shape[1] != width or self.filled_for != rank:
            self.offsets = [sum(rows[:k]) for k in range(len(rows) + 1)]
            ld = width if width % 32 == 0 or width < 64 else (width + 31) // 32 * 32  # wide rows on 128-byte boundaries
            self.buffer = torch.empty(self.offsets[-1], ld, dtype=own.dtype, device=own.device)[:, :width]
            for k, blk in enumerate(self):
                if k != rank:
                    if blk is None or blk.shape != (rows[k], width):
                        raise ValueError(f"stage {k}: resident block is missing or has the wrong shape")
                    self.buffer[self.offsets[k]:self.offsets[k + 1]].copy_(blk)
            self.filled_for = rank
        if own.shape[0] != rows[rank]:
            raise ValueError(f"own block has {own.shape[0]} rows, the sparse block of stage {rank} has {rows[rank]} columns")
        slot = self.buffer[self.offsets[rank]:self.offsets[rank + 1]]
        if own.data_ptr() != slot.data_ptr():
            with torch.no_grad():
                slot.copy_(own)
        return self.buffer


class ResidentBlocks:
    """Stands where the reference passes a process group: the dense blocks that its broadcasts
    would deliver (gcn_distr.py:230), already resident in HBM.  `forward[i]` is the H block and
    `backward[i]` the gradient block of stage i; the entry of the calling rank itself is ignored
    (its own tensor is used, as in the reference's `inputs.clone()` branch, gcn_distr.py:222-223).
    The blocks are taken as constant for the life of this object (they stand for received data)."""

    def __init__(self, forward: Sequence[Optional[torch.Tensor]], backward: Sequence[Optional[torch.Tensor]]):
        self.forward = StackedPeers(forward)
        self.backward = StackedPeers(backward)


_stacks: dict = {}   # id of a list's first block -> (weak references to its blocks, transpose, the stacked matrix)


def stacked_blocks(am_partitions: Sequence[CsrMatrix]) -> CsrMatrix:
    """[A_0 | A_1 | ...] for a list of blocks, built once per list (ops.CsrMatrix.hstack)."""
    import weakref

    key = id(am_partitions[0])
    hit = _stacks.get(key)
    if hit is not None and len(hit[0]) == len(am_partitions) and all(r() is b for r, b in zip(hit[0], am_partitions)):
        return hit[1]
    for k in [k for k, v in _stacks.items() if any(r() is None for r in v[0])]:
        del _stacks[k]
    stacked = CsrMatrix.hstack(am_partitions)
    _stacks[key] = ([weakref.ref(b) for b in am_partitions], stacked)
    return stacked


def _stage_operand(i: int, rank: int, own: torch.Tensor, peers: Optional[Sequence[Optional[torch.Tensor]]]):
    if i == rank or peers is None:
        if i != rank:
            raise ValueError(f"stage {i}: no resident block given and it is not the caller's own (rank {rank})")
        return own
    blk = peers[i]
    if blk is None:
        raise ValueError(f"stage {i}: resident block is missing")
    if blk.shape[1] != own.shape[1]:
        raise ValueError(f"stage {i}: resident block has width {blk.shape[1]}, expected {own.shape[1]}")
    return blk


def broad_func(node_count: int, am_partitions: Sequence[CsrMatrix], inputs: torch.Tensor, rank: int, size: int,
               group: Optional[Sequence[Optional[torch.Tensor]]] = None, transpose: bool = False,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """z_loc = sum_i am_partitions[i] @ H_i, the stage loop of gcn_distr.py:203-246 without the
    broadcasts.  `group` lists the resident H_i (None at index `rank`, where `inputs` is used).
    The first stage writes (beta = 0), later stages accumulate (beta = 1), so no zero fill.
    `out`, when given, receives the sum (it may be a column slice of a wider buffer)."""
    if len(am_partitions) != size:
        raise ValueError(f"{len(am_partitions)} sparse blocks for size {size}")
    if (fuse_stages and 1 < size <= 16 and not transpose and isinstance(group, StackedPeers) and len(group) == size
            and 0 <= rank < size):
        stacked = stacked_blocks(am_partitions)
        h_all = group.stacked(rank, inputs, [blk.m for blk in am_partitions])
        return stacked.spmm(h_all) if out is None else stacked.spmm(h_all, out=out, beta=0.0)
    z_loc = None
    for i in range(size):
        h_i = _aligned_rows(_stage_operand(i, rank, inputs, group))
        blk = am_partitions[i]
        if z_loc is None:
            z_loc = blk.spmm(h_i, transpose=transpose) if out is None else blk.spmm(h_i, out=out, beta=0.0,
                                                                                    transpose=transpose)
        else:
            blk.spmm(h_i, out=z_loc, beta=1.0, transpose=transpose)
    return z_loc


def stage_schedule_15d(rank: int, size: int, replication: int) -> List[tuple]:
    """Stages of one rank in the 1.5D algorithm (gcn_distr_15d.py:194-208): a list of
    (source rank q, block id).  The P/c block columns of a block row are dealt to the c replicas of
    that row, P/c^2 consecutive ones each; the last replica also takes what is left over."""
    if replication < 1 or size % replication != 0 or size // (replication ** 2) < 1:
        raise ValueError(f"size {size} is not a multiple of replication {replication} squared blocks")
    rank_col = rank % replication
    per_replica = size // (replication ** 2)
    stages = per_replica
    if rank_col == replication - 1:
        stages = (size // replication) - (replication - 1) * per_replica
    out = []
    for i in range(stages):
        block = rank_col * per_replica + i
        out.append((block * replication + rank_col, block))
    return out


def broad_func_15d(node_count: int, am_partitions: Sequence[CsrMatrix], inputs: torch.Tensor, rank: int, size: int,
                   replication: int, group: Optional[Sequence[Optional[torch.Tensor]]] = None,
                   replica_partials: Optional[Sequence[torch.Tensor]] = None, transpose: bool = False) -> torch.Tensor:
    """This rank's share of the 1.5D stage loop (gcn_distr_15d.py:173-245) without the broadcasts:
    z_loc = sum over its stages of am_partitions[block] @ H_block, where `am_partitions` are the
    P/c blocks of the rank's block row and `group[block]` the resident H block of that stage (the
    rank's own `inputs` when the stage's source is the rank itself).  The reference then sums
    z_loc over the c replicas of the row with an all-reduce (:239); `replica_partials`, when given,
    stands for the other replicas' results and is added in order."""
    if len(am_partitions) != size // replication:
        raise ValueError(f"{len(am_partitions)} sparse blocks for {size // replication} block columns")
    z_loc = None
    for q, block in stage_schedule_15d(rank, size, replication):
        h = inputs if q == rank else (group[block] if group is not None else None)
        if h is None:
            raise ValueError(f"stage of block {block}: resident block is missing")
        blk = am_partitions[block]
        if z_loc is None:
            z_loc = blk.spmm(h, transpose=transpose)
        else:
            blk.spmm(h, out=z_loc, beta=1.0, transpose=transpose)
    if z_loc is None:
        raise ValueError("rank has no stage")
    for part in replica_partials or ():
        z_loc = z_loc + part
    return z_loc


def outer_product2(inputs_t: torch.Tensor, ag: torch.Tensor, rank: int = 0, size: int = 1, group=None) -> torch.Tensor:
    """grad_weight = H^T @ AG (gcn_distr.py:178-201 without the all-reduce).  Takes H^T like the
    reference; the kernel reads H itself, so the transpose view is undone without a copy."""
    return ops.dense_xtg(inputs_t.t(), ag)


def _padded_width(c: int) -> int:
    """Widths that are not a multiple of 4 (41 classes) are carried in buffers padded to the next
    multiple of 4 with zero columns, so that the SpMM over them moves 16 bytes per lane."""
    return (c + 3) // 4 * 4


def _padded_ld(c: int) -> int:
    """Leading dimension of such a buffer: rows start on 64-byte boundaries (44 columns are stored 48
    apart), so that a gathered row never straddles one more cache line than it has to (Reddit shape,
    width 44: 1.97 -> 1.88 ms)."""
    return (c + 15) // 16 * 16


def _kind(func) -> str:
    if func is F.relu or func is torch.relu or func == "relu":
        return "relu"
    if func is F.log_softmax or func is torch.log_softmax or func == "log_softmax":
        return "log_softmax"
    return "none"


class GCNFunc(torch.autograd.Function):
    """One GCN layer, `func((sum_i A_i @ H_i) @ W)`; same argument list as gcn_distr.py:250."""

    @staticmethod
    def forward(ctx, inputs, weight, adj_matrix, am_partitions, rank, size, group, func):
        kind = _kind(func) if activations else "none"
        node_count = adj_matrix if isinstance(adj_matrix, int) else adj_matrix.size(0)
        peers_fwd = group.forward if isinstance(group, ResidentBlocks) else None
        z_kept = None
        if spmm_first or size != 1 or weight.shape[1] >= inputs.shape[1]:  # reordering only pays when the layer narrows
            out = None
            last = am_partitions[size - 1]
            short_rows = (last.nnz <= fused_forward_max_row_entries * max(last.n, 1)
                          and not _tile_plan_expected(last, inputs.shape[1]))
            if fused_forward and short_rows and weight.shape[1] <= 64 and inputs.shape[1] >= 128:
                # stages 0 .. size-2 accumulate as usual, the last one also applies W (and ReLU)
                z = broad_func(node_count, am_partitions[:-1], inputs, rank, size - 1, peers_fwd) if size > 1 else None
                h_last = _aligned_rows(_stage_operand(size - 1, rank, inputs, peers_fwd))
                out = am_partitions[size - 1].spmm_xw(h_last, weight, relu=(kind == "relu"), acc=z)
                if out is None and z is not None:      # no fused form for this width: finish the stage loop
                    am_partitions[size - 1].spmm(h_last, out=z, beta=1.0)
                    out = ops.dense_xw(z, weight, relu=(kind == "relu"))
            if out is None:
                z = broad_func(node_count, am_partitions, inputs, rank, size, peers_fwd)
                out = ops.dense_xw(z, weight, relu=(kind == "relu"))
                # dW = (A H)^T G is H^T (A^T G): the same as the reference's H^T (A G) only where backward multiplies
                # with A^T as well, i.e. the block stores its transpose (or the caller has declared A symmetric)
                if (narrow_backward and size == 1 and _padded_width(weight.shape[1]) > inputs.shape[1]
                        and (last.has_transpose or getattr(last, "symmetric", False))):
                    z_kept = z
                del z
        else:
            out = broad_func(node_count, am_partitions, ops.dense_xw(inputs, weight), rank, size, peers_fwd)
            if kind == "relu":
                out = ops.relu_fwd(out)
        if kind == "log_softmax":
            out = ops.log_softmax_fwd(out)
        ctx.save_for_backward(inputs, weight, out)
        ctx.z_kept = z_kept
        ctx.am_partitions = am_partitions
        ctx.rank, ctx.size, ctx.group, ctx.kind, ctx.node_count = rank, size, group, kind, node_count
        return out

    @staticmethod
    def backward(ctx, grad_output):
        inputs, weight, out = ctx.saved_tensors
        kind = ctx.kind
        if kind == "relu":
            grad_output = ops.relu_bwd(grad_output, out)
        elif kind == "log_softmax":
            grad_output = ops.log_softmax_bwd(grad_output, out)
        peers_bwd = ctx.group.backward if isinstance(ctx.group, ResidentBlocks) else None
        blocks = ctx.am_partitions
        use_t = ctx.size == 1 and blocks[0].has_transpose
        if ctx.z_kept is not None:  # the layer widens: SpMM at the input width (see narrow_backward)
            grad_weight = ops.dense_xtg(ctx.z_kept, grad_output) if ctx.needs_input_grad[1] else None
            grad_input = None
            if ctx.needs_input_grad[0]:
                dz = ops.dense_gwt(grad_output, weight)
                grad_input = broad_func(ctx.node_count, blocks, dz, ctx.rank, ctx.size, peers_bwd, transpose=use_t)
            ctx.z_kept = None
            return grad_input, grad_weight, None, None, None, None, None, None
        width = grad_output.shape[1]
        padded = _padded_width(width)
        ag_out = None
        if padded != width and peers_bwd is None:
            ld = _padded_ld(padded)
            wide = torch.zeros(grad_output.shape[0], ld, dtype=grad_output.dtype, device=grad_output.device)[:, :padded]
            wide[:, :width].copy_(grad_output)
            grad_output = wide
            rows_out = blocks[0].m if use_t else blocks[0].n
            ag_out = torch.empty(rows_out, ld, dtype=grad_output.dtype, device=grad_output.device)[:, :padded]
        # first backprop equation: A G (reference: same blocks, gcn_distr.py:326)
        ag = broad_func(ctx.node_count, blocks, grad_output, ctx.rank, ctx.size, peers_bwd, transpose=use_t, out=ag_out)
        if padded != width and peers_bwd is None:
            ag = ag[:, :width]  # a view: the dense products take the row stride as leading dimension
        grad_input = ops.dense_gwt(ag, weight) if ctx.needs_input_grad[0] else None
        # second backprop equation reuses A G (gcn_distr.py:337)
        grad_weight = outer_product2(inputs.t(), ag) if ctx.needs_input_grad[1] else None
        return grad_input, grad_weight, None, None, None, None, None, None


class MaskedNLLLoss(torch.autograd.Function):
    """F.nll_loss(outputs[mask], y[mask]) without materialising the gathered rows
    (gcn_distr.py:356); an empty mask gives a zero loss with zero gradient, which is what the
    reference's fake_loss branch produces (gcn_distr.py:359-362)."""

    @staticmethod
    def forward(ctx, outputs, y, mask):
        loss, count = ops.nll_loss_fwd(outputs, y, mask)
        ctx.save_for_backward(y, mask if mask is not None else torch.empty(0, device=y.device), count)
        ctx.has_mask = mask is not None
        ctx.shape = tuple(outputs.shape)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        y, mask, count = ctx.saved_tensors
        n, c = ctx.shape
        g = ops.nll_loss_bwd(y, mask if ctx.has_mask else None, count, grad_loss.float().reshape(()), n, c)
        return g, None, None


def masked_nll_loss(outputs: torch.Tensor, y: torch.Tensor, mask: Optional[torch.Tensor]) -> torch.Tensor:
    return MaskedNLLLoss.apply(outputs, y, mask)


# `train` ends in log_softmax followed by the masked NLL (gcn_distr.py:344, :356).  With this flag
# their backward passes are one kernel, dZ = (softmax(Z) - onehot(y)) * mask / |mask|, instead of the
# NLL gradient (an n x classes array that is zero except for one entry per row) written out and read
# again by the log_softmax gradient; forward likewise takes the loss from the log_softmax pass
# instead of reading the log-probabilities again.
fused_loss = True


class LogSoftmaxNLLLoss(torch.autograd.Function):
    """(log_softmax(z, dim=1), masked mean NLL of it): the last activation of `train` and its loss as
    one autograd node.  The log-probabilities are returned because `train` returns them; gradients
    flow through the loss only."""

    @staticmethod
    def forward(ctx, z, y, mask):
        logp, loss, count = ops.log_softmax_nll_fwd(z, y, mask)
        ctx.save_for_backward(logp, y, mask if mask is not None else torch.empty(0, device=y.device), count)
        ctx.has_mask = mask is not None
        ctx.mark_non_differentiable(logp)
        return logp, loss

    @staticmethod
    def backward(ctx, _grad_logp, grad_loss):
        logp, y, mask, count = ctx.saved_tensors
        dz = ops.log_softmax_nll_bwd(logp, y, mask if ctx.has_mask else None, count, grad_loss.float().reshape(()))
        return dz, None, None


def train(inputs, weight1, weight2, adj_matrix, am_partitions, optimizer, data, rank=0, size=1, group=None):
    """One epoch, gcn_distr.py:341-366.  `data` needs `.y` and `.train_mask`; `group` is None for a
    whole graph on one GPU, or a pair (layer-1 ResidentBlocks, layer-2 ResidentBlocks)."""
    g1, g2 = group if isinstance(group, (tuple, list)) else (group, group)
    outputs = GCNFunc.apply(inputs, weight1, adj_matrix, am_partitions, rank, size, g1, F.relu)
    fuse = fused_loss and activations
    outputs = GCNFunc.apply(outputs, weight2, adj_matrix, am_partitions, rank, size, g2, None if fuse else F.log_softmax)

    optimizer.zero_grad()

    node_count = adj_matrix if isinstance(adj_matrix, int) else adj_matrix.size(0)
    n_per_proc = int(math.ceil(float(node_count) / size))
    rank_train_mask = torch.split(data.train_mask.bool(), n_per_proc, dim=0)[rank]
    datay_rank = torch.split(data.y, n_per_proc, dim=0)[rank]

    if fuse:
        outputs, loss = LogSoftmaxNLLLoss.apply(outputs, datay_rank, rank_train_mask)
    else:
        loss = masked_nll_loss(outputs, datay_rank, rank_train_mask)
    loss.backward()
    optimizer.step()
    train.last_loss = loss.detach()
    return outputs


train.last_loss = None


class GraphedTrain:
    """`train` captured once into a HIP graph and replayed: one launch per epoch instead of some
    forty.  On graphs of a few thousand vertices an epoch is bound by launches and host work, not
    by kernels (4,096 vertices: 0.69 ms per eager epoch); on the large configurations it changes
    nothing measurable.  The reference has no counterpart (its epoch synchronises the device in
    every spmm_gpu call, sparse_coo_tensor.cu:229-231).

    The library's scratch buffers are cached per stream, so warm-up, capture and replay all use
    one private stream.  The constructor runs `warmup` ordinary epochs there (they train: weights
    and optimizer state advance) and then records one more epoch without executing it; `step()`
    replays it.  Every tensor the epoch reads (`inputs`, the weights, `data.y`, `data.train_mask`)
    is read from the same memory on every replay: update them in place.  Optimizers that keep
    scalars on the host must be built for capture (`torch.optim.Adam(..., capturable=True)`).

    The graph replays with the addresses of the library's scratch buffers of its stream and of the
    tables of the matrices it multiplies with; the library keeps both alive for as long as the matrices
    live (later eager calls that need other tables or more scratch get new memory).  `close()` drops
    the graph and hands that memory back: the private stream's scratch at once, a matrix's parked
    tables when the last graph captured over it is closed (the matrices count their graphs: `graph_retain`,
    `graph_release`)."""

    def __init__(self, inputs, weight1, weight2, adj_matrix, am_partitions, optimizer, data, rank=0, size=1,
                 group=None, warmup: int = 3):
        if warmup < 1:
            raise ValueError("at least one warm-up epoch is needed: it builds the schedules and grows the scratch")
        args = (inputs, weight1, weight2, adj_matrix, am_partitions, optimizer, data, rank, size, group)
        self.stream = torch.cuda.Stream(device=weight1.device)
        self.stream.wait_stream(torch.cuda.current_stream(weight1.device))
        with torch.cuda.stream(self.stream):
            for _ in range(warmup):
                train(*args)
                inputs.grad = None
        torch.cuda.current_stream(weight1.device).wait_stream(self.stream)
        torch.cuda.synchronize(weight1.device)
        optimizer.zero_grad(set_to_none=True)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=self.stream):
            self.outputs = train(*args)
            self.loss = train.last_loss
        self.epochs_run = warmup
        self._matrices = [m for m in am_partitions if hasattr(m, "graph_release")]
        for m in self._matrices:
            m.graph_retain()

    def close(self) -> None:
        """Drop the captured graph and free what the library kept alive for it.  Idempotent."""
        if getattr(self, "graph", None) is None:
            return
        self.graph = None
        torch.cuda.synchronize(self.stream.device)
        ops.scratch_release(self.stream)
        for m in self._matrices:
            m.graph_release()  # frees the parked tables only when no other live graph was captured over the matrix
        self._matrices = []

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown: the driver reclaims the memory
            pass

    def step(self) -> torch.Tensor:
        """One more epoch.  Returns the epoch's outputs (the same tensor every time; `self.loss`
        likewise holds the epoch's loss after the replay has run)."""
        if self.graph is None:
            raise RuntimeError("GraphedTrain.step() after close()")
        self.graph.replay()
        self.epochs_run += 1
        return self.outputs
