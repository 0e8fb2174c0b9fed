"""The path at the full sizes of the benchmark configurations, checked through properties that do
not need a CPU restatement of the whole product: structure of the CSR, involution of the transpose,
a checksum of checksums (1^T (A B) = (1^T A) B, with the column sums of A taken by torch in fp64),
rows sampled at random and recomputed in fp64 from the COO arrays, linearity, determinism, symmetry,
and the same identities for the three dense products.  torch is the independent party here; the
library is only ever on one side of a comparison."""
import pytest
import torch

from cagnet_amd import synth
from tests.util import REL_TOL

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _release_device_memory():
    """These tests hold tens of GB; hand the cached blocks back so later tests and the library's own
    allocations see the whole device."""
    yield
    torch.cuda.empty_cache()


REDDIT = dict(n=232_965, target_nnz=114_615_892, f=602, hidden=16, classes=41)
AMAZON = dict(n=14_249_639, target_nnz=230_600_000, f=300, hidden=16, classes=24)


def _graph(spec, dev):
    row, col = synth.rmat_graph_target_nnz(spec["n"], spec["target_nnz"], 1, dev)
    val = synth.gcn_normalize(row, col, spec["n"])
    return row, col, val


def _column_checksum(row, col, val, B, chunk=1 << 20):
    """(1^T A) B and (1^T |A|) |B| in fp64, from the COO arrays alone."""
    n = B.shape[0]
    colsum = torch.zeros(n, dtype=torch.float64, device=B.device).index_add_(0, col, val.double())
    colabs = torch.zeros(n, dtype=torch.float64, device=B.device).index_add_(0, col, val.double().abs())
    want = torch.zeros(B.shape[1], dtype=torch.float64, device=B.device)
    mag = torch.zeros_like(want)
    for lo in range(0, n, chunk):
        blk = B[lo:lo + chunk].double()
        want += colsum[lo:lo + chunk] @ blk
        mag += colabs[lo:lo + chunk] @ blk.abs()
    return want, mag


def _column_sums(C, chunk=1 << 20):
    out = torch.zeros(C.shape[1], dtype=torch.float64, device=C.device)
    for lo in range(0, C.shape[0], chunk):
        out += C[lo:lo + chunk].double().sum(dim=0)
    return out


def _check_sampled_rows(C, row, col, val, B, count, seed):
    """Rows drawn at random, recomputed in fp64 from the (row-sorted) COO arrays by torch."""
    n = C.shape[0]
    rowptr = torch.searchsorted(row, torch.arange(n + 1, device=row.device))
    picks = torch.randint(0, n, (count,), generator=torch.Generator().manual_seed(seed)).tolist()
    for i in picks + [0, n - 1]:
        s, e = int(rowptr[i]), int(rowptr[i + 1])
        a = val[s:e].double()
        rows = B[col[s:e]].double()
        want = a @ rows
        mag = a.abs() @ rows.abs()
        err = ((C[i].double() - want).abs() / mag.clamp_min(1e-30)).max()
        assert float(err) <= REL_TOL, f"row {i}: {float(err)}"


def _check_product(A, row, col, val, B, transpose=False, seed=0):
    C = A.spmm(B, transpose=transpose)
    want, mag = _column_checksum(row, col, val, B)
    got = _column_sums(C)
    # a column sum adds n rounded entries: the bound is the per-entry bound on the magnitudes' sum
    assert float(((got - want).abs() / mag.clamp_min(1e-30)).max()) <= REL_TOL
    _check_sampled_rows(C, row, col, val, B, 48, seed)
    assert torch.equal(C, A.spmm(B, transpose=transpose))  # fixed summation order
    return C


def _structure(rowptr, colind, n, nnz):
    assert int(rowptr[0]) == 0 and int(rowptr[-1]) == nnz
    assert bool((rowptr[1:] >= rowptr[:-1]).all())
    inside = torch.ones(nnz, dtype=torch.bool, device=colind.device)
    starts = rowptr[1:-1].long()
    inside[starts[starts < nnz]] = False  # the first entry of a row may be smaller than its predecessor
    inside[0] = False
    ascending = colind[1:] > colind[:-1]
    assert bool((ascending | ~inside[1:]).all())


def test_reddit_shape_conversions_and_products(cuda):
    """Configuration 3 (232,965 vertices, 114.6 M entries): conversions and the products of every
    width the epoch uses, on the schedules the library picks at this size (hub plan at 602)."""
    from cagnet_amd import ops
    spec = REDDIT
    n = spec["n"]
    row, col, val = _graph(spec, cuda)
    nnz = row.numel()
    r32, c32 = row.int(), col.int()

    rowptr, colind, values = ops.coo2csr(r32, c32, val, n, n)
    _structure(rowptr, colind, n, nnz)
    assert torch.equal(colind, c32) and torch.equal(values, val)       # sorted input: a permutation-free pass
    assert torch.equal(rowptr, ops.coo2csr_rowptr(r32, n))
    perm = torch.randperm(nnz, device=cuda, generator=torch.Generator(device=cuda).manual_seed(5))
    rp2, ci2, vv2 = ops.coo2csr(r32[perm], c32[perm], val[perm], n, n)  # any order in, the same CSR out
    assert torch.equal(rp2, rowptr) and torch.equal(ci2, colind) and torch.equal(vv2, values)
    del perm, rp2, ci2, vv2
    tp, ti, tv = ops.csr_transpose(rowptr, colind, values, n, n)
    _structure(tp, ti, n, nnz)
    bp, bi, bv = ops.csr_transpose(tp, ti, tv, n, n)                     # involution
    assert torch.equal(bp, rowptr) and torch.equal(bi, colind) and torch.equal(bv, values)
    # the normalised graph is symmetric bit for bit, so its transpose is itself
    assert torch.equal(tp, rowptr) and torch.equal(ti, colind) and torch.equal(tv, values)
    del tp, ti, tv, bp, bi, bv, rowptr, colind, values

    A = ops.CsrMatrix(r32, c32, val, n, n, is_sorted=True, transpose=True)
    gen = torch.Generator(device=cuda).manual_seed(7)
    for f in (spec["f"], spec["hidden"], 44):
        B = torch.randn(n, f, device=cuda, generator=gen)
        C = _check_product(A, row, col, val, B, seed=f)
        assert torch.equal(A.spmm(B, transpose=True), C)                # symmetric A: the same sums in the same order
        B2 = torch.randn(n, f, device=cuda, generator=gen)
        lin = A.spmm(2.0 * B - B2)
        scale = A.spmm(2.0 * B.abs() + B2.abs())                        # values are positive: the magnitude bound
        assert float(((lin - (2.0 * C - A.spmm(B2))).abs() / scale.clamp_min(1e-30)).max()) <= 4 * REL_TOL
        acc = C.clone()
        A.spmm(B2, out=acc, beta=1.0)                                   # accumulate form
        assert float(((acc - (C + A.spmm(B2))).abs() / scale.clamp_min(1e-30)).max()) <= 4 * REL_TOL
        del B, B2, C, lin, scale, acc


def _check_dense(X, W, G):
    """1^T (X W) = (1^T X) W,  (X^T G) 1 = X^T (G 1),  1^T (G W^T) = (1^T G) W^T, magnitudes alike."""
    from cagnet_amd import ops
    Wd, Wa = W.double(), W.double().abs()
    xs, xa = _column_sums(X), _column_sums(X.abs())
    Z = ops.dense_xw(X, W)
    assert float(((_column_sums(Z) - xs @ Wd).abs() / (xa @ Wa).clamp_min(1e-30)).max()) <= REL_TOL
    del Z
    dW = ops.dense_xtg(X, G)
    g1, ga = G.double().sum(dim=1), G.double().abs().sum(dim=1)
    want = torch.zeros(X.shape[1], dtype=torch.float64, device=X.device)
    mag = torch.zeros_like(want)
    for lo in range(0, X.shape[0], 1 << 20):
        blk = X[lo:lo + (1 << 20)].double()
        want += blk.t() @ g1[lo:lo + (1 << 20)]
        mag += blk.abs().t() @ ga[lo:lo + (1 << 20)]
    assert float(((dW.double().sum(dim=1) - want).abs() / mag.clamp_min(1e-30)).max()) <= REL_TOL
    assert torch.equal(dW, ops.dense_xtg(X, G))
    del dW
    dX = ops.dense_gwt(G, W)
    gs, gab = _column_sums(G), _column_sums(G.abs())
    assert float(((_column_sums(dX) - gs @ Wd.t()).abs() / (gab @ Wa.t()).clamp_min(1e-30)).max()) <= REL_TOL
    rows = torch.randint(0, X.shape[0], (64,), generator=torch.Generator().manual_seed(3)).to(X.device)
    ref = G[rows].double() @ Wd.t()
    bound = G[rows].double().abs() @ Wa.t()
    assert float(((dX[rows].double() - ref).abs() / bound.clamp_min(1e-30)).max()) <= REL_TOL


def test_reddit_shape_dense_products(cuda):
    spec = REDDIT
    gen = torch.Generator(device=cuda).manual_seed(11)
    X = torch.randn(spec["n"], spec["f"], device=cuda, generator=gen)
    W = torch.randn(spec["f"], spec["hidden"], device=cuda, generator=gen)
    G = torch.randn(spec["n"], spec["hidden"], device=cuda, generator=gen)
    _check_dense(X, W, G)


def test_amazon_shape_products(cuda):
    """Configuration 5 (14,249,639 vertices, 230.6 M entries, 300 features): operands of 17.1 GB,
    dense offsets beyond 2^31, the plain wide schedule and the narrow one."""
    from cagnet_amd import ops
    if torch.cuda.get_device_properties(cuda).total_memory < 120 * (1 << 30):
        pytest.skip("needs about 100 GB of device memory")
    spec = AMAZON
    n = spec["n"]
    row, col, val = _graph(spec, cuda)
    A = ops.CsrMatrix(row.int(), col.int(), val, n, n, is_sorted=True, transpose=True)
    gen = torch.Generator(device=cuda).manual_seed(13)
    X = torch.randn(n, spec["f"], device=cuda, generator=gen)
    C = _check_product(A, row, col, val, X, seed=1)
    assert torch.equal(A.spmm(X, transpose=True), C)
    W = torch.randn(spec["f"], spec["hidden"], device=cuda, generator=gen)
    fused = A.spmm_xw(X, W, relu=False)                                  # the fused layer product against its two steps
    if fused is not None:
        two = ops.dense_xw(C, W)
        mag = ops.dense_xw(A.spmm(X.abs()), W.abs())
        assert float(((fused - two).abs() / mag.clamp_min(1e-30)).max()) <= 4 * REL_TOL
        del two, mag, fused
    del C
    G = torch.randn(n, spec["hidden"], device=cuda, generator=gen)
    _check_product(A, row, col, val, G, seed=2)                          # narrow teams
    _check_product(A, row, col, val, torch.randn(n, spec["classes"], device=cuda, generator=gen), transpose=True, seed=3)
    _check_dense(X, W, G)


def test_rmat20_shape_products(cuda):
    """Configuration 2 (R-MAT scale 20: 1,048,576 vertices, 16,777,216 directed edges): A H and A^T G
    at the four widths, with the transpose built by the library from entries given in arbitrary order."""
    from cagnet_amd import ops
    row, col, n = synth.rmat_graph(20, 16_777_216, 1, cuda)
    val = synth.gcn_normalize(row, col, n)
    nnz = row.numel()
    perm = torch.randperm(nnz, device=cuda, generator=torch.Generator(device=cuda).manual_seed(2))
    A = ops.CsrMatrix(row.int()[perm], col.int()[perm], val[perm], n, n, is_sorted=False, transpose=True)
    del perm
    rowptr, colind, values = A.arrays()
    _structure(rowptr, colind, n, nnz)
    assert torch.equal(colind, col.int()) and torch.equal(values, val)   # any order in, the (row, col) order out
    tp, ti, tv = A.arrays(transpose=True)
    assert torch.equal(tp, rowptr) and torch.equal(ti, colind) and torch.equal(tv, values)  # symmetric bit for bit
    del rowptr, colind, values, tp, ti, tv
    gen = torch.Generator(device=cuda).manual_seed(19)
    for f in (16, 64, 128, 602):
        B = torch.randn(n, f, device=cuda, generator=gen)
        C = _check_product(A, row, col, val, B, seed=f)
        # the graph is symmetric, so the product with the stored transpose sums the same terms in the same order
        assert torch.equal(A.spmm(B, transpose=True), C)
        del B, C


def test_reddit_shape_grid_row_of_blocks(cuda):
    """Configuration 4: the four sparse blocks A(r, 0..3) of the last process row of the 4 x 4 grid
    (58,242 rows; block columns of 58,241 | 58,241 | 58,241 | 58,242), cut by the library, each times
    its 602-wide block of H and accumulated over the four stages through the reference's operator
    (gcn_distr_2d.py:333-417) -- against the same rows of the whole product."""
    from cagnet_amd import ops
    from cagnet_amd.sparse_coo_tensor_cpp import spmm_gpu
    spec = REDDIT
    n, f, q = spec["n"], spec["f"], 4
    row, col, val = _graph(spec, cuda)
    r32, c32 = row.int(), col.int()
    b = synth.block_bounds_2d(n, q)
    assert [b[k + 1] - b[k] for k in range(q)] == [58_241, 58_241, 58_241, 58_242]
    r = q - 1
    rows = b[r + 1] - b[r]
    H = torch.randn(n, f, device=cuda, generator=torch.Generator(device=cuda).manual_seed(23))
    z = torch.zeros(rows, f, device=cuda)
    mag = torch.zeros(rows, f, device=cuda)
    total = 0
    for k in range(q):
        br, bc, bv = ops.coo_block(r32, c32, val, b[r], b[r + 1], b[k], b[k + 1])
        inside = (row >= b[r]) & (row < b[r + 1]) & (col >= b[k]) & (col < b[k + 1])       # split_coo, gcn_distr.py:398-409
        assert torch.equal(br.long(), row[inside] - b[r]) and torch.equal(bc.long(), col[inside] - b[k])
        assert torch.equal(bv, val[inside])
        total += br.numel()
        Hk = H[b[k]:b[k + 1]].contiguous()
        for pass_ in range(2):                                                           # second pass: a block seen before
            zk = torch.zeros(rows, f, device=cuda)
            spmm_gpu(br, bc, bv, rows, b[k + 1] - b[k], Hk, zk)
            if pass_ == 0:
                first = zk
        assert torch.equal(first, zk)
        spmm_gpu(br, bc, bv, rows, b[k + 1] - b[k], Hk, z)                                # accumulates over the stages
        spmm_gpu(br, bc, bv, rows, b[k + 1] - b[k], Hk.abs(), mag)
        del br, bc, bv, inside, Hk, zk, first
    assert total == int(((row >= b[r]) & (row < b[r + 1])).sum())
    A = ops.CsrMatrix(r32, c32, val, n, n, is_sorted=True)
    whole = A.spmm(H)[b[r]:b[r + 1]]
    assert float(((z - whole).abs() / mag.clamp_min(1e-30)).max()) <= 4 * REL_TOL
    # rows recomputed in fp64 from the COO arrays
    rowptr = torch.searchsorted(row, torch.arange(n + 1, device=cuda))
    for i in torch.randint(b[r], b[r + 1], (32,), generator=torch.Generator().manual_seed(29)).tolist():
        s, e = int(rowptr[i]), int(rowptr[i + 1])
        a, hb = val[s:e].double(), H[col[s:e]].double()
        err = ((z[i - b[r]].double() - a @ hb).abs() / (a.abs() @ hb.abs()).clamp_min(1e-30)).max()
        assert float(err) <= REL_TOL, f"row {i}: {float(err)}"
    # the same stage loop as one product of the blocks side by side (gcn.broad_func with resident operands):
    # against the per-stage sums, against the rows recomputed in fp64, and bit-identical when repeated
    from cagnet_amd import gcn
    blocks = []
    for k in range(q):
        br, bc, bv = ops.coo_block(r32, c32, val, b[r], b[r + 1], b[k], b[k + 1])
        blocks.append(ops.CsrMatrix(br, bc, bv, rows, b[k + 1] - b[k]))
        del br, bc, bv
    peers = gcn.StackedPeers([None if k == r else H[b[k]:b[k + 1]] for k in range(q)])
    own = H[b[r]:b[r + 1]].contiguous()
    zf = gcn.broad_func(rows, blocks, own, r, q, peers)
    assert gcn.stacked_blocks(blocks).nnz == total and gcn.stacked_blocks(blocks).m == n
    assert float(((zf - z).abs() / mag.clamp_min(1e-30)).max()) <= 4 * REL_TOL
    assert torch.equal(zf, gcn.broad_func(rows, blocks, own, r, q, peers))
    for i in torch.randint(b[r], b[r + 1], (32,), generator=torch.Generator().manual_seed(31)).tolist():
        s, e = int(rowptr[i]), int(rowptr[i + 1])
        a, hb = val[s:e].double(), H[col[s:e]].double()
        err = ((zf[i - b[r]].double() - a @ hb).abs() / (a.abs() @ hb.abs()).clamp_min(1e-30)).max()
        assert float(err) <= REL_TOL, f"fused stage loop, row {i}: {float(err)}"


# ------------------------------------------------------------------------------------------------
# whole epochs at full size: forward, loss and backward of the 2-layer model through the library,
# against torch in fp64 on the device, computed from the COO arrays in the order A (H W) so that
# no fp64 product is wider than the hidden or class count
# ------------------------------------------------------------------------------------------------
def _spmm64(rows_out, tgt, src, val, M, chunk=1 << 23):
    """out[tgt[k]] += val[k] * M[src[k]] in fp64, entries taken in chunks."""
    out = torch.zeros(rows_out, M.shape[1], dtype=torch.float64, device=M.device)
    for lo in range(0, val.numel(), chunk):
        out.index_add_(0, tgt[lo:lo + chunk], val[lo:lo + chunk].double()[:, None] * M[src[lo:lo + chunk]])
    return out


def _matmul64(X, W, chunk=1 << 20):
    return torch.cat([X[lo:lo + chunk].double() @ W for lo in range(0, X.shape[0], chunk)])


def _xt_g64(X, G, chunk=1 << 20):
    out = torch.zeros(X.shape[1], G.shape[1], dtype=torch.float64, device=X.device)
    for lo in range(0, X.shape[0], chunk):
        out += X[lo:lo + chunk].double().t() @ G[lo:lo + chunk]
    return out


def _close_rel_max(got, ref64, what, tol=2e-4):
    """End-to-end quantities chain several products: relative to the largest entry of the reference
    (the per-product 1e-5 bound against the row-sum magnitude is checked product by product above)."""
    err = float((got.double() - ref64).abs().max()) / max(float(ref64.abs().max()), 1e-30)
    assert err <= tol, f"{what}: {err}"


def _reference_epoch(stages_fwd, stages_bwd, X, W1, W2, y, mask, rows):
    """fp64 forward + loss + backward.  stages_*: lists of (tgt, src, val, H or None): the layer sums
    sum_k A_k (H_k W); H None stands for the rank's own operand.  GCNFunc.backward multiplies the
    gradient by the same blocks as forward (gcn_distr.py:326); stages_bwd carries the peers' gradients."""
    W1d, W2d = W1.double(), W2.double()

    def layer_sum(stages, own, Wd, which):
        z = torch.zeros(rows, Wd.shape[1] if Wd is not None else own.shape[1], dtype=torch.float64, device=X.device)
        for tgt, src, val, peers in stages:
            op = own if peers is None else peers[which]
            opw = _matmul64(op, Wd) if Wd is not None else op.double()
            z += _spmm64(rows, tgt, src, val, opw)
        return z

    z1 = layer_sum(stages_fwd, X, W1d, 0)
    h = z1.clamp_min(0.0)
    z2 = layer_sum(stages_fwd, h, W2d, 1)
    logp = torch.log_softmax(z2, dim=1)
    cnt = int(mask.sum())
    loss = -(logp[torch.arange(rows, device=X.device), y] * mask.double()).sum() / cnt
    dz2 = torch.exp(logp)
    dz2[torch.arange(rows, device=X.device), y] -= 1.0
    dz2 *= (mask.double() / cnt)[:, None]
    ag2 = layer_sum(stages_bwd, dz2, None, 3)
    dw2 = h.t() @ ag2
    dz1 = (ag2 @ W2d.t()) * (z1 > 0).double()
    ag1 = layer_sum(stages_bwd, dz1, None, 2)
    dw1 = _xt_g64(X, ag1)
    return dict(loss=float(loss), hidden=h, outputs=logp, dw1=dw1, dw2=dw2, ag1=ag1, w1=W1d)


def _check_epoch(ref, x, w1, w2, h, out, loss, sample_seed):
    assert abs(float(loss) - ref["loss"]) <= 1e-4, (float(loss), ref["loss"])
    _close_rel_max(w2.grad, ref["dw2"], "dW2")
    _close_rel_max(w1.grad, ref["dw1"], "dW1")
    rows = torch.randint(0, x.shape[0], (256,), generator=torch.Generator().manual_seed(sample_seed)).to(x.device)
    _close_rel_max(h[rows], ref["hidden"][rows], "sampled rows of the hidden layer")
    _close_rel_max(out[rows], ref["outputs"][rows], "sampled rows of the outputs")
    _close_rel_max(x.grad[rows], ref["ag1"][rows] @ ref["w1"].t(), "sampled rows of dX")


@pytest.mark.parametrize("spec", [REDDIT, AMAZON], ids=["reddit", "amazon"])
def test_full_size_epoch_matches_fp64(cuda, spec):
    """Configurations 3 and 5: one forward + loss + backward of `train`'s model (gcn_distr.py:341-358)
    at the size the benchmark times, with the library's defaults (plans, fusion), against fp64."""
    from cagnet_amd import gcn, ops
    import torch.nn.functional as F
    if spec is AMAZON and torch.cuda.get_device_properties(cuda).total_memory < 200 * (1 << 30):
        pytest.skip("needs about 150 GB of device memory")
    p = synth.make_problem(n=spec["n"], target_nnz=spec["target_nnz"], features=spec["f"], hidden=spec["hidden"],
                           classes=spec["classes"], mask_fraction=0.66 if spec is REDDIT else 1.0, seed=0, device=cuda)
    n = p.n
    blk = ops.CsrMatrix(p.row.int(), p.col.int(), p.val, n, n, is_sorted=True, transpose=True)
    x = p.x.requires_grad_(True)
    w1 = p.w1.clone().requires_grad_(True)
    w2 = p.w2.clone().requires_grad_(True)
    h = gcn.GCNFunc.apply(x, w1, n, [blk], 0, 1, None, F.relu)
    z = gcn.GCNFunc.apply(h, w2, n, [blk], 0, 1, None, None)
    out, loss = gcn.LogSoftmaxNLLLoss.apply(z, p.y, p.train_mask)
    loss.backward()
    torch.cuda.synchronize()
    del blk
    # backward multiplies by A^T: row and column indices change places
    fwd = [(p.row, p.col, p.val, None)]
    bwd = [(p.col, p.row, p.val, None)]
    ref = _reference_epoch(fwd, bwd, p.x.detach(), p.w1, p.w2, p.y, p.train_mask, n)
    _check_epoch(ref, x, w1, w2, h.detach(), out.detach(), loss.detach(), 31)


def test_reddit_shape_grid_row_epoch_matches_fp64(cuda):
    """Configuration 4: forward and backward of both layers for the last process row of the 4 x 4 grid,
    four resident stages per product (gcn_distr_2d.py:333-417 without the broadcasts), against fp64."""
    from cagnet_amd import gcn, ops
    import torch.nn.functional as F
    spec = REDDIT
    q, r = 4, 3
    p = synth.make_problem(n=spec["n"], target_nnz=spec["target_nnz"], features=spec["f"], hidden=spec["hidden"],
                           classes=spec["classes"], mask_fraction=0.66, seed=0, device=cuda)
    b = synth.block_bounds_2d(p.n, q)
    rows = b[r + 1] - b[r]
    r32, c32 = p.row.int(), p.col.int()
    gen = torch.Generator(device=cuda).manual_seed(37)
    blocks, coo = [], []
    for k in range(q):
        br, bc, bv = ops.coo_block(r32, c32, p.val, b[r], b[r + 1], b[k], b[k + 1])
        blocks.append(ops.CsrMatrix(br, bc, bv, rows, b[k + 1] - b[k]))
        coo.append((br.long(), bc.long(), bv))
    del r32, c32

    def peers(width):
        return [None if k == r else torch.randn(b[k + 1] - b[k], width, device=cuda, generator=gen) for k in range(q)]

    p1f, p1b, p2f, p2b = peers(spec["f"]), peers(spec["hidden"]), peers(spec["hidden"]), peers(spec["classes"])
    x = p.x[b[r]:b[r + 1]].clone().requires_grad_(True)
    y, mask = p.y[b[r]:b[r + 1]], p.train_mask[b[r]:b[r + 1]]
    w1 = p.w1.clone().requires_grad_(True)
    w2 = p.w2.clone().requires_grad_(True)
    h = gcn.GCNFunc.apply(x, w1, rows, blocks, r, q, gcn.ResidentBlocks(p1f, p1b), F.relu)
    out = gcn.GCNFunc.apply(h, w2, rows, blocks, r, q, gcn.ResidentBlocks(p2f, p2b), F.log_softmax)
    loss = gcn.masked_nll_loss(out, y, mask)
    loss.backward()
    torch.cuda.synchronize()
    del blocks
    # per stage: (target rows, source rows, values, (layer-1 fwd, layer-2 fwd, layer-1 bwd, layer-2 bwd) operands)
    stages = [(coo[k][0], coo[k][1], coo[k][2], None if k == r else (p1f[k], p2f[k], p1b[k], p2b[k])) for k in range(q)]
    ref = _reference_epoch(stages, stages, x.detach(), p.w1, p.w2, y, mask, rows)
    _check_epoch(ref, x, w1, w2, h.detach(), out.detach(), loss.detach(), 41)
