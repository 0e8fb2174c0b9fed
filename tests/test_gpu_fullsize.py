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
