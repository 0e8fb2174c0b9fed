"""Pins the CPU oracle (oracle/gcn_oracle.py, oracle/csr_ref.c) against independent library
routines, closed forms and brute force.  The reference ships no tests or golden vectors, so these
checks are what the parity claims rest on; each is chosen so that a plausible mistake (an
off-by-one in rowptr, a transposed operand, a dropped beta, a wrong sign in a gradient) fails it."""
import math

import numpy as np
import pytest
import scipy.sparse as sp
import torch
import torch.nn.functional as F
from hypothesis import given, settings, strategies as st

from cagnet_amd import synth
from oracle import csr_ref
from oracle import gcn_oracle as orc
from tests.util import random_coo, small_graph


# ---------------------------------------------------------------------------------- coo2csr
def _rand_sorted_rows(n, nnz, seed):
    rng = np.random.default_rng(seed)
    return np.sort(rng.integers(0, n, size=nnz)).astype(np.int32)


@pytest.mark.parametrize("n,nnz,seed", [(1, 0, 0), (1, 5, 1), (10, 0, 2), (10, 3, 3), (1000, 5000, 4), (50000, 70000, 5)])
def test_rowptr_against_closed_form_scipy_torch_and_c(n, nnz, seed):
    row = _rand_sorted_rows(n, nnz, seed)
    got = orc.coo2csr_rowptr(row, n)
    # closed form: rowptr[i] = lower_bound(row, i)
    assert np.array_equal(got, np.searchsorted(row, np.arange(n + 1), side="left").astype(np.int32))
    # scipy
    col = np.zeros(nnz, dtype=np.int32)
    a = sp.coo_matrix((np.ones(nnz), (row, col)), shape=(n, 1))
    csr = sp.csr_matrix((np.ones(nnz), col, got), shape=(n, 1))
    assert np.array_equal(np.asarray(csr.sum(axis=1)).ravel(), np.asarray(a.sum(axis=1)).ravel())
    assert np.array_equal(np.diff(got), np.bincount(row, minlength=n))
    # torch's own compression
    crow = torch._convert_indices_from_coo_to_csr(torch.from_numpy(row.astype(np.int64)), n).numpy()
    assert np.array_equal(got, crow.astype(np.int32))
    # the C restatement
    assert np.array_equal(got, csr_ref.coo2csr_rowptr(row, n))
    assert got[0] == 0 and got[-1] == nnz and np.all(np.diff(got) >= 0)


@settings(max_examples=200, deadline=None)
@given(st.integers(1, 12), st.lists(st.integers(0, 11), max_size=40))
def test_rowptr_brute_force(n, rows):
    rows = sorted(r for r in rows if r < n)
    got = orc.coo2csr_rowptr(np.array(rows, dtype=np.int32), n)
    for i in range(n + 1):
        assert got[i] == sum(1 for r in rows if r < i)


@pytest.mark.parametrize("n,m,nnz,seed", [(1, 1, 1, 0), (13, 7, 40, 1), (300, 700, 5000, 2), (4096, 4096, 60000, 3)])
def test_coo2csr_against_scipy_and_torch(n, m, nnz, seed):
    row, col, val = random_coo(n, m, nnz, seed, sort=False)
    rp, ci, vv, perm = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    ref = sp.coo_matrix((val.numpy(), (row.numpy(), col.numpy())), shape=(n, m)).tocsr()
    ref.sort_indices()
    assert np.array_equal(rp, ref.indptr) and np.array_equal(ci, ref.indices) and np.array_equal(vv, ref.data)
    t = torch.sparse_coo_tensor(torch.stack([row, col]), val, (n, m)).coalesce()
    assert np.array_equal(ci, t.indices()[1].numpy()) and np.array_equal(vv, t.values().numpy())
    assert np.array_equal(rp, t.to_sparse_csr().crow_indices().numpy())
    assert np.array_equal(val.numpy()[perm], vv)


@pytest.mark.parametrize("n,m,nnz,seed", [(13, 7, 40, 1), (300, 700, 5000, 2), (700, 300, 5000, 3)])
def test_transpose_against_scipy_c_and_involution(n, m, nnz, seed):
    row, col, val = random_coo(n, m, nnz, seed)
    rp, ci, vv, _ = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    cp, ri, vt, perm = orc.csr_transpose(rp, ci, vv, n, m)
    ref = sp.csr_matrix((vv, ci, rp), shape=(n, m)).tocsc()
    ref.sort_indices()
    assert np.array_equal(cp, ref.indptr) and np.array_equal(ri, ref.indices) and np.array_equal(vt, ref.data)
    c = csr_ref.csr_transpose(rp, ci, vv, n, m)
    assert all(np.array_equal(x, y) for x, y in zip((cp, ri, vt, perm), c))
    rp2, ci2, vv2, _ = orc.csr_transpose(cp, ri, vt, m, n)
    assert np.array_equal(rp2, rp) and np.array_equal(ci2, ci) and np.array_equal(vv2, vv)


# ---------------------------------------------------------------------------------- SpMM
@pytest.mark.parametrize("n,m,nnz,f,seed", [(5, 4, 9, 3, 0), (200, 300, 4000, 16, 1), (300, 200, 4000, 41, 2)])
def test_spmm_against_scipy_dense_and_c(n, m, nnz, f, seed):
    row, col, val = random_coo(n, m, nnz, seed)
    g = torch.Generator().manual_seed(seed)
    B, C0 = torch.randn(m, f, generator=g), torch.randn(n, f, generator=g)
    got64 = orc.spmm(row, col, val, n, m, B, C0, torch.float64)
    a = sp.csr_matrix((val.double().numpy(), (row.numpy(), col.numpy())), shape=(n, m))
    ref = C0.double().numpy() + a @ B.double().numpy()
    assert np.allclose(got64.numpy(), ref, rtol=1e-13, atol=1e-13)
    dense = torch.zeros(n, m, dtype=torch.float64)
    dense[row, col] = val.double()
    assert torch.allclose(got64, C0.double() + dense @ B.double(), rtol=1e-13, atol=1e-13)
    # a transposed operand would fail here whenever n != m; beta dropped would lose C0
    rp, ci, vv, _ = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    c32 = csr_ref.csr_spmm(rp, ci, vv, n, m, B.numpy(), C0.numpy(), beta=1.0)
    cw = csr_ref.csr_spmm(rp, ci, vv, n, m, B.numpy(), C0.numpy(), beta=1.0, wide=True)
    got32 = orc.spmm(row, col, val, n, m, B, C0, torch.float32)
    mag = (orc.spmm_abs(row, col, val, n, m, B) + C0.double().abs()).numpy()
    assert np.max(np.abs(c32 - ref) / mag) < 1e-5
    assert np.max(np.abs(cw - ref) / mag) < 2e-7
    assert np.max(np.abs(got32.numpy() - ref) / mag) < 1e-5
    z = csr_ref.csr_spmm(rp, ci, vv, n, m, B.numpy(), C0.numpy(), beta=0.0, wide=True)
    assert np.max(np.abs(z - (ref - C0.double().numpy())) / mag) < 2e-7


def test_spmm_special_cases():
    n, f = 6, 3
    B = torch.arange(n * f, dtype=torch.float32).reshape(n, f)
    C0 = torch.ones(n, f)
    eye = torch.arange(n)
    assert torch.equal(orc.spmm(eye, eye, torch.ones(n), n, n, B, C0), C0 + B)
    # one dense row: C[2] = C0[2] + sum_j v_j B[j]
    v = torch.tensor([1.0, -2.0, 0.5, 4.0, 0.0, 3.0])
    out = orc.spmm(torch.full((n,), 2), eye, v, n, n, B, C0)
    assert torch.allclose(out[2], C0[2] + (v[:, None] * B).sum(0))
    assert torch.equal(out[[0, 1, 3, 4, 5]], C0[[0, 1, 3, 4, 5]])   # empty rows untouched
    # stage splitting: sum over column blocks equals the whole product
    row, col, val, nn = small_graph(8, 3000, 3)
    H = torch.randn(nn, 5, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    whole = orc.spmm(row, col, val, nn, nn, H, torch.zeros(nn, 5), torch.float64)
    b = orc.block_bounds_2d(nn, 4)
    blocks, dense = [], []
    for k in range(4):
        r, c, v2 = orc.coo_block(row.numpy(), col.numpy(), val.numpy(), 0, nn, b[k], b[k + 1])
        blocks.append(orc.coo_tensor(r, c, v2, nn, b[k + 1] - b[k], torch.float64))
        dense.append(H[b[k]:b[k + 1]])
    assert torch.allclose(orc.stage_loop(blocks, dense, torch.float64), whole, rtol=1e-12, atol=1e-14)


# ---------------------------------------------------------------------------------- GCNFunc / train
def _tiny_problem(seed=0, n_scale=6):
    return synth.make_problem(scale=n_scale, n_edges=300, features=10, hidden=6, classes=4, mask_fraction=0.7, seed=seed)


def test_gcnfunc_backward_against_plain_autograd():
    """The hand-written backward (recompute + three products) equals autograd through the plain
    composition log_softmax((A relu((A X) W1)) W2) for a symmetric A."""
    p = _tiny_problem()
    A = orc.coo_tensor(p.row, p.col, p.val, p.n, p.n, torch.float64)
    ref = orc.forward_backward(p.x, p.w1, p.w2, [A], p.y, p.train_mask, dtype=torch.float64)
    x = p.x.double().requires_grad_(True)
    w1 = p.w1.double().requires_grad_(True)
    w2 = p.w2.double().requires_grad_(True)
    Ad = A.to_dense()
    h = F.relu((Ad @ x) @ w1)
    out = F.log_softmax((Ad @ h) @ w2, dim=1)
    loss = F.nll_loss(out[p.train_mask], p.y[p.train_mask])
    loss.backward()
    assert abs(float(loss) - float(ref["loss"])) < 1e-12
    for name, t in (("dw1", w1.grad), ("dw2", w2.grad), ("dx", x.grad)):
        assert torch.allclose(ref[name], t, rtol=1e-10, atol=1e-12), name
    # closed form of the fused loss gradient: (softmax - onehot) * mask / |mask|
    sm = out.detach().exp()
    onehot = F.one_hot(p.y, 4).double()
    dz = (sm - onehot) * p.train_mask[:, None] / p.train_mask.sum()
    ag = Ad @ dz
    assert torch.allclose(ref["dw2"], h.detach().t() @ ag, rtol=1e-10, atol=1e-12)


def test_gcnfunc_backward_uses_given_backward_blocks():
    """Non-symmetric A: the gradient is only right when backward multiplies by A^T; with the same
    blocks (what the reference does, gcn_distr.py:326) it differs."""
    n = 40
    row, col, val = random_coo(n, n, 300, 5)
    A = orc.coo_tensor(row, col, val, n, n, torch.float64)
    At = A.t().coalesce()
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(n, 5, generator=g, dtype=torch.float64), torch.randn(5, 3, generator=g, dtype=torch.float64)
    xr = x.clone().requires_grad_(True)
    out = orc.gcn_layer(xr, w.clone().requires_grad_(True), [A], "relu", [At])
    out.sum().backward()
    xa = x.clone().requires_grad_(True)
    F.relu((A.to_dense() @ xa) @ w).sum().backward()
    assert torch.allclose(xr.grad, xa.grad, rtol=1e-10, atol=1e-12)
    xs = x.clone().requires_grad_(True)
    orc.gcn_layer(xs, w.clone().requires_grad_(True), [A], "relu").sum().backward()
    assert not torch.allclose(xs.grad, xa.grad, rtol=1e-3, atol=1e-6)


def test_gcnfunc_gradcheck():
    p = _tiny_problem(seed=2, n_scale=4)
    A = orc.coo_tensor(p.row, p.col, p.val, p.n, p.n, torch.float64)
    x = p.x.double().requires_grad_(True)
    w = p.w1.double().requires_grad_(True)
    for kind in ("none", "log_softmax"):
        assert torch.autograd.gradcheck(lambda a, b: orc.gcn_layer(a, b, [A], kind), (x, w), eps=1e-6, atol=1e-5)


def test_masked_nll_and_empty_mask():
    g = torch.Generator().manual_seed(1)
    out = F.log_softmax(torch.randn(9, 4, generator=g, dtype=torch.float64), dim=1).requires_grad_(True)
    y = torch.randint(0, 4, (9,), generator=g)
    mask = torch.tensor([1, 0, 1, 1, 0, 0, 1, 0, 1], dtype=torch.bool)
    loss = orc.masked_nll(out, y, mask)
    manual = -sum(float(out[i, y[i]]) for i in range(9) if mask[i]) / int(mask.sum())
    assert abs(float(loss) - manual) < 1e-14
    loss.backward()
    assert torch.count_nonzero(out.grad[~mask]) == 0
    assert torch.allclose(out.grad[mask].sum(), torch.tensor(-1.0, dtype=torch.float64))
    out2 = out.detach().clone().requires_grad_(True)
    empty = orc.masked_nll(out2, y, torch.zeros(9, dtype=torch.bool))
    empty.backward()
    assert float(empty) == 0.0 and torch.count_nonzero(out2.grad) == 0


def test_training_fp32_tracks_fp64_and_learns():
    p = synth.make_problem(scale=8, n_edges=2048, features=32, hidden=16, classes=4, seed=4)
    A = orc.coo_tensor(p.row, p.col, p.val, p.n, p.n)
    l32, _, _ = orc.train_epochs(p.x, p.w1, p.w2, [A], p.y, p.train_mask, 30, dtype=torch.float32)
    l64, _, _ = orc.train_epochs(p.x, p.w1, p.w2, [A], p.y, p.train_mask, 30, dtype=torch.float64)
    assert max(abs(a - b) for a, b in zip(l32, l64)) < 1e-4
    assert l64[-1] < l64[0]
    la, _, _ = orc.train_epochs(p.x, p.w1, p.w2, [A], p.y, p.train_mask, 30, optimizer="adam", dtype=torch.float64)
    assert la[-1] < l64[-1]  # Adam at the same rate moves further than plain SGD here


# ---------------------------------------------------------------------------------- input preparation
def test_normalisation_against_dense_fp64_and_symmetry():
    row, col, n = synth.rmat_graph(7, 600, 11)
    v_t = synth.gcn_normalize(row, col, n)
    v_np = orc.gcn_normalize(row.numpy(), col.numpy(), n)
    assert np.array_equal(v_t.numpy(), v_np)                     # two implementations, identical bits
    pattern = torch.zeros(n, n, dtype=torch.float64)
    pattern[row, col] = 1.0
    assert torch.equal(pattern, pattern.t()) and torch.all(pattern.diagonal() == 1)
    deg = pattern.sum(1)
    assert torch.equal(deg, torch.bincount(row, minlength=n).double())
    dense = deg.pow(-0.5)[:, None] * pattern * deg.pow(-0.5)[None, :]
    got = torch.zeros(n, n, dtype=torch.float64)
    got[row, col] = v_t.double()
    assert float((got - dense).abs().max() / dense.max()) < 3 * 2.0 ** -24   # three fp32 roundings
    g32 = torch.zeros(n, n)
    g32[row, col] = v_t
    assert torch.equal(g32, g32.t())                              # fp32 products commute: bitwise symmetric
    # torch.histc on [min, max] with n bins equals the per-row count the reference relies on
    assert torch.equal(torch.histc(row.double(), bins=n), deg)


@pytest.mark.parametrize("n,parts", [(10, 3), (232965, 16), (232965, 8), (7, 7), (100, 1)])
def test_block_bounds_1d(n, parts):
    b = orc.block_bounds_1d(n, parts)
    step = math.ceil(n / parts)
    assert b == synth.block_bounds_1d(n, parts)
    assert b[0] == 0 and b[-1] == n and all(y - x == step for x, y in zip(b[:-2], b[1:-1])) and 0 < b[-1] - b[-2] <= step


def test_block_bounds_2d_reddit_grid():
    b = orc.block_bounds_2d(232965, 4)
    assert b == synth.block_bounds_2d(232965, 4) == [0, 58241, 116482, 174723, 232965]
    assert [y - x for x, y in zip(b, b[1:])] == [58241, 58241, 58241, 58242]
    assert orc.block_bounds_2d(16, 4) == [0, 4, 8, 12, 16]
    r, c, v = orc.coo_block(np.array([0, 5, 5, 9]), np.array([1, 4, 8, 9]), np.array([1., 2., 3., 4.]), 4, 10, 4, 10)
    assert r.tolist() == [1, 1, 5] and c.tolist() == [0, 4, 5] and v.tolist() == [2., 3., 4.]


@pytest.mark.parametrize("n,nnz,seed", [(1, 1, 0), (9, 30, 1), (300, 4000, 2), (2000, 3000, 3)])
def test_add_self_loops_against_scipy(n, nnz, seed):
    """The diagonal is present exactly once whether or not the input held it: scipy's pattern of
    (A - diag(A)) + I, indices sorted."""
    row, col, _ = random_coo(n, n, nnz, seed)
    r, c = orc.add_self_loops(row.numpy(), col.numpy(), n)
    a = sp.coo_matrix((np.ones(row.numel()), (row.numpy(), col.numpy())), shape=(n, n)).tocsr()
    a.setdiag(0)
    a.eliminate_zeros()
    ref = (a + sp.identity(n, format="csr")).tocsr()
    ref.sort_indices()
    ref = ref.tocoo()
    assert np.array_equal(r, ref.row) and np.array_equal(c, ref.col)
    assert np.count_nonzero(r == c) == n


def test_inverse_sqrt_degree_forms_agree_after_fp32_rounding():
    """The device computes fl32(1 / sqrt(d)) with correctly rounded fp64 operations, the host
    restatements fl32(d ** -0.5) through pow: both round to the same fp32 value for every degree a
    graph of this size class can have (exhaustive over 1 .. 2^22)."""
    d = np.arange(1, (1 << 22) + 1, dtype=np.float64)
    a = (1.0 / np.sqrt(d)).astype(np.float32)
    b = np.power(d, -0.5).astype(np.float32)
    c = torch.from_numpy(d).pow(-0.5).to(torch.float32).numpy()
    assert np.array_equal(a, b) and np.array_equal(a, c)


@pytest.mark.parametrize("seed", [0, 1])
def test_coo_block_against_scipy_slicing(seed):
    n, m = 70, 90
    row, col, val = random_coo(n, m, 900, seed)
    r0, r1, c0, c1 = 13, 50, 30, 77
    r, c, v = orc.coo_block(row.numpy(), col.numpy(), val.numpy(), r0, r1, c0, c1)
    ref = sp.coo_matrix((val.numpy(), (row.numpy(), col.numpy())), shape=(n, m)).tocsr()[r0:r1, c0:c1].tocoo()
    order = np.lexsort((ref.col, ref.row))
    assert np.array_equal(r, ref.row[order]) and np.array_equal(c, ref.col[order])
    assert np.array_equal(v, ref.data[order])


def test_blob_roundtrip_layout_and_rejections():
    """Header fields sit at the documented offsets, arrays on 64-byte boundaries, and every kind
    of damage (magic, truncation, flipped payload bit, non-monotone rowptr, column out of range)
    is refused."""
    import struct
    n, m = 37, 50
    row, col, val = random_coo(n, m, 400, 5)
    rp, ci, vv, _ = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    blob = orc.blob_write(rp, ci, vv, n, m, True)
    assert blob[:8] == b"CGNTCSR\x00" and struct.unpack_from("<II", blob, 8) == (1, 1)
    assert struct.unpack_from("<qqq", blob, 16) == (n, m, 400)
    o_r, o_c, o_v, total = struct.unpack_from("<QQQQ", blob, 40)
    assert o_r == 128 and o_c % 64 == 0 and o_v % 64 == 0 and total == len(blob) and total % 64 == 0
    assert np.array_equal(np.frombuffer(blob, "<i4", n + 1, o_r), rp)
    got = orc.blob_read(blob)
    assert np.array_equal(got[0], rp) and np.array_equal(got[1], ci) and np.array_equal(got[2], vv)
    assert got[3:] == (n, m, True)
    for bad in (b"X" + blob[1:], blob[:len(blob) - 64], blob[:o_v + 3] + bytes([blob[o_v + 3] ^ 1]) + blob[o_v + 4:]):
        with pytest.raises(ValueError):
            orc.blob_read(bad)
    rp_bad = rp.copy(); rp_bad[3], rp_bad[4] = rp[4] + 1, rp[3]
    ci_bad = ci.copy(); ci_bad[7] = m
    for args in ((rp_bad, ci, vv), (rp, ci_bad, vv)):
        with pytest.raises(ValueError):
            orc.blob_read(orc.blob_write(*args, n, m, False))
    empty = orc.blob_read(orc.blob_write(np.zeros(4, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), 3, 9, False))
    assert empty[3:] == (3, 9, False) and empty[1].size == 0
