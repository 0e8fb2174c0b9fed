"""Committed golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py):
the oracle must keep reproducing them (CPU), and the HIP path must match them (GPU)."""
from pathlib import Path

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import csr_ref
from oracle import gcn_oracle as orc
from tests.util import LOSS_TOL, REL_TOL

GOLD = Path(__file__).resolve().parent / "golden"
GRAPHS = ["graph_s6_f5", "graph_s8_f41"]


def _load(name):
    return np.load(GOLD / f"{name}.npz", allow_pickle=False)


@pytest.mark.parametrize("name", GRAPHS)
def test_oracle_reproduces_graph_vectors(name):
    g = _load(name)
    n = int(g["n"])
    rp, ci, vv, perm = orc.coo2csr(g["row_shuffled"], g["col_shuffled"], g["val_shuffled"], n, n)
    assert all(np.array_equal(a, g[k]) for a, k in ((rp, "rowptr"), (ci, "colind"), (vv, "values"), (perm, "perm")))
    cp, ri, vt, pt = csr_ref.csr_transpose(rp, ci, vv, n, n)    # the C restatement, not the Python one
    assert all(np.array_equal(a, g[k]) for a, k in ((cp, "colptr"), (ri, "rowind"), (vt, "values_t"), (pt, "perm_t")))
    wide = csr_ref.csr_spmm(rp, ci, vv, n, n, g["B"], g["C0"], beta=1.0, wide=True)
    assert np.max(np.abs(wide - g["C_out_f64"]) / g["magnitude_f64"]) < 2e-7
    assert np.array_equal(g["rowptr"], g["colptr"]) and np.array_equal(g["colind"], g["rowind"])  # symmetric graph


def test_oracle_reproduces_training_vectors():
    g = _load("train_s7")
    n = int(g["n"])
    A = orc.coo_tensor(g["row"], g["col"], g["val"], n, n, torch.float64)
    t = lambda k: torch.from_numpy(g[k])
    losses, _, _ = orc.train_epochs(t("x"), t("w1"), t("w2"), [A], t("y"), t("mask"), 20, dtype=torch.float64)
    assert np.allclose(losses, g["sgd_losses_f64"], rtol=0, atol=1e-12)
    assert abs(losses[0] - float(g["loss0"])) < 1e-12


@pytest.mark.gpu
@pytest.mark.parametrize("name", GRAPHS)
def test_gpu_matches_graph_vectors(cuda, name):
    from cagnet_amd import ops
    from cagnet_amd.sparse_coo_tensor_cpp import coo2csr, spmm_gpu
    g = _load(name)
    n = int(g["n"])
    d = lambda k: torch.from_numpy(g[k]).to(cuda)
    rp, ci, vv = coo2csr(d("row_shuffled"), d("col_shuffled"), d("val_shuffled"), n, n)
    assert np.array_equal(rp.cpu().numpy(), g["rowptr"]) and np.array_equal(ci.cpu().numpy(), g["colind"])
    assert np.array_equal(vv.cpu().numpy(), g["values"])
    cp, ri, vt, pt = ops.csr_transpose(rp, ci, vv, n, n, return_perm=True)
    assert np.array_equal(cp.cpu().numpy(), g["colptr"]) and np.array_equal(ri.cpu().numpy(), g["rowind"])
    assert np.array_equal(vt.cpu().numpy(), g["values_t"]) and np.array_equal(pt.cpu().numpy(), g["perm_t"])
    row = torch.from_numpy(orc.csr_expand_rows(g["rowptr"]).astype(np.int32)).to(cuda)
    C = d("C0").clone()
    spmm_gpu(row, ci, vv, n, n, d("B"), C)
    err = np.max(np.abs(C.cpu().double().numpy() - g["C_out_f64"]) / g["magnitude_f64"])
    assert err <= REL_TOL
    A = ops.CsrMatrix(d("row_shuffled"), d("col_shuffled"), d("val_shuffled"), n, n, is_sorted=False, transpose=True)
    for tr in (False, True):
        C = d("C0").clone()
        A.spmm(d("B"), out=C, beta=1.0, transpose=tr)
        assert np.max(np.abs(C.cpu().double().numpy() - g["C_out_f64"]) / g["magnitude_f64"]) <= REL_TOL


@pytest.mark.gpu
def test_gpu_matches_training_vectors(cuda):
    from cagnet_amd import gcn, ops
    g = _load("train_s7")
    n = int(g["n"])
    d = lambda k: torch.from_numpy(g[k]).to(cuda)
    blk = ops.CsrMatrix(d("row"), d("col"), d("val"), n, n, transpose=True)
    x = d("x").requires_grad_(True)
    w1, w2 = d("w1").requires_grad_(True), d("w2").requires_grad_(True)
    h = gcn.GCNFunc.apply(x, w1, n, [blk], 0, 1, None, F.relu)
    out = gcn.GCNFunc.apply(h, w2, n, [blk], 0, 1, None, F.log_softmax)
    loss = gcn.masked_nll_loss(out, d("y"), d("mask"))
    loss.backward()
    assert abs(float(loss.detach()) - float(g["loss0"])) <= LOSS_TOL
    for got, key in ((out, "outputs_f64"), (w1.grad, "dw1_f64"), (w2.grad, "dw2_f64"), (x.grad, "dx_f64")):
        ref = g[key]
        assert np.max(np.abs(got.detach().cpu().double().numpy() - ref)) <= 1e-5 * max(1.0, np.abs(ref).max()), key

    class Data:
        y, train_mask = d("y"), d("mask")

    w1, w2 = d("w1").requires_grad_(True), d("w2").requires_grad_(True)
    opt = torch.optim.SGD([w1, w2], lr=0.01)
    losses = []
    for _ in range(20):
        gcn.train(d("x"), w1, w2, n, [blk], opt, Data, 0, 1, None)
        losses.append(float(gcn.train.last_loss))
    assert np.max(np.abs(np.array(losses) - g["sgd_losses_f64"])) <= LOSS_TOL


def test_oracle_reproduces_preparation_and_blob_vectors():
    g = _load("prep_n97")
    n = int(g["n"])
    lr, lc = orc.add_self_loops(g["row"], g["col"], n)
    assert np.array_equal(lr, g["loops_row"]) and np.array_equal(lc, g["loops_col"])
    already = int(np.count_nonzero(g["row"] == g["col"]))
    assert 0 < already < n and len(lr) == len(g["row"]) - already + n   # some diagonal entries were there, not all
    val = orc.gcn_normalize(lr, lc, n)
    assert np.array_equal(val, g["values"])
    b = [int(v) for v in g["bounds"]]
    br, bc, bv = orc.coo_block(lr, lc, val, b[1], b[2], b[2], b[3])
    assert np.array_equal(br, g["block_row"]) and np.array_equal(bc, g["block_col"]) and np.array_equal(bv, g["block_val"])
    rp, ci, vv, nn, mm, has_t = orc.blob_read(g["blob"].tobytes())
    assert (nn, mm, has_t) == (n, n, True) and np.array_equal(vv, val)
    assert np.array_equal(orc.csr_expand_rows(rp), lr) and np.array_equal(ci, lc)


@pytest.mark.gpu
def test_gpu_matches_preparation_and_blob_vectors(cuda):
    from cagnet_amd import ops
    g = _load("prep_n97")
    n = int(g["n"])
    d = lambda k: torch.from_numpy(g[k]).to(cuda)
    lr, lc = ops.add_self_loops(d("row"), d("col"), n)
    assert np.array_equal(lr.cpu().numpy(), g["loops_row"]) and np.array_equal(lc.cpu().numpy(), g["loops_col"])
    val = ops.gcn_normalize(lr, lc, n)
    assert np.array_equal(val.cpu().numpy(), g["values"])
    b = [int(v) for v in g["bounds"]]
    br, bc, bv = ops.coo_block(lr, lc, val, b[1], b[2], b[2], b[3])
    assert np.array_equal(br.cpu().numpy(), g["block_row"]) and np.array_equal(bc.cpu().numpy(), g["block_col"])
    assert np.array_equal(bv.cpu().numpy(), g["block_val"])
    A = ops.CsrMatrix(lr, lc, val, n, n, transpose=True)
    assert np.array_equal(A.to_blob(), g["blob"])
    A2 = ops.CsrMatrix.from_blob(g["blob"])
    assert all(torch.equal(x, y) for x, y in zip(A2.arrays(), A.arrays()))
