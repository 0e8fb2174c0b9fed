"""GPU parity of the input preparation (self-loops, normalisation, block extraction) through the
C ABI against the CPU oracle: integer results and the fp32 values are compared bit for bit."""
import numpy as np
import pytest
import torch

from tests.util import random_coo, small_graph
from oracle import gcn_oracle as orc

pytestmark = pytest.mark.gpu


def _i32(t, dev):
    return t.to(torch.int32).to(dev)


@pytest.mark.parametrize("n,nnz,seed", [(1, 1, 0), (1, 0, 0), (9, 30, 1), (300, 4000, 2), (5000, 3000, 3),
                                        (70000, 900000, 4)])
def test_add_self_loops_bit_exact(cuda, n, nnz, seed):
    from cagnet_amd import ops
    row, col, _ = random_coo(n, n, nnz, seed)          # holds some diagonal entries already, not all
    r, c = ops.add_self_loops(_i32(row, cuda), _i32(col, cuda), n)
    er, ec = orc.add_self_loops(row.numpy(), col.numpy(), n)
    assert np.array_equal(r.cpu().numpy(), er) and np.array_equal(c.cpu().numpy(), ec)


def test_add_self_loops_long_rows_and_full_diagonal(cuda):
    """Rows longer than a wavefront on both sides of the diagonal, and an input that already holds
    every self-loop (idempotence)."""
    from cagnet_amd import ops
    n = 700
    row, col, _ = random_coo(n, n, n * 400, 7)
    r, c = ops.add_self_loops(_i32(row, cuda), _i32(col, cuda), n)
    er, ec = orc.add_self_loops(row.numpy(), col.numpy(), n)
    assert np.array_equal(r.cpu().numpy(), er) and np.array_equal(c.cpu().numpy(), ec)
    r2, c2 = ops.add_self_loops(r, c, n)
    assert torch.equal(r2, r) and torch.equal(c2, c)


def test_add_self_loops_rejects_unsorted(cuda):
    from cagnet_amd import ops
    row = torch.tensor([1, 0], dtype=torch.int32, device=cuda)
    col = torch.tensor([0, 1], dtype=torch.int32, device=cuda)
    with pytest.raises(ops.CagnetError, match="CG_ERR_UNSORTED"):
        ops.add_self_loops(row, col, 2)


@pytest.mark.parametrize("scale,edges,seed", [(6, 200, 0), (11, 30000, 1), (14, 400000, 2)])
def test_gcn_normalize_bit_exact(cuda, scale, edges, seed):
    from cagnet_amd import ops
    row, col, val, n = small_graph(scale, edges, seed=seed)     # symmetric pattern with self-loops
    got, dinv = ops.gcn_normalize(_i32(row, cuda), _i32(col, cuda), n, return_dinv=True)
    expect = orc.gcn_normalize(row.numpy(), col.numpy(), n)
    assert np.array_equal(got.cpu().numpy(), expect)
    assert np.array_equal(got.cpu().numpy(), val.numpy())       # the generator's own values
    deg = np.bincount(row.numpy(), minlength=n).astype(np.float64)
    assert np.array_equal(dinv.cpu().numpy(), np.power(deg, -0.5).astype(np.float32))


def test_gcn_normalize_any_order_and_isolated_vertices(cuda):
    from cagnet_amd import ops
    # vertex 3 has no entries: its factor is +inf like the reference's pow, and no value uses it
    row = torch.tensor([2, 0, 1, 0, 2, 1, 4], dtype=torch.int32)
    col = torch.tensor([2, 1, 0, 0, 1, 1, 4], dtype=torch.int32)
    got, dinv = ops.gcn_normalize(row.to(cuda), col.to(cuda), 5, return_dinv=True)
    assert np.array_equal(got.cpu().numpy(), orc.gcn_normalize(row.numpy(), col.numpy(), 5))
    assert torch.isinf(dinv[3])


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_coo_block_bit_exact(cuda, seed):
    from cagnet_amd import ops
    n, m = 3000, 2500
    row, col, val = random_coo(n, m, 200000, seed)
    rng = np.random.default_rng(seed)
    r0, r1 = sorted(rng.integers(0, n + 1, size=2).tolist())
    c0, c1 = sorted(rng.integers(0, m + 1, size=2).tolist())
    r, c, v = ops.coo_block(_i32(row, cuda), _i32(col, cuda), val.to(cuda), r0, r1, c0, c1)
    er, ec, ev = orc.coo_block(row.numpy(), col.numpy(), val.numpy(), r0, r1, c0, c1)
    assert np.array_equal(r.cpu().numpy(), er) and np.array_equal(c.cpu().numpy(), ec)
    assert np.array_equal(v.cpu().numpy(), ev)


def test_coo_block_grid_partition_covers_matrix(cuda):
    """The 4 x 4 blocks of the 2D partition (remainder in the last block) hold every entry once,
    and an empty range gives an empty block."""
    from cagnet_amd import ops, synth
    row, col, val, n = small_graph(11, 30000, seed=3)
    b = synth.block_bounds_2d(n, 4)
    dr, dc, dv = _i32(row, cuda), _i32(col, cuda), val.to(cuda)
    total = 0
    for i in range(4):
        for j in range(4):
            r, c, v = ops.coo_block(dr, dc, dv, b[i], b[i + 1], b[j], b[j + 1])
            er, ec, ev = orc.coo_block(row.numpy(), col.numpy(), val.numpy(), b[i], b[i + 1], b[j], b[j + 1])
            assert np.array_equal(r.cpu().numpy(), er) and np.array_equal(c.cpu().numpy(), ec)
            assert np.array_equal(v.cpu().numpy(), ev)
            total += r.numel()
    assert total == row.numel()
    r, c, v = ops.coo_block(dr, dc, None, 5, 5, 0, n)
    assert r.numel() == 0 and v is None


def test_prepared_graph_feeds_spmm(cuda):
    """Raw pattern -> self-loops -> normalisation -> CSR handle -> product, all on the device,
    against the oracle chain on the host."""
    from cagnet_amd import ops
    from tests.util import REL_TOL, spmm_error
    n = 2000
    row, col, _ = random_coo(n, n, 30000, 11)
    r, c = ops.add_self_loops(_i32(row, cuda), _i32(col, cuda), n)
    v = ops.gcn_normalize(r, c, n)
    A = ops.CsrMatrix(r, c, v, n, n)
    B = torch.randn(n, 24, generator=torch.Generator().manual_seed(1))
    er, ec = orc.add_self_loops(row.numpy(), col.numpy(), n)
    ev = orc.gcn_normalize(er, ec, n)
    got = A.spmm(B.to(cuda))
    assert spmm_error(got, torch.from_numpy(er), torch.from_numpy(ec), torch.from_numpy(ev), n, n, B) <= REL_TOL
