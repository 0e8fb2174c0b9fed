"""GPU parity of coo2csr / transpose / SpMM through the C ABI against the CPU oracle."""
import numpy as np
import pytest
import torch

from tests.util import REL_TOL, gemm_error, random_coo, small_graph, spmm_error
from oracle import gcn_oracle as orc

pytestmark = pytest.mark.gpu


def _i32(t, dev):
    return t.to(torch.int32).to(dev)


@pytest.mark.parametrize("n,nnz_per_row,seed", [(1, 1, 0), (7, 2, 1), (1000, 5, 2), (5000, 40, 3), (100000, 3, 4)])
def test_rowptr_sorted_bit_exact(cuda, n, nnz_per_row, seed):
    from cagnet_amd import ops
    row, col, val = random_coo(n, n, n * nnz_per_row, seed)
    got = ops.coo2csr_rowptr(_i32(row, cuda), n).cpu().numpy()
    assert np.array_equal(got, orc.coo2csr_rowptr(row.numpy(), n))


def test_rowptr_empty_rows_and_empty_matrix(cuda):
    from cagnet_amd import ops
    # long runs of empty rows (wave-cooperative fill) and rows only at the far end
    row = torch.tensor([3, 3, 500, 99998], dtype=torch.int32, device=cuda)
    got = ops.coo2csr_rowptr(row, 100000).cpu().numpy()
    assert np.array_equal(got, orc.coo2csr_rowptr(row.cpu().numpy(), 100000))
    got = ops.coo2csr_rowptr(torch.empty(0, dtype=torch.int32, device=cuda), 1000).cpu().numpy()
    assert np.array_equal(got, np.zeros(1001, dtype=np.int32))
    got = ops.coo2csr_rowptr(torch.empty(0, dtype=torch.int32, device=cuda), 0).cpu().numpy()
    assert np.array_equal(got, np.zeros(1, dtype=np.int32))


@pytest.mark.parametrize("n,m,nnz,seed", [(1, 1, 1, 0), (13, 7, 40, 1), (300, 70000, 50000, 2), (70000, 300, 50000, 3),
                                          (4096, 4096, 200000, 4), (1 << 17, 1 << 17, 600000, 5)])
def test_coo2csr_unsorted_bit_exact(cuda, n, m, nnz, seed):
    from cagnet_amd import ops
    row, col, val = random_coo(n, m, nnz, seed, sort=False)
    rp, ci, vv, perm = ops.coo2csr(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m, return_perm=True)
    erp, eci, evv, eperm = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    assert np.array_equal(rp.cpu().numpy(), erp)
    assert np.array_equal(ci.cpu().numpy(), eci)
    assert np.array_equal(perm.cpu().numpy(), eperm)
    assert np.array_equal(vv.cpu().numpy(), evv)  # values are moved, never recomputed: bit exact


def test_coo2csr_duplicates_keep_input_order(cuda):
    from cagnet_amd import ops
    row = torch.tensor([2, 0, 2, 2, 0, 1], dtype=torch.int32)
    col = torch.tensor([1, 3, 1, 0, 3, 2], dtype=torch.int32)
    val = torch.arange(6, dtype=torch.float32)
    rp, ci, vv, perm = ops.coo2csr(row.to(cuda), col.to(cuda), val.to(cuda), 3, 4, return_perm=True)
    erp, eci, evv, eperm = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), 3, 4)
    assert np.array_equal(perm.cpu().numpy(), eperm)
    assert np.array_equal(vv.cpu().numpy(), evv)
    assert np.array_equal(rp.cpu().numpy(), erp)


@pytest.mark.parametrize("n,m,nnz,seed", [(13, 7, 40, 1), (300, 70000, 50000, 2), (70000, 300, 50000, 3),
                                          (1 << 16, 1 << 16, 500000, 5)])
def test_csr_transpose_bit_exact_and_involution(cuda, n, m, nnz, seed):
    from cagnet_amd import ops
    row, col, val = random_coo(n, m, nnz, seed)
    rp, ci, vv, _ = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    d = [torch.from_numpy(a).to(cuda) for a in (rp, ci, vv)]
    cp, ri, vt, perm = ops.csr_transpose(d[0], d[1], d[2], n, m, return_perm=True)
    ecp, eri, evt, eperm = orc.csr_transpose(rp, ci, vv, n, m)
    assert np.array_equal(cp.cpu().numpy(), ecp)
    assert np.array_equal(ri.cpu().numpy(), eri)
    assert np.array_equal(vt.cpu().numpy(), evt)
    assert np.array_equal(perm.cpu().numpy(), eperm)
    # T(T(A)) == A
    rp2, ci2, vv2 = ops.csr_transpose(cp, ri, vt, m, n)
    assert np.array_equal(rp2.cpu().numpy(), rp)
    assert np.array_equal(ci2.cpu().numpy(), ci)
    assert np.array_equal(vv2.cpu().numpy(), vv)


@pytest.mark.parametrize("n,m,nnz,seed", [(1, 1, 1, 0), (13, 7, 40, 1), (200, 200, 20000, 6), (300, 70000, 50000, 2),
                                          (1 << 17, 1 << 17, 600000, 5)])
def test_conversions_without_permutation_and_in_place(cuda, n, m, nnz, seed):
    """Without a permutation output the values travel with the records; without values the keys travel
    alone; and outputs may be the input arrays themselves (a single-pass sort then goes through a copy)."""
    from cagnet_amd import ops
    from cagnet_amd._lib import lib
    from cagnet_amd.ops import _ptr, _stream, check
    row, col, val = random_coo(n, m, nnz, seed, sort=False)
    erp, eci, evv, _ = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    r, c, v = _i32(row, cuda), _i32(col, cuda), val.to(cuda)
    rp, ci, vv = ops.coo2csr(r, c, v, n, m)
    assert np.array_equal(rp.cpu().numpy(), erp) and np.array_equal(ci.cpu().numpy(), eci)
    assert np.array_equal(vv.cpu().numpy(), evv)
    rp0, ci0, none = ops.coo2csr(r, c, None, n, m)
    assert none is None and torch.equal(rp0, rp) and torch.equal(ci0, ci)
    assert torch.equal(r, _i32(row, cuda)) and torch.equal(c, _i32(col, cuda)) and torch.equal(v, val.to(cuda))  # inputs intact
    # in place: colind and values land in the arrays that held col and val
    c2, v2 = c.clone(), v.clone()
    rp2 = torch.empty(n + 1, dtype=torch.int32, device=cuda)
    check(lib.cg_coo2csr(_ptr(r), _ptr(c2), _ptr(v2), r.numel(), n, m, _ptr(rp2), _ptr(c2), _ptr(v2), None, _stream()),
          "cg_coo2csr")
    assert torch.equal(rp2, rp) and torch.equal(c2, ci) and torch.equal(v2, vv)
    # transpose, the same three ways
    ecp, eri, evt, _ = orc.csr_transpose(erp, eci, evv, n, m)
    cp, ri, vt = ops.csr_transpose(rp, ci, vv, n, m)
    assert np.array_equal(cp.cpu().numpy(), ecp) and np.array_equal(ri.cpu().numpy(), eri)
    assert np.array_equal(vt.cpu().numpy(), evt)
    cp0, ri0, none = ops.csr_transpose(rp, ci, None, n, m)
    assert none is None and torch.equal(cp0, cp) and torch.equal(ri0, ri)
    ci3, vv3 = ci.clone(), vv.clone()
    cp3 = torch.empty(m + 1, dtype=torch.int32, device=cuda)
    check(lib.cg_csr_transpose(_ptr(rp), _ptr(ci3), _ptr(vv3), ci3.numel(), n, m, _ptr(cp3), _ptr(ci3), _ptr(vv3), None,
                               _stream()), "cg_csr_transpose")
    assert torch.equal(cp3, cp) and torch.equal(ci3, ri) and torch.equal(vv3, vt)


def test_coo_check_reports(cuda):
    from cagnet_amd import ops
    ok_r = torch.tensor([0, 0, 1, 2], dtype=torch.int32, device=cuda)
    ok_c = torch.tensor([0, 2, 1, 0], dtype=torch.int32, device=cuda)
    ops.coo_check(ok_r, ok_c, 3, 3, require_sorted=2)
    with pytest.raises(ops.CagnetError, match="CG_ERR_INDEX"):
        ops.coo_check(ok_r, ok_c, 2, 3)
    with pytest.raises(ops.CagnetError, match="CG_ERR_INDEX"):
        ops.coo_check(ok_r, torch.tensor([0, -1, 1, 0], dtype=torch.int32, device=cuda), 3, 3)
    with pytest.raises(ops.CagnetError, match="CG_ERR_UNSORTED"):
        ops.coo_check(torch.tensor([0, 2, 1, 2], dtype=torch.int32, device=cuda), ok_c, 3, 3)
    with pytest.raises(ops.CagnetError, match="CG_ERR_UNSORTED"):
        ops.coo_check(ok_r, torch.tensor([2, 0, 1, 0], dtype=torch.int32, device=cuda), 3, 3, require_sorted=2)


WIDTHS = [1, 3, 16, 24, 41, 64, 100, 128, 300, 602, 1300]


@pytest.mark.parametrize("f", WIDTHS)
def test_spmm_handle_matches_oracle(cuda, f):
    """Power-law graph (R-MAT scale 11, degrees from 1 to hundreds) at every width class."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(11, 30000, seed=f)
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(f))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
    got = A.spmm(B.to(cuda))
    assert spmm_error(got, row, col, val, n, n, B) <= REL_TOL
    # accumulate form: C = C0 + A B (beta = 1), the reference operator's semantics
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(f + 1))
    C = C0.to(cuda).clone()
    A.spmm(B.to(cuda), out=C, beta=1.0)
    assert spmm_error(C, row, col, val, n, n, B, C0) <= REL_TOL


@pytest.fixture(params=[False, True], ids=["rebuild", "cached"])
def spmm_gpu(request, monkeypatch):
    """The drop-in operator in both of its modes: tables rebuilt on every call (cg_spmm_coo) and
    blocks recognised by digest (cg_spmm_coo_cached)."""
    from cagnet_amd import ops, sparse_coo_tensor_cpp as mod
    monkeypatch.setattr(mod, "cache_blocks", request.param)
    yield mod.spmm_gpu
    ops.coo_cache_clear()


@pytest.mark.parametrize("f", [16, 41, 602])
def test_spmm_gpu_one_shot_matches_oracle(cuda, spmm_gpu, f):
    row, col, val, n = small_graph(10, 20000, seed=100 + f)
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(f))
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(f + 1))
    C = C0.to(cuda).clone()
    ret = spmm_gpu(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, B.to(cuda), C)
    assert ret is None
    assert spmm_error(C, row, col, val, n, n, B, C0) <= REL_TOL
    assert C.is_contiguous()


@pytest.mark.parametrize("f", [16, 41, 602, 2600])
def test_spmm_gpu_one_shot_split_rows_and_reuse(cuda, spmm_gpu, f):
    """The one-shot operator rebuilds its tables in a reused arena on every call (or finds the
    block again by its digest): long rows (several segments), then a smaller matrix with empty
    rows on the same stream, then the first again; every result is checked, and the repeat is
    bit-identical to the first."""
    n, m = 40, 6000
    row, col, val = random_coo(n, m, n * 3000, seed=f)
    B = torch.randn(m, f, generator=torch.Generator().manual_seed(1))
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(2))
    args = (_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m, B.to(cuda))
    C = C0.to(cuda).clone()
    spmm_gpu(*args, C)
    assert spmm_error(C, row, col, val, n, m, B, C0) <= REL_TOL
    n2 = 300
    r2, c2, v2 = random_coo(n2, n2, 900, seed=f + 1)
    r2 = r2 // 3 * 3                       # two of every three rows are empty; still sorted
    B2 = torch.randn(n2, f, generator=torch.Generator().manual_seed(3))
    D0 = torch.randn(n2, f, generator=torch.Generator().manual_seed(4))
    D = D0.to(cuda).clone()
    spmm_gpu(_i32(r2, cuda), _i32(c2, cuda), v2.to(cuda), n2, n2, B2.to(cuda), D)
    assert spmm_error(D, r2, c2, v2, n2, n2, B2, D0) <= REL_TOL
    empty = torch.ones(n2, dtype=torch.bool)
    empty[r2.long()] = False
    assert torch.equal(D.cpu()[empty], D0[empty])      # beta = 1: rows without entries are untouched
    C2 = C0.to(cuda).clone()
    spmm_gpu(*args, C2)
    assert torch.equal(C, C2)


def test_spmm_gpu_one_shot_empty_inputs(cuda, spmm_gpu):
    e32 = torch.empty(0, dtype=torch.int32, device=cuda)
    B = torch.randn(9, 8, device=cuda)
    C0 = torch.randn(5, 8, device=cuda)
    C = C0.clone()
    spmm_gpu(e32, e32, torch.empty(0, device=cuda), 5, 9, B, C)   # no stored entries: C is unchanged
    assert torch.equal(C, C0)


def test_spmm_gpu_block_cache(cuda, tune):
    """cg_spmm_coo_cached: a block is recognised by content, not by address or tensor identity; a
    changed value is a different block; the result is the handle's, bit for bit; the least recently
    used block is dropped beyond the capacity; unsorted rows are reported at the first sighting."""
    from cagnet_amd import ops
    tune("spmm_hub", 1)     # every product takes a column-popularity plan, so every block is kept
    ops.coo_cache_clear()
    base = ops.coo_cache_info()
    n, f = 3000, 602
    row, col, val = random_coo(n, n, 90000, seed=11)
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(12))
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(13))
    Bd = B.to(cuda)
    r, c, v = _i32(row, cuda), _i32(col, cuda), val.to(cuda)

    def product(r, c, v):
        C = C0.to(cuda).clone()
        ops.spmm_coo(r, c, v, n, n, Bd, C, beta=1.0, cached=True)
        return C

    first = product(r, c, v)
    assert spmm_error(first, row, col, val, n, n, B, C0) <= REL_TOL
    again = product(r.clone(), c.clone(), v.clone())           # same content at other addresses
    assert torch.equal(first, again)
    pad = torch.zeros(r.numel() + 1, dtype=torch.int32, device=cuda)
    pad[1:] = r                                                 # 4-byte aligned only: the scalar digest agrees
    assert torch.equal(first, product(pad[1:], c, v))
    assert ops.coo_cache_info()["hits"] - base["hits"] == 2
    base["hits"] += 1
    info = ops.coo_cache_info()
    assert (info["blocks"], info["hits"] - base["hits"], info["misses"] - base["misses"]) == (1, 1, 1)
    handle = ops.CsrMatrix(r, c, v, n, n)
    assert torch.equal(first, handle.spmm(Bd, out=C0.to(cuda).clone(), beta=1.0))

    v2 = v.clone()
    v2[12345] += 1.0                                            # one value changed in place: another block
    val2 = v2.cpu()
    changed = product(r, c, v2)
    assert spmm_error(changed, row, col, val2, n, n, B, C0) <= REL_TOL
    assert not torch.equal(changed, first)
    assert ops.coo_cache_info()["blocks"] == 2
    swapped = c.clone()
    swapped[[0, 1]] = swapped[[1, 0]]                           # same multiset of entries, other order
    if not torch.equal(swapped, c):
        product(r, swapped, v)
        assert ops.coo_cache_info()["blocks"] == 3

    tune("coo_cache_blocks", 2)
    ops.coo_cache_clear()
    blocks = []
    for seed in (21, 22, 23):
        rr, cc, vv = random_coo(500, 500, 4000, seed=seed)
        blocks.append((_i32(rr, cuda), _i32(cc, cuda), vv.to(cuda), rr, cc, vv))
    Bs = torch.randn(500, 16, generator=torch.Generator().manual_seed(1))
    before = ops.coo_cache_info()
    for k in (0, 1, 2, 0):                                       # 0 is evicted by 2 and rebuilt
        rr, cc, vv, hr, hc, hv = blocks[k]
        C = torch.zeros(500, 16, device=cuda)
        ops.spmm_coo(rr, cc, vv, 500, 500, Bs.to(cuda), C, beta=0.0, cached=True)
        assert spmm_error(C, hr, hc, hv, 500, 500, Bs, None) <= REL_TOL
    after = ops.coo_cache_info()
    assert after["blocks"] == 2
    assert after["misses"] - before["misses"] == 4 and after["hits"] == before["hits"]
    assert after["evictions"] - before["evictions"] == 2

    bad = torch.tensor([5, 3, 7], dtype=torch.int32, device=cuda)  # rows descend
    ones = torch.ones(3, device=cuda)
    with pytest.raises(ops.CagnetError):
        ops.spmm_coo(bad, bad, ones, 10, 10, torch.zeros(10, 4, device=cuda), torch.zeros(10, 4, device=cuda),
                     cached=True)
    ops.coo_cache_clear()
    assert ops.coo_cache_info()["blocks"] == 0


@pytest.mark.parametrize("f", [16, 41, 128, 602])
def test_spmm_split_rows(cuda, f):
    """Rows longer than a segment (1024 to 4096 entries by width class) are split over several
    wavefronts and recombined in order: a dense-ish rectangular block whose 40 rows hold ~9000
    entries each exercises the partial-row path at every class."""
    from cagnet_amd import ops
    n, m = 40, 12000
    row, col, val = random_coo(n, m, n * 9000, seed=f)
    B = torch.randn(m, f, generator=torch.Generator().manual_seed(1))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
    got = A.spmm(B.to(cuda))
    assert spmm_error(got, row, col, val, n, m, B) <= REL_TOL
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(2))
    C = C0.to(cuda).clone()
    A.spmm(B.to(cuda), out=C, beta=1.0)
    assert spmm_error(C, row, col, val, n, m, B, C0) <= REL_TOL


def test_spmm_special_cases(cuda):
    from cagnet_amd import ops
    n, f = 257, 48
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(0)).to(cuda)
    eye = torch.arange(n, dtype=torch.int32, device=cuda)
    I = ops.CsrMatrix(eye, eye, torch.ones(n, device=cuda), n, n)
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(1)).to(cuda)
    C = C0.clone()
    I.spmm(B, out=C, beta=1.0)
    assert torch.equal(C, C0 + B)            # A = I: C = C0 + B exactly
    assert torch.equal(I.spmm(B), B)
    # empty rows leave C untouched under beta = 1 and become zero under beta = 0
    row = torch.tensor([5, 5, 200], dtype=torch.int32, device=cuda)
    col = torch.tensor([0, 9, 256], dtype=torch.int32, device=cuda)
    val = torch.tensor([1.0, 2.0, -1.0], device=cuda)
    S = ops.CsrMatrix(row, col, val, n, n)
    C = C0.clone()
    S.spmm(B, out=C, beta=1.0)
    expect = C0.clone()
    expect[5] += B[0] + 2.0 * B[9]
    expect[200] -= B[256]
    assert torch.allclose(C, expect, rtol=0, atol=1e-6)
    untouched = torch.ones(n, dtype=torch.bool)
    untouched[[5, 200]] = False
    assert torch.equal(C[untouched.to(cuda)], C0[untouched.to(cuda)])
    Z = S.spmm(B)
    assert torch.count_nonzero(Z[untouched.to(cuda)]) == 0
    # all-empty matrix
    E = ops.CsrMatrix(torch.empty(0, dtype=torch.int32, device=cuda), torch.empty(0, dtype=torch.int32, device=cuda),
                      torch.empty(0, device=cuda), n, n)
    assert torch.count_nonzero(E.spmm(B)) == 0


def test_spmm_transpose_and_symmetry(cuda):
    from cagnet_amd import ops
    # rectangular, non-symmetric: A^T G against the oracle on the transposed triplets
    n, m, f = 500, 1300, 41
    row, col, val = random_coo(n, m, 20000, seed=9)
    G = torch.randn(n, f, generator=torch.Generator().manual_seed(3))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m, transpose=True)
    got = A.spmm(G.to(cuda), transpose=True)
    order = np.lexsort((row.numpy(), col.numpy()))
    assert spmm_error(got, col[order], row[order], val[order], m, n, G) <= REL_TOL
    with pytest.raises(ops.CagnetError, match="CG_ERR_NO_TRANSPOSE"):
        ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m).spmm(G.to(cuda), transpose=True)
    # symmetric normalised graph: A^T G == A G bit for bit (same rows, same order)
    row, col, val, n = small_graph(10, 20000, seed=77)
    S = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, transpose=True)
    G = torch.randn(n, 16, generator=torch.Generator().manual_seed(4)).to(cuda)
    assert torch.equal(S.spmm(G), S.spmm(G, transpose=True))
    a, t = S.arrays(False), S.arrays(True)
    assert all(torch.equal(x, y) for x, y in zip(a, t))


def test_spmm_deterministic_and_linear(cuda):
    from cagnet_amd import ops
    row, col, val, n = small_graph(12, 32768, seed=5)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
    g = torch.Generator().manual_seed(6)
    B1, B2 = torch.randn(n, 602, generator=g).to(cuda), torch.randn(n, 602, generator=g).to(cuda)
    r1 = A.spmm(B1)
    assert torch.equal(r1, A.spmm(B1))       # fixed summation order: bit identical
    lin = A.spmm(B1 + B2)
    ref = r1 + A.spmm(B2)
    scale = (A.spmm(B1.abs()) + A.spmm(B2.abs())).clamp_min(1e-30)
    assert float(((lin - ref).abs() / scale).max()) <= 4e-6


def test_stage_splitting_invariance(cuda):
    """sum_k A[:, block k] H[block k] == A H: the local form of the 1D/2D stage loops."""
    from cagnet_amd import ops, synth
    row, col, val, n = small_graph(11, 30000, seed=8)
    f = 64
    H = torch.randn(n, f, generator=torch.Generator().manual_seed(7))
    bounds = synth.block_bounds_2d(n, 4)
    z = None
    for k in range(4):
        r, c, v = synth.coo_block(row, col, val, 0, n, bounds[k], bounds[k + 1])
        blk = ops.CsrMatrix(_i32(r, cuda), _i32(c, cuda), v.to(cuda), n, bounds[k + 1] - bounds[k])
        Hk = H[bounds[k]:bounds[k + 1]].to(cuda)
        z = blk.spmm(Hk) if z is None else blk.spmm(Hk, out=z, beta=1.0)
    assert spmm_error(z, row, col, val, n, n, H) <= REL_TOL


def test_from_torch_coo_takes_the_reference_block_type(cuda):
    """The reference keeps its blocks as torch.sparse_coo tensors, transposed and coalesced on the
    device (gcn_distr.py:493-512, :543-546); a handle is built straight from one, duplicates summed by
    the coalescing as torch does."""
    from cagnet_amd import ops
    n, m, f = 300, 200, 24
    row, col, val = random_coo(n, m, 4000, 17, sort=False)
    idx = torch.stack([torch.cat([row, row[:50]]), torch.cat([col, col[:50]])])          # 50 duplicates
    vals = torch.cat([val, val[:50]])
    blk = torch.sparse_coo_tensor(idx, vals, (n, m)).to(cuda)
    A = ops.CsrMatrix.from_torch_coo(blk.t(), transpose=True)                          # the drivers hold A^T
    assert A.shape == (m, n) and A.nnz == row.numel()
    B = torch.randn(n, f, device=cuda)
    dense = blk.to_dense().double()
    got = A.spmm(B)
    mag = dense.abs().t() @ B.double().abs()
    assert float(((got.double() - dense.t() @ B.double()).abs() / mag.clamp_min(1e-30)).max()) <= REL_TOL
    G = torch.randn(m, f, device=cuda)
    back = A.spmm(G, transpose=True)
    mag = dense.abs() @ G.double().abs()
    assert float(((back.double() - dense @ G.double()).abs() / mag.clamp_min(1e-30)).max()) <= REL_TOL


def test_spmm_rejects_bad_arguments(cuda):
    from cagnet_amd import ops
    row, col, val, n = small_graph(8, 2000, seed=1)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
    with pytest.raises(ValueError):
        A.spmm(torch.zeros(n + 1, 4, device=cuda))
    with pytest.raises(ValueError):
        A.spmm(torch.zeros(n, 4))             # CPU tensor: no CPU path
    with pytest.raises(TypeError):
        A.spmm(torch.zeros(n, 4, device=cuda, dtype=torch.float64))
    with pytest.raises(ops.CagnetError, match="CG_ERR_INDEX"):
        ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n - 1, n)
    with pytest.raises(ops.CagnetError, match="CG_ERR_UNSORTED"):
        ops.CsrMatrix(_i32(row.flip(0), cuda), _i32(col.flip(0), cuda), val.flip(0).to(cuda), n, n)
    # the same unsorted triplets are fine on the general path
    U = ops.CsrMatrix(_i32(row.flip(0), cuda), _i32(col.flip(0), cuda), val.flip(0).to(cuda), n, n, is_sorted=False)
    B = torch.randn(n, 16, generator=torch.Generator().manual_seed(2)).to(cuda)
    assert torch.equal(U.spmm(B), A.spmm(B))


@pytest.fixture
def tune():
    """Set schedule knobs for one test and put the built-in choices back afterwards."""
    from cagnet_amd._lib import lib
    touched = []

    def set_knob(key, value):
        assert lib.cg_tune_set(key.encode(), int(value)) == 0
        touched.append(key)

    yield set_knob
    for key in touched:
        lib.cg_tune_set(key.encode(), 0)


@pytest.mark.parametrize("groups,tiers", [(8, 1), (2, 1), (1, 1), (8, 2), (4, 3)])
@pytest.mark.parametrize("f", [602, 256, 300])
def test_spmm_hub_plan_matches_oracle(cuda, tune, f, groups, tiers):
    """Hub plan forced on a small power-law graph: hot columns dealt to XCD groups, cold class
    straight into C, hot partial rows folded in afterwards.  A 64 KB hot budget keeps only a few
    dozen columns hot, so all three classes of entries (hot, cold, rows without hot entries) occur."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(11, 60000, seed=300 + f)
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(f))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, transpose=True)
    plain = A.spmm(B.to(cuda))
    tune("spmm_hub", 1)
    tune("spmm_hub_kb", 64)
    tune("spmm_hub_groups", groups)
    tune("spmm_hub_tiers", tiers)
    got = A.spmm(B.to(cuda))
    assert spmm_error(got, row, col, val, n, n, B) <= REL_TOL
    assert torch.equal(got, A.spmm(B.to(cuda)))                       # deterministic
    scale = A.spmm(B.abs().to(cuda)).clamp_min(1e-30)
    assert float(((got - plain).abs() / scale).max()) <= 4e-6          # same sum, different order
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(f + 1))
    C = C0.to(cuda).clone()
    A.spmm(B.to(cuda), out=C, beta=1.0)
    assert spmm_error(C, row, col, val, n, n, B, C0) <= REL_TOL
    assert torch.equal(A.spmm(B.to(cuda), transpose=True), got)        # symmetric graph, same plan on A^T


def test_spmm_hub_plan_rectangular_and_all_hot(cuda, tune):
    from cagnet_amd import ops
    n, m, f = 700, 1500, 320
    row, col, val = random_coo(n, m, 60000, seed=12)
    B = torch.randn(m, f, generator=torch.Generator().manual_seed(5))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
    tune("spmm_hub", 1)
    tune("spmm_hub_kb", 16)
    assert spmm_error(A.spmm(B.to(cuda)), row, col, val, n, m, B) <= REL_TOL
    tune("spmm_hub_kb", 1 << 20)   # every column is hot: the cold class is empty
    assert spmm_error(A.spmm(B.to(cuda)), row, col, val, n, m, B) <= REL_TOL
    # long hot rows are split into segments as well
    n, m = 24, 6000
    row, col, val = random_coo(n, m, n * 5000, seed=13)
    B = torch.randn(m, f, generator=torch.Generator().manual_seed(6))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
    tune("spmm_hub_kb", 4096)
    assert spmm_error(A.spmm(B.to(cuda)), row, col, val, n, m, B) <= REL_TOL


@pytest.mark.parametrize("min_degree", [1, 40, 10 ** 6])
def test_spmm_hub_plan_short_rows_stay_cold(cuda, tune, min_degree):
    """Only rows with at least `spmm_hub_row` entries get hot entries (and partial rows); the
    others keep everything in the cold class.  Rows of 0..4 and of ~120 entries, thresholds below
    all, between the two kinds, and above all (no hot task at all)."""
    from cagnet_amd import ops
    n, m, f = 900, 1200, 300
    gen = torch.Generator().manual_seed(31)
    dense = torch.rand(n, m, generator=gen)
    keep = torch.where(torch.arange(n).unsqueeze(1) % 3 == 0, dense < 0.1, dense < 0.002)   # long rows, short rows
    keep[5] = False                                                                        # and an empty one
    row, col = keep.nonzero(as_tuple=True)
    val = torch.randn(row.numel(), generator=gen)
    B = torch.randn(m, f, generator=gen)
    C0 = torch.randn(n, f, generator=gen)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
    tune("spmm_hub", 1)
    tune("spmm_hub_kb", 64)
    tune("spmm_hub_row", min_degree)
    got = A.spmm(B.to(cuda))
    assert spmm_error(got, row, col, val, n, m, B) <= REL_TOL
    assert torch.equal(got[5], torch.zeros(f, device=cuda))
    C = C0.to(cuda).clone()
    A.spmm(B.to(cuda), out=C, beta=1.0)
    assert spmm_error(C, row, col, val, n, m, B, C0) <= REL_TOL


def test_spmm_hub_plan_is_declined_when_columns_are_not_skewed(cuda):
    """Built-in choice at a size where a plan is considered (>= 3e9 multiply-adds): with uniformly
    spread columns the first tier would hold a tenth of the entries, the plan is declined and the
    plain schedule computes the product; with power-law columns of the same size it is taken.  Both
    must match the oracle and repeat bit for bit."""
    from cagnet_amd import ops
    n, f = 100_000, 602
    gen = torch.Generator().manual_seed(41)
    B = torch.randn(n, f, generator=gen)
    Bd = B.to(cuda)
    per_row = 96                                                       # rows long enough to have hot entries
    row = torch.arange(n).repeat_interleave(per_row)
    sample = torch.randint(0, n, (3000,), generator=gen)               # rows checked against the oracle
    for skewed in (False, True):
        u = torch.rand(n * per_row, generator=gen)
        col = ((u ** 6) * n).long() if skewed else (u * n).long()      # u^6: a few columns take most entries
        key = torch.unique(row * n + col)                              # (row, col) ascending, duplicates dropped
        r, c = key // n, key % n
        v = torch.rand(key.numel(), generator=gen) + 0.5
        A = ops.CsrMatrix(_i32(r, cuda), _i32(c, cuda), v.to(cuda), n, n)
        got = A.spmm(Bd)
        assert torch.equal(got, A.spmm(Bd))
        assert key.numel() * f >= 3e9                                  # large enough for a plan to be considered
        tiers, panel, tile = A.info()["plan_tiers"], _panel_info(A)["state"], _tile_info(A, f)["state"]
        if skewed:                                                     # one of the plans takes the popular columns
            assert panel == 1 or tile == 1 or tiers >= 1, (panel, tile, tiers)
        else:                                                          # the panel plan was looked at and declined (or not
                                                                       # considered at this size); then the tile plan takes
            assert panel in (0, -1) and (tile == 1 or tiers == -1), (panel, tile, tiers)   # the product, or the hub plan declines too
        keep = torch.isin(r, sample)
        ref_rows = torch.unique(r[keep])
        remap = torch.full((n,), -1, dtype=torch.long)
        remap[ref_rows] = torch.arange(ref_rows.numel())
        err = spmm_error(got[ref_rows.to(cuda)], remap[r[keep]], c[keep], v[keep], ref_rows.numel(), n, B)
        assert err <= REL_TOL, (skewed, err)


def test_spmm_hub_plans_of_several_widths_on_one_handle(cuda, tune):
    """A handle keeps two hub plans (the hot-column count depends on the width); cycling through
    three widths exercises reuse and replacement, and every product stays bit-identical to its
    first evaluation."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(11, 60000, seed=77)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
    tune("spmm_hub", 1)
    tune("spmm_hub_kb", 64)
    Bs = {f: torch.randn(n, f, generator=torch.Generator().manual_seed(f)) for f in (602, 256, 128)}
    first = {}
    for f in (602, 256, 602, 128, 256, 602, 128):
        got = A.spmm(Bs[f].to(cuda))
        if f not in first:
            assert spmm_error(got, row, col, val, n, n, Bs[f]) <= REL_TOL
            first[f] = got
        else:
            assert torch.equal(got, first[f])


def _xw_error(got, row, col, val, n, m, B, W, C0=None, relu=False):
    """max |got - ref64| / (sum |a||b| (+|c0|)) |W|, ref64 = act((C0 + A B) W) in fp64."""
    B64, W64 = B.double(), W.double()
    C64 = torch.zeros(n, B.shape[1], dtype=torch.float64) if C0 is None else C0.double()
    ab = orc.spmm(row, col, val, n, m, B64, C64, torch.float64)
    ref = ab @ W64
    if relu:
        ref = ref.clamp_min(0.0)
    mag = (orc.spmm_abs(row, col, val, n, m, B64) + C64.abs()) @ W64.abs()
    return orc.max_rel_error(got, ref, mag)


@pytest.mark.parametrize("hub", [-1, 1])
@pytest.mark.parametrize("f,fo,relu", [(602, 16, True), (300, 24, False), (256, 7, True), (130, 41, False), (192, 64, False)])
def test_spmm_xw_fused_layer_product(cuda, tune, f, fo, relu, hub):
    """Z = act((acc + A B) W) in one pass against the fp64 oracle of the two separate products:
    plain and hub-plan schedules, with and without an accumulated input, and on A^T."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(11, 60000, seed=900 + f)
    g = torch.Generator().manual_seed(f + fo)
    B, W = torch.randn(n, f, generator=g), torch.randn(f, fo, generator=g)
    C0 = torch.randn(n, f, generator=g)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, transpose=True)
    tune("spmm_hub", hub)
    tune("spmm_hub_kb", 64)
    Z = A.spmm_xw(B.to(cuda), W.to(cuda), relu=relu)
    assert Z is not None and tuple(Z.shape) == (n, fo)
    assert _xw_error(Z, row, col, val, n, n, B, W, relu=relu) <= 2 * REL_TOL
    assert torch.equal(Z, A.spmm_xw(B.to(cuda), W.to(cuda), relu=relu))          # deterministic
    acc = C0.to(cuda)
    keep = acc.clone()
    Z2 = A.spmm_xw(B.to(cuda), W.to(cuda), relu=relu, acc=acc)
    assert _xw_error(Z2, row, col, val, n, n, B, W, C0=C0, relu=relu) <= 2 * REL_TOL
    assert torch.equal(acc, keep)                                                 # the accumulated input is only read
    assert torch.equal(A.spmm_xw(B.to(cuda), W.to(cuda), relu=relu, transpose=True), Z)   # symmetric graph
    # the separate kernels give the same numbers up to summation order
    two = ops.dense_xw(A.spmm(B.to(cuda)), W.to(cuda), relu=relu)
    scale = ops.dense_xw(A.spmm(B.abs().to(cuda)), W.abs().to(cuda)).clamp_min(1e-30)
    assert float(((Z - two).abs() / scale).max()) <= 8e-6


def test_spmm_xw_split_rows_and_unsupported_widths(cuda, tune):
    from cagnet_amd import ops
    # rows of ~4000 entries are split over several wavefronts: their epilogue runs in the reduce kernel
    n, m, f, fo = 40, 9000, 320, 16
    row, col, val = random_coo(n, m, n * 4000, seed=31)
    g = torch.Generator().manual_seed(5)
    B, W, C0 = torch.randn(m, f, generator=g), torch.randn(f, fo, generator=g), torch.randn(n, f, generator=g)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
    for hub in (-1, 1):
        tune("spmm_hub", hub)
        tune("spmm_hub_kb", 256)
        Z = A.spmm_xw(B.to(cuda), W.to(cuda), relu=True, acc=C0.to(cuda))
        assert _xw_error(Z, row, col, val, n, m, B, W, C0=C0, relu=True) <= 2 * REL_TOL
    tune("spmm_hub", 0)
    # narrow products have no fused form: the wrapper says so instead of computing something else
    assert A.spmm_xw(torch.randn(m, 64, device=cuda), torch.randn(64, 16, device=cuda)) is None
    assert A.spmm_xw(torch.randn(m, 602, device=cuda), torch.randn(602, 64, device=cuda)) is None     # W beyond the LDS budget
    with pytest.raises(ValueError):
        A.spmm_xw(B.to(cuda), torch.randn(f + 1, fo, device=cuda))
    # rows without entries: Z = act(acc W)
    e32 = torch.empty(0, dtype=torch.int32, device=cuda)
    E = ops.CsrMatrix(e32, e32, torch.empty(0, device=cuda), n, m)
    Z = E.spmm_xw(B.to(cuda), W.to(cuda), acc=C0.to(cuda))
    ref = C0.double() @ W.double()
    assert float((Z.cpu().double() - ref).abs().max()) <= 1e-4 * float(ref.abs().max())
    assert torch.count_nonzero(E.spmm_xw(B.to(cuda), W.to(cuda))) == 0


def test_blob_matches_format_restatement_and_roundtrips(cuda, tmp_path):
    """The library's bytes equal the oracle's independent writer bit for bit; a blob written by
    the oracle loads; a file round trip gives a handle whose products are bit-identical."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(10, 20000, seed=21)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, transpose=True)
    blob = A.to_blob()
    rp, ci, vv, _ = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, n)
    assert blob.tobytes() == orc.blob_write(rp, ci, vv, n, n, True)
    parsed = orc.blob_read(blob.tobytes())
    assert np.array_equal(parsed[1], ci) and parsed[5] is True
    B = torch.randn(n, 48, generator=torch.Generator().manual_seed(3)).to(cuda)
    A2 = ops.CsrMatrix.from_blob(orc.blob_write(rp, ci, vv, n, n, False))
    assert not A2.has_transpose and torch.equal(A2.spmm(B), A.spmm(B))
    path = tmp_path / "block.cgcsr"
    A.save(path)
    A3 = ops.CsrMatrix.load(path)
    assert A3.has_transpose and A3.shape == (n, n) and A3.nnz == A.nnz
    assert torch.equal(A3.spmm(B), A.spmm(B)) and torch.equal(A3.spmm(B, transpose=True), A.spmm(B, transpose=True))
    assert all(torch.equal(x, y) for x, y in zip(A3.arrays(), A.arrays()))
    # rectangular, empty rows at the end, and an empty block
    r2, c2, v2 = random_coo(50, 3000, 700, 4)
    R = ops.CsrMatrix(_i32(r2, cuda), _i32(c2, cuda), v2.to(cuda), 64, 3000)
    R2 = ops.CsrMatrix.from_blob(R.to_blob(), transpose=True)
    assert R2.has_transpose and all(torch.equal(x, y) for x, y in zip(R2.arrays(), R.arrays()))
    e32 = torch.empty(0, dtype=torch.int32, device=cuda)
    E = ops.CsrMatrix.from_blob(ops.CsrMatrix(e32, e32, torch.empty(0, device=cuda), 5, 7).to_blob())
    assert E.nnz == 0 and E.shape == (5, 7)


def test_blob_rejects_damage(cuda):
    from cagnet_amd import ops
    n, m = 40, 60
    row, col, val = random_coo(n, m, 500, 8)
    rp, ci, vv, _ = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    good = orc.blob_write(rp, ci, vv, n, m, False)
    ops.CsrMatrix.from_blob(good)
    cases = {
        "CG_ERR_UNSUPPORTED": b"X" + good[1:],
        "CG_ERR_SIZE": good[:len(good) - 64],
        "CG_ERR_INDEX": good[:200] + bytes([good[200] ^ 4]) + good[201:],
    }
    for err, blob in cases.items():
        with pytest.raises(ops.CagnetError, match=err):
            ops.CsrMatrix.from_blob(blob)
    rp_bad = rp.copy(); rp_bad[3], rp_bad[4] = rp[4] + 1, rp[3]
    with pytest.raises(ops.CagnetError, match="CG_ERR_UNSORTED"):
        ops.CsrMatrix.from_blob(orc.blob_write(rp_bad, ci, vv, n, m, False))
    ci_bad = ci.copy(); ci_bad[7] = m            # valid checksum, column outside the matrix
    with pytest.raises(ops.CagnetError, match="CG_ERR_INDEX"):
        ops.CsrMatrix.from_blob(orc.blob_write(rp, ci_bad, vv, n, m, False))
    with pytest.raises(ops.CagnetError, match="CG_ERR_SIZE"):
        ops.CsrMatrix.from_blob(good[:64])


def test_dense_offsets_beyond_int32(cuda):
    """Row-major operands with more than 2^31 elements (9.0 M rows x 256 floats = 9.2 GB each): a
    few stored entries that touch the first and the last rows exercise the 64-bit addressing of the
    gather, of the store and of the dense kernels without needing a large sparse matrix."""
    from cagnet_amd import ops
    n, f = 9_000_000, 256
    assert n * f > 2 ** 31
    gen = torch.Generator(device=cuda).manual_seed(3)
    B = torch.randn(n, f, device=cuda, generator=gen)
    rows = torch.tensor([0, 5, 4_500_000, n - 2, n - 1, n - 1], dtype=torch.int32, device=cuda)
    cols = torch.tensor([n - 1, 7, n - 3, 0, n - 1, 11], dtype=torch.int32, device=cuda)
    vals = torch.tensor([1.5, -2.0, 0.5, 3.0, -1.0, 2.0], device=cuda)
    order = torch.argsort(rows.long() * n + cols.long())
    rows, cols, vals = rows[order], cols[order], vals[order]
    A = ops.CsrMatrix(rows, cols, vals, n, n)
    C = A.spmm(B)
    expect = {}
    for r, c, v in zip(rows.tolist(), cols.tolist(), vals.tolist()):
        expect[r] = expect.get(r, 0) + v * B[c].double()
    for r, e in expect.items():
        assert float((C[r].double() - e).abs().max()) <= 1e-5 * float(e.abs().max())
    assert torch.count_nonzero(C[1]) == 0 and torch.count_nonzero(C[n - 3]) == 0
    # dense products over the same tall operand: compare the last rows / the reduction with torch
    W = torch.randn(f, 16, device=cuda, generator=gen)
    Z = ops.dense_xw(B, W)
    ref = B[n - 4:].double() @ W.double()
    assert float((Z[n - 4:].double() - ref).abs().max()) <= 1e-4 * float(ref.abs().max())
    G = torch.randn(n, 16, device=cuda, generator=gen)
    dX = ops.dense_gwt(G, W, out=C)                   # reuses the 9.2 GB buffer
    ref = G[n - 4:].double() @ W.double().t()
    assert float((dX[n - 4:].double() - ref).abs().max()) <= 1e-4 * float(ref.abs().max())
    G[: n - 1000] = 0                                  # X^T G then only sees the last 1000 rows
    dW = ops.dense_xtg(B, G)
    ref = B[n - 1000:].double().t() @ G[n - 1000:].double()
    assert float((dW.double() - ref).abs().max()) <= 1e-4 * float(ref.abs().max())
    del dX, C, G
    H = ops.relu_fwd(B)                                # elementwise kernels index the same 2.3e9 elements
    assert torch.equal(H[n - 1], B[n - 1].clamp_min(0)) and torch.equal(H[0], B[0].clamp_min(0))


def test_sparse_coo_tensor_gpu_on_device_tensors(cuda):
    """sparse_coo_tensor_gpu (sparse-extension/sparse_coo_tensor.cu:43-54) on device int64 indices, the
    way the 2D driver calls it (gcn_distr_2d.py:385-389): the result equals torch.sparse_coo_tensor's,
    shares the storage of its arguments (no copy, no validation pass), and feeds a handle."""
    from cagnet_amd import ops
    from cagnet_amd.sparse_coo_tensor_cpp import sparse_coo_tensor_gpu
    n, m, f = 211, 157, 20
    row, col, val = random_coo(n, m, 3000, 31)
    idx = torch.stack([row, col]).to(cuda)
    v = val.to(cuda)
    t = sparse_coo_tensor_gpu(idx, v, (n, m))
    assert t.is_sparse and t.device.type == "cuda" and tuple(t.shape) == (n, m)
    assert t._indices().dtype == torch.int64 and t._values().dtype == torch.float32
    assert t._indices().data_ptr() == idx.data_ptr() and t._values().data_ptr() == v.data_ptr()
    ref = torch.sparse_coo_tensor(idx, v, (n, m))
    assert torch.equal(t.to_dense(), ref.to_dense())
    assert t.sparse_dim() == 2 and t.dense_dim() == 0           # sparse_dim = indices.size(0), dense_dim = values.dim() - 1
    B = torch.randn(m, f, device=cuda)
    A = ops.CsrMatrix.from_torch_coo(t)
    assert spmm_error(A.spmm(B), row, col, val, n, m, B.cpu()) <= REL_TOL
    # an index that torch's validating constructor would reject passes unchecked, like the reference's
    bad = idx.clone()
    bad[0, 0] = n + 5
    assert sparse_coo_tensor_gpu(bad, v, (n, m))._nnz() == v.numel()
    # values with a dense dimension: dense_dim = values.dim() - 1
    tv = sparse_coo_tensor_gpu(idx, torch.randn(v.numel(), 3, device=cuda), (n, m, 3))
    assert tv.sparse_dim() == 2 and tv.dense_dim() == 1


def test_spmm_from_two_host_threads_on_two_streams(cuda, tune):
    """The digest-cached drop-in and the handle product called concurrently from two host threads,
    each on a stream of its own and on a matrix of its own: both results against the oracle.  (One
    handle serves one host thread at a time; the block cache is what two threads may share.)"""
    import threading
    from cagnet_amd import ops
    f = 96
    cases = []
    for seed in (41, 42):
        row, col, val, n = small_graph(11, 40000, seed=seed)
        B = torch.randn(n, f, generator=torch.Generator().manual_seed(seed))
        cases.append((row, col, val, n, B))
    results, errors = [None, None], []

    def work(k):
        try:
            row, col, val, n, B = cases[k]
            stream = torch.cuda.Stream(device=cuda)
            with torch.cuda.stream(stream):
                r32, c32, v, Bd = _i32(row, cuda), _i32(col, cuda), val.to(cuda), B.to(cuda)
                handle = ops.CsrMatrix(r32, c32, v, n, n)
                outs = []
                for _ in range(6):
                    C = torch.zeros(n, f, device=cuda)
                    ops.spmm_coo(r32, c32, v, n, n, Bd, C, beta=1.0, cached=True)
                    outs.append(C)
                    outs.append(handle.spmm(Bd))
                stream.synchronize()
            results[k] = outs
        except Exception as e:  # noqa: BLE001  (reported by the main thread)
            errors.append(e)

    tune("spmm_hub", 1)                          # the cached entry point only keeps blocks that take a plan
    try:
        threads = [threading.Thread(target=work, args=(k,)) for k in range(2)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    finally:
        ops.coo_cache_clear()
    assert not errors, errors
    for k in range(2):
        row, col, val, n, B = cases[k]
        for C in results[k]:
            assert spmm_error(C, row, col, val, n, n, B) <= REL_TOL
        assert all(torch.equal(results[k][0], C) for C in results[k][2::2])      # cached form: bit-identical repeats
        assert all(torch.equal(results[k][1], C) for C in results[k][3::2])      # handle form likewise


def _panel_info(A, transpose=False, narrow=False):
    import ctypes
    from cagnet_amd._lib import check, lib
    buf = (ctypes.c_int64 * 12)()
    check(lib.cg_csr_panel_info(A._handle, int(transpose) | (2 if narrow else 0), buf), "cg_csr_panel_info")   # bit 1: plan of the narrow products
    return dict(state=buf[0], covered=buf[1], tiles=buf[2], units=buf[3], split=buf[4], rest=buf[5], emin=buf[6], cols=buf[7],
                dense_covered=buf[8], dense_tiles=buf[9], dense_units=buf[10], dmin=buf[11])


@pytest.mark.parametrize("f", [258, 300, 384, 602, 636])
@pytest.mark.parametrize("emin,unit", [(4, 300), (24, 100000)])
def test_spmm_panel_plan_matches_oracle(cuda, tune, f, emin, unit):
    """Wide products with the panel plan forced on: dense (row panel, column block) tiles are multiplied
    out of LDS into partial rows, the other entries by the row-wise kernels, which add those rows in.
    Small units split the heavy panels over several workgroups (their partial blocks are then summed)."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(12, 120000, seed=7 * f + emin)
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(f))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, transpose=True)
    tune("spmm_panel", 1)
    tune("spmm_panel_emin", emin)
    tune("spmm_panel_cols", 1024)
    tune("spmm_panel_unit", unit)
    got = A.spmm(B.to(cuda))
    info = _panel_info(A)
    assert info["state"] == 1 and info["covered"] > 0
    assert info["covered"] + info["dense_covered"] + info["rest"] == row.numel()
    assert info["tiles"] > 0 and info["units"] >= 1
    if unit < 1000:
        assert info["split"] > 0
    assert spmm_error(got, row, col, val, n, n, B) <= REL_TOL
    assert torch.equal(got, A.spmm(B.to(cuda)))                      # fixed summation order
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(f + 1))
    C = C0.to(cuda).clone()
    A.spmm(B.to(cuda), out=C, beta=1.0)
    assert spmm_error(C, row, col, val, n, n, B, C0) <= REL_TOL
    gotT = A.spmm(B.to(cuda), transpose=True)                        # the graph is symmetric: same product
    assert _panel_info(A, transpose=True)["state"] == 1
    assert spmm_error(gotT, row, col, val, n, n, B) <= REL_TOL
    tune("spmm_panel", -1)
    plain = A.spmm(B.to(cuda))
    assert spmm_error(plain, row, col, val, n, n, B) <= REL_TOL


@pytest.mark.parametrize("f", [258, 384, 512, 514, 602, 636])
def test_spmm_panel_staged_tiles_through_either_kernel(cuda, tune, f):
    """The staged tiles of the panel plan go through the tile kernel (records as they are) or, with spmm_panel_legacy or
    for a B whose rows are not 8-byte aligned, through the older kernel on padded records: both against the fp64 oracle,
    each bit-identical on repeats, with accumulation into C."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(12, 140000, seed=5 * f)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(f))
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(f + 1))
    tune("spmm_panel", 1)
    tune("spmm_panel_dmin", 200)
    results = []
    for legacy in (0, 1, 0):
        tune("spmm_panel_legacy", legacy)
        got = A.spmm(B.to(cuda))
        info = _panel_info(A)
        assert info["state"] == 1 and info["covered"] > 0 and info["dense_tiles"] > 0 and info["rest"] == 0
        assert spmm_error(got, row, col, val, n, n, B) <= REL_TOL
        assert torch.equal(got, A.spmm(B.to(cuda)))
        C = C0.to(cuda).clone()
        A.spmm(B.to(cuda), out=C, beta=1.0)
        assert spmm_error(C, row, col, val, n, n, B, C0) <= REL_TOL
        results.append(got)
    assert torch.equal(results[0], results[2])                       # the plan is rebuilt the same way
    tune("spmm_panel_legacy", 0)
    wide = torch.zeros(n, f + 1, device=cuda)                         # rows 4 bytes off an 8-byte boundary when f is even
    wide[:, 1:] = B.to(cuda)
    odd = A.spmm(wide[:, 1:])
    assert spmm_error(odd, row, col, val, n, n, B) <= REL_TOL


@pytest.mark.parametrize("f", [258, 320, 384, 448, 512, 576, 602, 636])
@pytest.mark.parametrize("dmin,dwg", [(40, 3), (200, 0)])
def test_spmm_panel_dense_tiles_on_matrix_cores(cuda, tune, f, dmin, dwg):
    """The panel plan with its dense tiles forced on: (row panel, column block) tiles with at least dmin entries are
    stored whole and multiplied by v_mfma_f32_16x16x4_f32 (exact fp32 products); dwg workgroups (0: one per compute
    unit) share them equally, and the blocks of partial rows their units write are summed with those of the other
    units of the panel; every result width class
    (5..10 groups of 64 columns).  Same 1e-5 bound against the fp64 oracle, bit-identical repeats."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(12, 160000, seed=11 * f + dmin)
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(f))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, transpose=True)
    tune("spmm_panel", 1)
    tune("spmm_panel_emin", 8)
    tune("spmm_panel_cols", 2048)
    tune("spmm_panel_dmin", dmin)
    tune("spmm_panel_dwg", dwg)
    got = A.spmm(B.to(cuda))
    info = _panel_info(A)
    assert info["state"] == 1 and info["dmin"] == dmin
    assert info["dense_tiles"] > 0 and info["dense_covered"] >= dmin * info["dense_tiles"]
    assert info["dense_units"] >= (min(dwg, info["dense_tiles"]) if dwg else 1)
    assert info["covered"] + info["dense_covered"] + info["rest"] == row.numel()
    assert spmm_error(got, row, col, val, n, n, B) <= REL_TOL
    assert torch.equal(got, A.spmm(B.to(cuda)))                      # fixed summation order
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(f + 1))
    C = C0.to(cuda).clone()
    A.spmm(B.to(cuda), out=C, beta=1.0)
    assert spmm_error(C, row, col, val, n, n, B, C0) <= REL_TOL
    gotT = A.spmm(B.to(cuda), transpose=True)
    assert _panel_info(A, transpose=True)["dense_tiles"] > 0
    assert spmm_error(gotT, row, col, val, n, n, B) <= REL_TOL
    tune("spmm_panel_dmin", -1)                                      # the same plan without dense tiles
    rec = A.spmm(B.to(cuda))
    assert _panel_info(A)["dense_tiles"] == 0 and _panel_info(A)["dmin"] == 0
    assert spmm_error(rec, row, col, val, n, n, B) <= REL_TOL


@pytest.mark.parametrize("f", [1, 8, 16, 24, 41, 44, 48, 64])
@pytest.mark.parametrize("dmin,dwg", [(40, 3), (300, 0)])
def test_spmm_narrow_products_with_dense_tiles(cuda, tune, f, dmin, dwg):
    """Narrow products (f <= 64) with their panel plan forced on: tiles with at least dmin entries are multiplied on
    the fp32 matrix cores, the other entries by the row-wise kernels, and the partial rows are added to the result
    afterwards.  Same 1e-5 bound against the fp64 oracle, bit-identical repeats, accumulate form, A^T, strided
    operands; every entry is in the dense tiles or in the rest."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(12, 160000, seed=13 * f + dmin)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, transpose=True)
    tune("spmm_panel_narrow", 1)
    tune("spmm_panel_narrow_dmin", dmin)
    tune("spmm_panel_cols", 2048)
    tune("spmm_panel_dwg", dwg)
    g = torch.Generator().manual_seed(f)
    big = torch.randn(n, f + 3, generator=g).to(cuda)
    B = big[:, 1:1 + f]
    got = A.spmm(B)
    info = _panel_info(A, transpose=2)
    assert info["state"] == 1 and info["dense_tiles"] > 0 and info["tiles"] == 0 and info["covered"] == 0
    assert info["dense_covered"] + info["rest"] == row.numel() and info["dmin"] == dmin
    pi = A.panel_info(narrow=True)
    assert pi["state"] == 1 and pi["dense_entries"] == info["dense_covered"] and pi["rest_entries"] == info["rest"]
    assert spmm_error(got, row, col, val, n, n, B.cpu()) <= REL_TOL
    assert torch.equal(got, A.spmm(B))
    C0 = torch.randn(n, f, generator=g)
    Cbig = torch.zeros(n, f + 5, device=cuda)
    C = Cbig[:, 2:2 + f]
    C.copy_(C0)
    A.spmm(B, out=C, beta=1.0)
    assert spmm_error(C, row, col, val, n, n, B.cpu(), C0) <= REL_TOL
    assert float(Cbig[:, :2].abs().max()) == 0.0 and float(Cbig[:, 2 + f:].abs().max()) == 0.0
    gotT = A.spmm(B, transpose=True)
    assert _panel_info(A, transpose=3)["dense_tiles"] > 0
    assert spmm_error(gotT, row, col, val, n, n, B.cpu()) <= REL_TOL
    tune("spmm_panel_narrow", -1)
    plain = A.spmm(B)
    assert spmm_error(plain, row, col, val, n, n, B.cpu()) <= REL_TOL


def test_spmm_panel_all_tiles_dense_and_duplicate_entries(cuda, tune):
    """A small full matrix: every tile is dense and no unit of the record kind is left (also with a row count that is
    not a multiple of the panel height and B as a strided slice).  Then a matrix that stores some (row, column) pairs
    twice: two entries cannot share a place of a dense tile, so the plan falls back to records for every tile and the
    product still adds both."""
    from cagnet_amd import ops
    n, m, f = 300, 200, 602
    g = torch.Generator().manual_seed(3)
    dense = torch.randn(n, m, generator=g)
    row, col = torch.nonzero(torch.ones(n, m), as_tuple=True)
    val = dense[row, col].contiguous()
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m, transpose=True)
    tune("spmm_panel", 1)
    tune("spmm_panel_dmin", 512)
    big = torch.randn(m, f + 8, generator=g).to(cuda)
    B = big[:, 2:2 + f]
    got = A.spmm(B)
    info = _panel_info(A)
    assert info["state"] == 1 and info["dense_tiles"] > 0 and info["dense_covered"] > 0
    assert spmm_error(got, row, col, val, n, m, B.cpu()) <= REL_TOL
    assert gemm_error(got, dense, B.cpu()) <= REL_TOL
    G = torch.randn(n, f, generator=g).to(cuda)
    gotT = A.spmm(G, transpose=True)
    assert spmm_error(gotT, col, row, val, m, n, G.cpu()) <= REL_TOL
    # duplicates: rows stay sorted, some pairs appear twice
    rng = np.random.default_rng(9)
    r = np.sort(rng.integers(0, 256, 40000))
    c = rng.integers(0, 64, 40000)
    order = np.lexsort((c, r))
    r, c = torch.from_numpy(r[order]), torch.from_numpy(c[order])
    v = torch.from_numpy(rng.standard_normal(40000).astype(np.float32))
    try:
        D = ops.CsrMatrix(_i32(r, cuda), _i32(c, cuda), v.to(cuda), 256, 64)
    except Exception:
        pytest.skip("handles refuse duplicate (row, column) pairs")
    Bd = torch.randn(64, 300, generator=g).to(cuda)
    got = D.spmm(Bd)
    info = _panel_info(D)
    assert info["state"] == 1 and info["dense_tiles"] == 0 and info["covered"] > 0
    assert spmm_error(got, r, c, v, 256, 64, Bd.cpu()) <= REL_TOL


def test_spmm_panel_last_block_with_empty_places_and_columns_ranked_per_panel(cuda, tune):
    """Columns are ranked inside every panel, so a panel's last block can have fewer than 32 columns: 40 columns give
    one full block and one of 8, as a dense tile (1024 entries) and, with dense tiles off, as a staged one (the empty
    places name a column of the tile).  Second matrix: two panels whose busy columns interleave (the even columns
    0..62 in the first 128 rows, the odd columns 1..63 in the next 128, one stray entry per row elsewhere): each panel
    gets one full tile of its own 32 busy columns, where blocks of one ranking for the whole matrix would have given
    each panel two half-filled ones, and only the stray entries stay in the rest matrix."""
    from cagnet_amd import ops
    n, m, f = 128, 40, 300
    g = torch.Generator().manual_seed(12)
    dense = torch.randn(n, m, generator=g)
    row, col = torch.nonzero(torch.ones(n, m), as_tuple=True)
    val = dense[row, col].contiguous()
    B = torch.randn(m, f, generator=g)
    Bd = B.to(cuda)
    tune("spmm_panel", 1)
    for dmin, kind in ((0, "dense_tiles"), (-1, "tiles")):
        tune("spmm_panel_dmin", dmin)
        A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
        got = A.spmm(Bd)
        info = _panel_info(A)
        assert info["state"] == 1 and info[kind] == 2 and info["rest"] == 0, info
        assert gemm_error(got, dense, B) <= REL_TOL
    tune("spmm_panel_dmin", -1)
    tune("spmm_panel_emin", 64)                                         # a tile of 32 stray columns (32 entries) is not staged
    n, m = 256, 2000
    rng = np.random.default_rng(21)
    r = np.repeat(np.arange(n), 32)
    c = 2 * np.tile(np.arange(32), n) + np.where(r < 128, 0, 1)
    stray_c = 100 + rng.permutation(800)[:n]                            # one more entry per row, all in different columns
    key = np.unique(np.concatenate([r * m + c, np.arange(n) * m + stray_c]))
    row, col = torch.from_numpy(key // m), torch.from_numpy(key % m)
    val = torch.from_numpy(rng.standard_normal(key.size).astype(np.float32))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
    Bd = torch.randn(m, f, generator=g).to(cuda)
    got = A.spmm(Bd)
    info = _panel_info(A)
    assert info["state"] == 1 and info["tiles"] == 2 and info["covered"] == n * 32 and info["rest"] == n, info
    assert spmm_error(got, row, col, val, n, m, Bd.cpu()) <= REL_TOL


def test_spmm_panel_single_block_panels_write_c_themselves(cuda, tune):
    """A panel whose tiles are one staged unit has a single block of partial rows: that unit writes its rows of C
    (in the order of the rows' ranks) and the pass over the partial rows leaves them alone.  Five panels (one of 60
    rows, rows without entries among them), one heavy enough for several units; C is a column slice of a wider
    matrix and is read only where beta asks for it: full of NaN for beta = 0, then beta = -0.5 on known values,
    and what lies beside the slice stays as it was."""
    from cagnet_amd import ops
    n, m, f = 572, 2400, 262                                            # 75 column blocks: units are cut every 32
    rng = np.random.default_rng(33)
    deg = np.where(np.arange(n) < 128, 300, rng.integers(0, 12, n))    # first panel: 38,400 entries, the others light
    r = np.repeat(np.arange(n), deg)
    c = np.concatenate([rng.choice(m, d, replace=False) for d in deg])
    perm = rng.permutation(n)                                           # ranks are not the row numbers
    key = np.unique(perm[r] * m + c)
    row, col = torch.from_numpy(key // m), torch.from_numpy(key % m)
    val = torch.from_numpy(rng.standard_normal(key.size).astype(np.float32))
    tune("spmm_panel", 1)
    tune("spmm_panel_unit", 8192)                                       # the heavy panel is cut into several units
    tune("spmm_panel_dmin", -1)                                         # ... of staged tiles
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
    B = torch.randn(m, f, generator=torch.Generator().manual_seed(3)).to(cuda)
    Cbig = torch.full((n, f + 5), float("nan"), device=cuda)
    C = Cbig[:, 3:3 + f]
    A.spmm(B, out=C, beta=0.0)
    info = _panel_info(A)
    assert info["state"] == 1 and info["rest"] == 0 and info["units"] >= 6, info
    assert torch.isnan(Cbig[:, :3]).all() and torch.isnan(Cbig[:, 3 + f:]).all() and not torch.isnan(C).any()
    assert spmm_error(C, row, col, val, n, m, B.cpu()) <= REL_TOL
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(4))
    Cbig.zero_()
    C.copy_(C0)
    A.spmm(B, out=C, beta=-0.5)
    ref = -0.5 * C0.double() + torch.sparse_coo_tensor(torch.stack([row, col]), val.double(), (n, m)) @ B.cpu().double()
    mag = 0.5 * C0.double().abs() + torch.sparse_coo_tensor(torch.stack([row, col]), val.double().abs(), (n, m)) @ B.cpu().double().abs()
    assert ((C.cpu().double() - ref).abs() / mag.clamp_min(1e-30)).max().item() <= REL_TOL
    assert (Cbig[:, :3] == 0).all() and (Cbig[:, 3 + f:] == 0).all()


def test_spmm_panel_plan_rectangular_strided_and_declined(cuda, tune):
    """A non-symmetric rectangular matrix, B and C as column slices of wider matrices, rows without any
    entry; and a matrix without dense tiles, on which the automatic choice declines the plan."""
    from cagnet_amd import ops
    n, m, f = 700, 1500, 302
    rng = np.random.default_rng(5)
    # skewed pattern: popular columns and heavy rows, plus empty rows at the end
    r = (rng.pareto(1.2, 90000) * 20).astype(np.int64) % (n - 50)
    c = (rng.pareto(1.2, 90000) * 30).astype(np.int64) % m
    key = np.unique(r * m + c)
    row, col = torch.from_numpy(key // m), torch.from_numpy(key % m)
    val = torch.from_numpy(rng.standard_normal(key.size).astype(np.float32))
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m, transpose=True)
    tune("spmm_panel", 1)
    tune("spmm_panel_emin", 6)
    tune("spmm_panel_cols", 512)
    big = torch.randn(m, f + 10, generator=torch.Generator().manual_seed(1)).to(cuda)
    B = big[:, 4:4 + f]                                              # ld f + 10, base 16 bytes into a row
    Cbig = torch.zeros(n, f + 6, device=cuda)
    C = Cbig[:, 2:2 + f]
    A.spmm(B, out=C)
    assert _panel_info(A)["state"] == 1
    assert spmm_error(C, row, col, val, n, m, B.cpu()) <= REL_TOL
    assert float(Cbig[:, :2].abs().max()) == 0.0 and float(Cbig[:, 2 + f:].abs().max()) == 0.0
    G = torch.randn(n, f, device=cuda)
    got = A.spmm(G, transpose=True)
    assert _panel_info(A, transpose=True)["state"] == 1
    assert spmm_error(got, col, row, val, m, n, G.cpu()) <= REL_TOL
    # uniform pattern: no tile reaches the threshold
    tune("spmm_panel", 0)
    tune("spmm_panel_emin", 0)
    tune("spmm_panel_cols", 0)
    ur, uc, uv = random_coo(3000, 3000, 60000, 3)
    U = ops.CsrMatrix(_i32(ur, cuda), _i32(uc, cuda), uv.to(cuda), 3000, 3000)
    Bu = torch.randn(3000, 300, device=cuda)
    got = U.spmm(Bu)
    assert _panel_info(U)["state"] in (0, -1)                       # not considered (small product) or declined
    assert spmm_error(got, ur, uc, uv, 3000, 3000, Bu.cpu()) <= REL_TOL
    tune("spmm_panel", 1)
    got = U.spmm(Bu)                                                 # forced: still correct, whatever the coverage
    assert spmm_error(got, ur, uc, uv, 3000, 3000, Bu.cpu()) <= REL_TOL


def _tile_info(A, f, transpose=False):
    """The tile plan (spmm_tile_kernel) a product of width f uses: panels of 256 / 512 / 1024 rows."""
    import ctypes
    from cagnet_amd._lib import check, lib
    which = 1 + (2 if f <= 64 else 1 if f <= 128 else 0)
    buf = (ctypes.c_int64 * 12)()
    check(lib.cg_csr_panel_info(A._handle, int(transpose) | (which << 2), buf), "cg_csr_panel_info")
    return dict(state=buf[0], covered=buf[1], tiles=buf[2], units=buf[3], split=buf[4], rest=buf[5])


@pytest.mark.parametrize("f", [16, 44, 64, 68, 96, 128, 132, 192, 256, 260, 302, 320, 602, 636, 640, 1000])
def test_spmm_tile_plan_matches_oracle(cuda, tune, f):
    """Every width class of the tile kernel with its plan forced on: one register per row and panels of 1024 rows
    (f <= 64), two and 512 (f <= 128), four or five and 256 (wider, in column slices of up to 316: 602 takes two, 1000
    four).  Both accumulate forms, the transpose side, bit-identical repeats; small units so that panels have several
    blocks of partial rows as well as units that write C themselves."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(13, 400000, seed=3 * f + 1)
    g = torch.Generator().manual_seed(f)
    B = torch.randn(n, f, generator=g)
    C0 = torch.randn(n, f, generator=g)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n, transpose=True)
    tune("spmm_tile", 1)
    for unit in (0, 3000):
        tune("spmm_panel_unit", unit)
        got = A.spmm(B.to(cuda))
        info = _tile_info(A, f)
        assert info["state"] == 1 and info["covered"] == row.numel() and info["rest"] == 0 and info["tiles"] > 0
        if unit:
            assert info["split"] > 0
        assert spmm_error(got, row, col, val, n, n, B) <= REL_TOL
        assert torch.equal(got, A.spmm(B.to(cuda)))
        C = C0.to(cuda).clone()
        A.spmm(B.to(cuda), out=C, beta=1.0)
        assert spmm_error(C, row, col, val, n, n, B, C0) <= REL_TOL
    gotT = A.spmm(B.to(cuda), transpose=True)                        # the graph is symmetric: same product
    assert _tile_info(A, f, transpose=True)["state"] == 1
    assert spmm_error(gotT, row, col, val, n, n, B) <= REL_TOL


def test_spmm_tile_plan_rectangular_strided_and_refused_operands(cuda, tune):
    """A rectangular, non-symmetric matrix with empty rows; B and C as column slices of wider buffers.  Operands the
    tile kernel cannot copy from (rows an odd number of floats apart; a narrow width that is not a multiple of 4)
    go to the other kernels and give the same product."""
    from cagnet_amd import ops
    from tests.util import random_coo
    n, m = 3000, 5000
    row, col, val = random_coo(n, m, 150000, seed=21)
    keep = row % 7 != 3                                              # rows without entries
    row, col, val = row[keep], col[keep], val[keep]
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m, transpose=True)
    tune("spmm_tile", 1)
    for f, ld in ((300, 308), (602, 610), (128, 136), (64, 72), (48, 64)):
        Bw = torch.randn(m, ld, generator=torch.Generator().manual_seed(f))
        B = Bw[:, 4:4 + f]                                           # rows ld floats apart, 16 bytes into the buffer
        Cd = torch.full((n, f + 5), 3.0, device=cuda)
        A.spmm(Bw.to(cuda)[:, 4:4 + f], out=Cd[:, 2:2 + f])
        assert _tile_info(A, f)["state"] == 1
        assert spmm_error(Cd[:, 2:2 + f], row, col, val, n, m, B) <= REL_TOL
        assert bool((Cd[:, :2] == 3.0).all()) and bool((Cd[:, 2 + f:] == 3.0).all())
        Bt = torch.randn(n, f, generator=torch.Generator().manual_seed(f + 1))
        assert spmm_error(A.spmm(Bt.to(cuda), transpose=True), col, row, val, m, n, Bt) <= REL_TOL
    for f in (301, 63, 46):                                          # odd leading dimension / narrow and not a multiple of 4
        B = torch.randn(m, f, generator=torch.Generator().manual_seed(f))
        assert spmm_error(A.spmm(B.to(cuda)), row, col, val, n, m, B) <= REL_TOL


@pytest.mark.parametrize("f", [602, 64])
def test_non_finite_rows_of_B(cuda, tune, f):
    """One row of B holds +inf, another NaN.  cusparseSpMM (sparse-extension/sparse_coo_tensor.cu:215-226) and
    torch.sparse.mm touch only the rows of C that reference them: that is what the row-wise kernels, the tile plans
    and `spmm_strict_nonfinite` give, exactly.  The panel plan with tiles on the matrix cores is documented to differ:
    a dense tile multiplies its zeros, so a non-finite row of B reaches every row of the tile (rows that reference
    neither column come out either untouched or non-finite, never as another finite number), and the zero records
    that pad odd runs can turn an infinity into a NaN in a row that references it; without dense tiles
    (`spmm_panel_dmin = -1`) the rows that reference neither column are untouched."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(11, 260000, seed=5)               # 127 entries per row: dense and staged tiles
    deg = torch.bincount(col, minlength=n)
    order = torch.argsort(deg, descending=True)
    j_inf, j_nan = int(order[3]), int(order[40])                     # two popular columns
    refs_inf = torch.zeros(n, dtype=torch.bool)
    refs_nan = torch.zeros(n, dtype=torch.bool)
    refs_inf[row[col == j_inf]] = True
    refs_nan[row[col == j_nan]] = True
    assert 0 < int(refs_inf.sum()) < n and 0 < int(refs_nan.sum()) < n and int((~refs_inf & ~refs_nan).sum()) > 0
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(2))
    Bbad = B.clone()
    Bbad[j_inf] = float("inf")
    Bbad[j_nan] = float("nan")
    ref = torch.sparse.mm(orc.coo_tensor(row, col, val, n, n, torch.float32), Bbad)   # the reference's CPU twin
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
    clean_rows = ~refs_inf & ~refs_nan

    def check_reference_semantics(what):
        clean = A.spmm(B.to(cuda)).cpu()
        got = A.spmm(Bbad.to(cuda)).cpu()
        assert torch.equal(torch.isnan(got), torch.isnan(ref)), what
        assert torch.equal(torch.isinf(got) & (got > 0), torch.isinf(ref) & (ref > 0)), what
        assert torch.equal(torch.isinf(got) & (got < 0), torch.isinf(ref) & (ref < 0)), what
        assert torch.equal(got[clean_rows], clean[clean_rows]), what

    tune("spmm_panel", -1)
    tune("spmm_panel_narrow", -1)
    check_reference_semantics("row-wise kernels")
    tune("spmm_panel", 0)
    tune("spmm_panel_narrow", 0)
    tune("spmm_tile", 1)
    check_reference_semantics("tile plan")
    assert _tile_info(A, f)["state"] == 1
    tune("spmm_tile", -1)
    tune("spmm_panel", 1)
    tune("spmm_panel_narrow", 1)
    tune("spmm_strict_nonfinite", 1)                                 # the plans that deviate stand back
    check_reference_semantics("strict")
    tune("spmm_strict_nonfinite", 0)
    clean = A.spmm(B.to(cuda)).cpu()
    got = A.spmm(Bbad.to(cuda)).cpu()
    info = _panel_info(A, narrow=(f <= 64)) if f <= 64 else _panel_info(A)
    assert info["state"] == 1 and info["dense_tiles"] > 0
    assert not bool(torch.isfinite(got[refs_inf | refs_nan]).all(dim=1).any())       # every referencing row is non-finite
    untouched = (got[clean_rows] == clean[clean_rows]).all(dim=1)
    tainted = ~torch.isfinite(got[clean_rows]).all(dim=1)
    assert bool((untouched | tainted).all())
    assert bool(tainted.any())                                       # the documented deviation is real on this matrix
    if f > 64:
        tune("spmm_panel_dmin", -1)
        A2 = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
        clean2 = A2.spmm(B.to(cuda)).cpu()
        got2 = A2.spmm(Bbad.to(cuda)).cpu()
        assert _panel_info(A2)["state"] == 1 and _panel_info(A2)["dense_tiles"] == 0
        assert torch.equal(got2[clean_rows], clean2[clean_rows])
        assert not bool(torch.isfinite(got2[refs_inf | refs_nan]).all(dim=1).any())


def test_captured_graph_outlives_plan_eviction_and_scratch_growth(cuda, tune):
    """A HIP graph captured over a product keeps the addresses of the handle's tables and of the
    stream's scratch.  Later eager products at other widths evict hub plans (two are kept per side),
    recycle schedules and grow the scratch; the tables and buffers the graph names must be parked, not
    freed: the replay stays bit-identical, unpin() and scratch_release() report what was kept."""
    from cagnet_amd import ops
    from cagnet_amd._lib import CagnetError
    row, col, val, n = small_graph(11, 60000, seed=77)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
    tune("spmm_hub", 1)
    tune("spmm_hub_kb", 64)
    f = 256
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(1)).to(cuda)
    C = torch.empty(n, f, device=cuda)
    s = torch.cuda.Stream(device=cuda)
    s.wait_stream(torch.cuda.current_stream(cuda))
    with torch.cuda.stream(s):
        A.spmm(B, out=C)                      # builds the plan and grows the scratch: not possible under capture
    s.synchronize()
    expect = C.clone()
    assert spmm_error(expect, row, col, val, n, n, B.cpu()) <= REL_TOL
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        A.spmm(B, out=C)
        # a width that has never run would have to build tables: refused, with nothing enqueued
        with pytest.raises(CagnetError, match="CG_ERR_CAPTURE"):
            A.spmm(torch.empty(n, 272, device=cuda), out=torch.empty(n, 272, device=cuda))
    C.zero_()
    g.replay()
    s.synchronize()
    assert torch.equal(C, expect)
    with torch.cuda.stream(s):
        for f2 in (288, 320, 384, 636):       # other plans, other schedules, more scratch, on the graph's stream
            B2 = torch.randn(n, f2, generator=torch.Generator().manual_seed(f2)).to(cuda)
            assert spmm_error(A.spmm(B2), row, col, val, n, n, B2.cpu()) <= REL_TOL
        tune("spmm_win", 128)                 # other window tables for the schedule the graph uses
        assert torch.equal(A.spmm(B), expect) or spmm_error(A.spmm(B), row, col, val, n, n, B.cpu()) <= REL_TOL
    s.synchronize()
    for _ in range(2):
        C.zero_()
        g.replay()
        s.synchronize()
        assert torch.equal(C, expect)
    del g
    assert A.unpin() > 0                      # tables were parked for the graph
    assert ops.scratch_release(s) > 0
    with torch.cuda.stream(s):
        assert spmm_error(A.spmm(B), row, col, val, n, n, B.cpu()) <= REL_TOL   # and everything still works
    s.synchronize()


def test_captured_panel_product_replays(cuda, tune):
    """A product with the panel plan, captured into a HIP graph: the staged-tile kernel takes its units from queues
    whose counters a small kernel of the same capture zeroes, so every replay — with eager products of the same
    handle on the same stream in between — gives the eager result bit for bit, also with beta != 0."""
    from cagnet_amd import ops
    row, col, val, n = small_graph(12, 120000, seed=41)
    A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
    tune("spmm_panel", 1)
    tune("spmm_panel_unit", 4096)             # many units per queue
    f = 300
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(1)).to(cuda)
    C0 = torch.randn(n, f, generator=torch.Generator().manual_seed(2)).to(cuda)
    C = C0.clone()
    s = torch.cuda.Stream(device=cuda)
    s.wait_stream(torch.cuda.current_stream(cuda))
    with torch.cuda.stream(s):
        A.spmm(B, out=C, beta=0.5)            # builds the plan: not possible under capture
    s.synchronize()
    assert _panel_info(A)["state"] == 1 and _panel_info(A)["units"] > 16
    expect = C.clone()
    g = torch.cuda.CUDAGraph()
    C.copy_(C0)
    with torch.cuda.graph(g, stream=s):
        A.spmm(B, out=C, beta=0.5)
    for k in range(3):
        C.copy_(C0)
        g.replay()
        s.synchronize()
        assert torch.equal(C, expect), k
        with torch.cuda.stream(s):
            assert spmm_error(A.spmm(B), row, col, val, n, n, B.cpu()) <= REL_TOL
        s.synchronize()


def test_plan_build_that_runs_out_of_memory_falls_back_for_good(cuda, tune):
    """An allocation failure while a hub or panel plan is built must not fail the product: it runs on the
    plain schedule, and the plan is not tried again on later calls."""
    from cagnet_amd import ops
    from cagnet_amd._lib import CagnetError
    row, col, val, n = small_graph(11, 60000, seed=78)
    f = 300
    B = torch.randn(n, f, generator=torch.Generator().manual_seed(2)).to(cuda)
    for knob in ("spmm_hub", "spmm_panel"):
        A = ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
        tune("spmm_hub", -1)
        tune("spmm_panel", -1)
        plain = A.spmm(B)
        tune(knob, 1)
        tune("test_alloc_fail", 2)            # the second table allocation of the build fails
        got = A.spmm(B)
        assert torch.equal(got, plain)
        if knob == "spmm_hub":
            assert A.info()["plan_tiers"] == -1
        else:
            assert _panel_info(A)["state"] == -1
        tune("test_alloc_fail", 1)            # would hit the first allocation of a second attempt
        assert torch.equal(A.spmm(B), plain)
        with pytest.raises(CagnetError, match="CG_ERR_ALLOC"):   # still armed: the product allocated nothing
            ops.CsrMatrix(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, n)
        tune("test_alloc_fail", 0)
        tune(knob, 0)


def test_dropin_coo2csr_with_transpose_outputs_and_validate_flag(cuda):
    """The drop-in module's coo2csr: three arrays by default, seven with transpose=True (the CSR of A^T
    and the permutation that links the two value arrays), bit-exact against the oracle.  validate_inputs
    makes spmm_gpu report unsorted rows on the path that otherwise checks nothing."""
    import cagnet_amd.sparse_coo_tensor_cpp as mod
    n, m = 300, 700
    row, col, val = random_coo(n, m, 5000, seed=5, sort=False)
    out = mod.coo2csr(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m)
    assert len(out) == 3
    rp, ci, vv, cp, ri, vt, perm = mod.coo2csr(_i32(row, cuda), _i32(col, cuda), val.to(cuda), n, m, transpose=True)
    erp, eci, evv, _ = orc.coo2csr(row.numpy(), col.numpy(), val.numpy(), n, m)
    ecp, eri, evt, eperm = orc.csr_transpose(erp, eci, evv, n, m)
    for got, want in ((rp, erp), (ci, eci), (vv, evv), (cp, ecp), (ri, eri), (vt, evt), (perm, eperm)):
        assert np.array_equal(got.cpu().numpy(), want)
    assert torch.equal(vt, vv[perm.long()])
    assert all(torch.equal(a, b) for a, b in zip(out, (rp, ci, vv)))

    bad_r = torch.tensor([5, 3, 7], dtype=torch.int32, device=cuda)   # rows descend
    cols = torch.tensor([1, 2, 3], dtype=torch.int32, device=cuda)
    B, C = torch.ones(10, 4, device=cuda), torch.zeros(10, 4, device=cuda)
    mod.spmm_gpu(bad_r, cols, torch.ones(3, device=cuda), 10, 10, B, C)   # unchecked on the narrow path, like the reference
    mod.validate_inputs = True
    try:
        with pytest.raises(ops_error()):
            mod.spmm_gpu(bad_r, cols, torch.ones(3, device=cuda), 10, 10, B, C)
        good_r = torch.tensor([3, 5, 7], dtype=torch.int32, device=cuda)
        C.zero_()
        mod.spmm_gpu(good_r, cols, torch.ones(3, device=cuda), 10, 10, B, C)
        assert float(C.sum()) == 12.0
    finally:
        mod.validate_inputs = False


def ops_error():
    from cagnet_amd._lib import CagnetError
    return CagnetError


def test_host_code_under_sanitizers_with_real_products(cuda):
    """The same sanitized build doing real work on the GPU: handle creation, hub and panel plans at seven
    widths (plan eviction, schedule recycling), a plan build that runs out of memory, the block cache with
    evictions, unpin and scratch release; the driver checks every product against a host loop."""
    from tests.test_abi import run_host_driver
    run_host_driver("gpu")
