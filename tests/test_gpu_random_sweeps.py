"""Seeded random sweeps over shapes, strides and schedule knobs.  torch on the same device is the
independent party: fp64 dense products for the floating-point kernels (bound: REL_TOL of the
magnitude sum), sort / searchsorted / boolean masks for the integer kernels (bit-exact).  Every input is
valid; the sweeps look for shape and knob combinations the hand-written cases do not name."""
import random

import pytest
import torch
import torch.nn.functional as F

from cagnet_amd import synth
from tests.util import REL_TOL

pytestmark = pytest.mark.gpu

SPMM_KNOBS = [b"spmm_seg", b"spmm_win", b"spmm_vec", b"spmm_hub", b"spmm_hub_kb", b"spmm_hub_groups",
              b"spmm_hub_tiers", b"spmm_hub_row"]


@pytest.fixture
def knobs_restored():
    from cagnet_amd._lib import lib
    yield lib
    for key in SPMM_KNOBS + [b"dense_mfma"]:
        lib.cg_tune_set(key, 0)


def _rel(got, ref, mag):
    return float(((got.double() - ref).abs() / mag.clamp_min(1e-30)).max()) if ref.numel() else 0.0


def _strided(rows, cols, extra, gen, dev):
    return torch.randn(rows, cols + extra, device=dev, generator=gen)[:, :cols]


@pytest.mark.parametrize("seed", [11, 12])
def test_spmm_schedules_random(cuda, knobs_restored, seed):
    """Handle, one-shot and digest-cached products over random patterns (empty, sparse, nearly dense,
    with full rows and full columns), widths of every kernel family, both sides, accumulate forms,
    padded leading dimensions and random schedule knobs (segment and window lengths, vector cap,
    hub plans with 1 to 8 tiers over 1 to 8 groups and several row thresholds)."""
    from cagnet_amd import ops
    lib = knobs_restored
    rng = random.Random(seed)
    for case in range(120):
        n = rng.choice([1, 7, 63, 64, 65, 300, 1000, 4097])
        m = rng.choice([1, 5, 64, 129, 1000, 3001])
        dens = rng.choice([0.0, 0.002, 0.02, 0.2, 0.9])
        f = rng.choice([1, 2, 3, 4, 8, 16, 24, 41, 44, 64, 100, 128, 130, 256, 300, 301, 602, 640, 644, 1300, 2562])
        g = torch.Generator().manual_seed(rng.randrange(1 << 30))
        mask = torch.rand(n, m, generator=g) < dens
        if rng.random() < 0.5 and n > 2:
            mask[rng.randrange(n)] = True
            mask[:, rng.randrange(m)] = True
        dense = torch.where(mask, torch.randn(n, m, generator=g), torch.zeros(()))
        idx = mask.nonzero()
        row, col, val = idx[:, 0].int().to(cuda), idx[:, 1].int().to(cuda), dense[mask].to(cuda)
        values = [rng.choice([0, 64, 100, 512, 1024, 4096]), rng.choice([0, 64, 200, 512]), rng.choice([0, 1, 2]),
                  rng.choice([-1, 0, 1, 1, 1]), rng.choice([0, 1, 4, 64]), rng.choice([0, 1, 2, 4, 8]),
                  rng.choice([0, 1, 2, 3, 6, 8]), rng.choice([0, 1, 8, 64, 1000])]
        for key, v in zip(SPMM_KNOBS, values):
            assert lib.cg_tune_set(key, v) == 0
        tr = rng.random() < 0.4
        beta = rng.choice([0.0, 1.0, 1.0, -0.5])
        extra_b, extra_c = rng.choice([0, 0, 1, 4]), rng.choice([0, 0, 2, 4])
        what = f"seed {seed} case {case}: n={n} m={m} nnz={val.numel()} f={f} tr={tr} beta={beta} ld+{extra_b}/{extra_c} knobs={values}"
        gen = torch.Generator(device=cuda).manual_seed(case)
        B = _strided(n if tr else m, f, extra_b, gen, cuda)
        C0 = torch.randn(m if tr else n, f, device=cuda, generator=gen)
        A = ops.CsrMatrix(row, col, val, n, m, is_sorted=True, transpose=tr)
        outs = []
        for _ in range(2):
            C = torch.empty(C0.shape[0], f + extra_c, device=cuda)[:, :f].copy_(C0)
            A.spmm(B, out=C, beta=beta, transpose=tr)
            outs.append(C)
        A64 = dense.double().to(cuda)
        A64 = A64.t() if tr else A64
        ref = beta * C0.double() + A64 @ B.double()
        mag = abs(beta) * C0.double().abs() + A64.abs() @ B.double().abs()
        assert _rel(outs[0], ref, mag) <= REL_TOL, what
        assert torch.equal(outs[0], outs[1]), what
        if not tr and val.numel() > 0:
            ref1 = C0.double() + A64 @ B.double()
            mag1 = C0.double().abs() + A64.abs() @ B.double().abs()
            for cached in (False, True):
                C = C0.clone()
                ops.spmm_coo(row, col, val, n, m, B.contiguous(), C, cached=cached)
                assert _rel(C, ref1, mag1) <= REL_TOL, f"{what} one-shot cached={cached}"
        del A
    ops.coo_cache_clear()


PANEL_KNOBS = [b"spmm_panel", b"spmm_panel_emin", b"spmm_panel_cols", b"spmm_panel_unit", b"spmm_panel_dmin", b"spmm_panel_dwg",
               b"spmm_panel_narrow", b"spmm_panel_narrow_dmin", b"spmm_panel_share"]


@pytest.mark.parametrize("seed", [31, 32])
def test_spmm_panel_plan_random(cuda, knobs_restored, seed):
    """The panel plan forced on over random patterns (skewed and uniform, with full rows and columns, rectangular),
    every even width class it is built for and the narrow widths (dense tiles only), both sides, accumulate forms,
    padded leading dimensions, and random plan knobs: entries a tile needs, ranked columns, unit size, dense-tile
    threshold (off, low, high), the number of workgroups that share the dense tiles and the order of a panel's
    columns (the whole matrix's, or the panel's own).  Every entry is in exactly one of the parts of the plan."""
    import ctypes
    from cagnet_amd import ops
    from cagnet_amd._lib import check
    lib = knobs_restored
    rng = random.Random(seed)
    try:
        for case in range(150):
            n = rng.choice([1, 64, 127, 128, 129, 300, 1000, 2500])
            m = rng.choice([31, 32, 33, 64, 500, 1000, 3001])
            g = torch.Generator().manual_seed(rng.randrange(1 << 30))
            if rng.random() < 0.6:       # skewed: popular columns and heavy rows
                pr = torch.rand(n, 1, generator=g) ** 3
                pc = torch.rand(1, m, generator=g) ** 3
                mask = torch.rand(n, m, generator=g) < (pr * pc * rng.choice([0.5, 2.0, 8.0])).clamp(max=1.0)
            else:
                mask = torch.rand(n, m, generator=g) < rng.choice([0.01, 0.1, 0.6, 1.0])
            if rng.random() < 0.5 and n > 2:
                mask[rng.randrange(n)] = True
                mask[:, rng.randrange(m)] = True
            dense = torch.where(mask, torch.randn(n, m, generator=g), torch.zeros(()))
            idx = mask.nonzero()
            if idx.shape[0] == 0:
                continue
            row, col, val = idx[:, 0].int().to(cuda), idx[:, 1].int().to(cuda), dense[mask].to(cuda)
            f = rng.choice([258, 260, 300, 320, 322, 384, 448, 450, 512, 576, 602, 636, 1, 3, 16, 17, 41, 44, 63, 64])
            narrow = f <= 64
            values = [1, rng.choice([1, 4, 16, 64]), rng.choice([0, 32, 64, 1024]), rng.choice([0, 50, 2000]),
                      rng.choice([-1, 0, 8, 40, 200, 3000]), rng.choice([0, 1, 5, 300]), 1, rng.choice([0, 4, 30, 500]),
                      rng.choice([0, 0, -1])]
            for key, v in zip(PANEL_KNOBS, values):
                assert lib.cg_tune_set(key, v) == 0
            tr = rng.random() < 0.4
            beta = rng.choice([0.0, 1.0, -0.5])
            extra_b, extra_c = rng.choice([0, 0, 2, 6]), rng.choice([0, 0, 2, 4])
            what = f"seed {seed} case {case}: n={n} m={m} nnz={val.numel()} f={f} tr={tr} beta={beta} ld+{extra_b}/{extra_c} knobs={values}"
            gen = torch.Generator(device=cuda).manual_seed(case)
            B = _strided(n if tr else m, f, extra_b, gen, cuda)
            C0 = torch.randn(m if tr else n, f, device=cuda, generator=gen)
            A = ops.CsrMatrix(row, col, val, n, m, is_sorted=True, transpose=tr)
            outs = []
            for _ in range(2):
                C = torch.empty(C0.shape[0], f + extra_c, device=cuda)[:, :f].copy_(C0)
                A.spmm(B, out=C, beta=beta, transpose=tr)
                outs.append(C)
            info = (ctypes.c_int64 * 12)()
            check(lib.cg_csr_panel_info(A._handle, int(tr) | (2 if narrow else 0), info), "cg_csr_panel_info")
            assert info[0] in (1, -1), what                       # in use, or no tile reached the threshold
            if info[0] == 1:
                assert info[1] + info[8] + info[5] == val.numel(), what
                if narrow:
                    assert info[1] == 0 and info[2] == 0, what    # no staged tiles
                elif values[4] < 0:
                    assert info[9] == 0, what
            A64 = dense.double().to(cuda)
            A64 = A64.t() if tr else A64
            ref = beta * C0.double() + A64 @ B.double()
            mag = abs(beta) * C0.double().abs() + A64.abs() @ B.double().abs()
            assert _rel(outs[0], ref, mag) <= REL_TOL, what
            assert torch.equal(outs[0], outs[1]), what
            del A
    finally:
        for key in PANEL_KNOBS:
            lib.cg_tune_set(key, 0)


TILE_KNOBS = [b"spmm_tile", b"spmm_panel", b"spmm_panel_legacy", b"spmm_panel_unit", b"spmm_panel_costcap",
              b"spmm_strict_nonfinite", b"spmm_panel_dmin"]


@pytest.mark.parametrize("seed", [41, 42])
def test_spmm_tile_plans_random(cuda, knobs_restored, seed):
    """The tile plans forced on (every entry through the tile kernel: panels of 256, 512 or 1024 rows by width, column
    slices for wide products) and the panel plan with its staged tiles through either kernel, over random patterns,
    widths of every register layout (1 .. 10 registers per row, one to four slices), both sides, accumulate forms,
    leading dimensions that keep or break the alignment the kernel's copies need (such operands must come out right
    through the other kernels), unit sizes, and a row of B made of infinities."""
    from cagnet_amd import ops
    lib = knobs_restored
    rng = random.Random(seed)
    try:
        for case in range(120):
            n = rng.choice([1, 15, 64, 255, 256, 257, 600, 1100, 2500])
            m = rng.choice([16, 63, 64, 65, 300, 1000, 3001])
            g = torch.Generator().manual_seed(rng.randrange(1 << 30))
            if rng.random() < 0.6:
                pr = torch.rand(n, 1, generator=g) ** 3
                pc = torch.rand(1, m, generator=g) ** 3
                mask = torch.rand(n, m, generator=g) < (pr * pc * rng.choice([0.5, 2.0, 8.0])).clamp(max=1.0)
            else:
                mask = torch.rand(n, m, generator=g) < rng.choice([0.01, 0.1, 0.6, 1.0])
            if rng.random() < 0.5 and n > 2:
                mask[rng.randrange(n)] = True
                mask[:, rng.randrange(m)] = True
            dense = torch.where(mask, torch.randn(n, m, generator=g), torch.zeros(()))
            idx = mask.nonzero()
            if idx.shape[0] == 0:
                continue
            row, col, val = idx[:, 0].int().to(cuda), idx[:, 1].int().to(cuda), dense[mask].to(cuda)
            f = rng.choice([4, 8, 16, 44, 48, 64, 65, 66, 96, 100, 128, 130, 192, 256, 258, 300, 316, 320, 384, 500, 512, 514,
                            602, 636, 640, 700, 950, 1000, 1300])
            mode = rng.choice(["tile", "tile", "panel", "panel_legacy"])
            values = {b"spmm_tile": 1 if mode == "tile" else -1, b"spmm_panel": 1 if mode != "tile" else 0,
                      b"spmm_panel_legacy": 1 if mode == "panel_legacy" else 0,
                      b"spmm_panel_unit": rng.choice([0, 0, 64, 1000, 20000]), b"spmm_panel_costcap": rng.choice([0, 0, 1, 50]),
                      b"spmm_strict_nonfinite": 0, b"spmm_panel_dmin": rng.choice([0, 40, -1])}
            tr = rng.random() < 0.4
            beta = rng.choice([0.0, 1.0, -0.5])
            extra_b, extra_c = rng.choice([0, 0, 2, 4, 1, 3]), rng.choice([0, 0, 2, 4])
            with_inf = rng.random() < 0.15
            if with_inf:
                values[b"spmm_strict_nonfinite"] = 1          # entry-by-entry semantics: the fp64 product is the oracle
            for key, v in values.items():
                assert lib.cg_tune_set(key, v) == 0
            what = (f"seed {seed} case {case}: n={n} m={m} nnz={val.numel()} f={f} mode={mode} tr={tr} beta={beta} "
                    f"ld+{extra_b}/{extra_c} inf={with_inf} knobs={values}")
            gen = torch.Generator(device=cuda).manual_seed(case)
            B = _strided(n if tr else m, f, extra_b, gen, cuda)
            C0 = torch.randn(m if tr else n, f, device=cuda, generator=gen)
            A64 = dense.double().to(cuda)
            A64 = A64.t() if tr else A64
            if with_inf:
                # a row of B that no entry refers to holds infinities: they must reach no row of C
                unused = (A64 != 0).sum(0) == 0
                if bool(unused.any()):
                    B[int(unused.nonzero()[0])] = float("inf")
                else:
                    with_inf = False
            A = ops.CsrMatrix(row, col, val, n, m, is_sorted=True, transpose=tr)
            outs = []
            for _ in range(2):
                C = torch.empty(C0.shape[0], f + extra_c, device=cuda)[:, :f].copy_(C0)
                A.spmm(B, out=C, beta=beta, transpose=tr)
                outs.append(C)
            Bf = torch.where(torch.isfinite(B), B, torch.zeros((), device=cuda)).double()
            ref = beta * C0.double() + A64 @ Bf
            mag = abs(beta) * C0.double().abs() + A64.abs() @ Bf.abs()
            assert torch.isfinite(outs[0]).all(), what
            assert _rel(outs[0], ref, mag) <= REL_TOL, what
            assert torch.equal(outs[0], outs[1]), what
            del A
    finally:
        for key in TILE_KNOBS:
            lib.cg_tune_set(key, 0)


@pytest.mark.parametrize("seed", [21, 22])
def test_dense_and_rowwise_random(cuda, knobs_restored, seed):
    """The three dense products (both kernel families) on strided operands and outputs, and the
    row-wise kernels, over random n, k and output widths from 1 to 100."""
    from cagnet_amd import ops
    lib = knobs_restored
    rng = random.Random(seed)
    for case in range(150):
        n = rng.choice([1, 2, 15, 16, 17, 63, 64, 65, 255, 1000, 4099, 70001])
        k = rng.choice([1, 2, 3, 4, 7, 16, 31, 64, 65, 100, 128, 300, 301, 302, 320, 322, 602, 640, 700, 1026])
        fo = rng.choice([1, 2, 3, 7, 8, 16, 17, 24, 32, 41, 44, 64, 65, 100])
        ex = [rng.choice([0, 0, 1, 2, 4]) for _ in range(6)]
        assert lib.cg_tune_set(b"dense_mfma", rng.choice([0, 0, 0, -1])) == 0
        relu = rng.random() < 0.5
        what = f"seed {seed} case {case}: n={n} k={k} fo={fo} extras={ex} relu={relu}"
        gen = torch.Generator(device=cuda).manual_seed(case)
        X, W, G = _strided(n, k, ex[0], gen, cuda), _strided(k, fo, ex[1], gen, cuda), _strided(n, fo, ex[2], gen, cuda)
        Xd, Wd, Gd = X.double(), W.double(), G.double()
        Z = torch.empty(n, fo + ex[3], device=cuda)[:, :fo]
        ops.dense_xw(X, W, relu=relu, out=Z)
        ref = (Xd @ Wd).clamp_min(0) if relu else Xd @ Wd
        assert _rel(Z, ref, Xd.abs() @ Wd.abs()) <= REL_TOL, what + " xw"
        dX = torch.empty(n, k + ex[4], device=cuda)[:, :k]
        ops.dense_gwt(G, W, out=dX)
        assert _rel(dX, Gd @ Wd.t(), Gd.abs() @ Wd.abs().t()) <= REL_TOL, what + " gwt"
        dW = [torch.empty(k, fo + ex[5], device=cuda)[:, :fo] for _ in range(2)]
        for out in dW:
            ops.dense_xtg(X, G, out=out)
        assert _rel(dW[0], Xd.t() @ Gd, Xd.abs().t() @ Gd.abs()) <= REL_TOL, what + " xtg"
        assert torch.equal(dW[0], dW[1]), what + " xtg repeat"
        Zc = G.contiguous()
        lp = ops.log_softmax_fwd(Zc)
        assert float((lp.double() - F.log_softmax(Zc.double(), dim=1)).abs().max()) <= 2e-6 * max(1.0, float(Zc.abs().max())), what
        go = torch.randn(n, fo, device=cuda, generator=gen)
        gi = ops.log_softmax_bwd(go, lp)
        p = torch.exp(lp.double())
        refg = go.double() - p * go.double().sum(dim=1, keepdim=True)
        magg = go.double().abs() + p * go.double().abs().sum(dim=1, keepdim=True)
        assert _rel(gi, refg, magg) <= REL_TOL, what + " log_softmax_bwd"
        h = ops.relu_fwd(Zc)
        assert torch.equal(h, Zc.clamp_min(0)), what
        assert torch.equal(ops.relu_bwd(go, h), go * (h > 0)), what
        y = torch.randint(0, fo, (n,), device=cuda, generator=gen)
        mask = torch.rand(n, device=cuda, generator=gen) < 0.6
        loss, count = ops.nll_loss_fwd(lp, y, mask)
        cnt = int(mask.sum())
        assert int(count) == cnt, what
        refl = float(-(lp.double()[mask, y[mask]]).sum() / cnt) if cnt else 0.0
        assert abs(float(loss) - refl) <= 1e-5 * max(1.0, abs(refl)), what + " nll"


@pytest.mark.parametrize("seed", [31])
def test_conversions_and_preparation_random(cuda, seed):
    """COO in arbitrary order -> CSR, transposes (with and without the permutation), block extraction,
    self-loops and normalisation, bit for bit against sort / searchsorted / masks."""
    from cagnet_amd import ops
    rng = random.Random(seed)
    for case in range(150):
        n = rng.choice([1, 2, 5, 64, 255, 256, 257, 1000, 65536, 70001, 300000])
        m = rng.choice([1, 3, 64, 255, 256, 257, 4097, 65537, 262145]) if rng.random() < 0.5 else n
        cap = n * m
        nnz = min(cap, rng.choice([0, 1, 5, 1000, 4096, 4097, 100000, 1500000]))
        gen = torch.Generator(device=cuda).manual_seed(case * 7 + 1)
        if cap <= 4_000_000:
            key = torch.randperm(cap, device=cuda, generator=gen)[:nnz]
        else:
            key = torch.unique(torch.randint(0, cap, (nnz,), device=cuda, generator=gen))
            key = key[torch.randperm(key.numel(), device=cuda, generator=gen)]
        nnz = key.numel()
        row, col = (key // m).int(), (key % m).int()
        val = torch.randn(nnz, device=cuda, generator=gen)
        what = f"seed {seed} case {case}: n={n} m={m} nnz={nnz}"
        order = torch.sort(key, stable=True).indices
        srow, scol, sval = row[order], col[order], val[order]
        want_rp = torch.searchsorted(srow.long(), torch.arange(n + 1, device=cuda)).int()
        rp, ci, vv, perm = ops.coo2csr(row, col, val, n, m, return_perm=True)
        assert torch.equal(rp, want_rp) and torch.equal(ci, scol) and torch.equal(vv, sval), what
        assert torch.equal(perm.long(), order), what
        rp, ci, vv = ops.coo2csr(row, col, val, n, m)
        assert torch.equal(rp, want_rp) and torch.equal(ci, scol) and torch.equal(vv, sval), what
        assert torch.equal(ops.coo2csr_rowptr(srow, n), want_rp), what
        torder = torch.sort(scol.long() * n + srow.long(), stable=True).indices
        want_cp = torch.searchsorted(scol[torder].long(), torch.arange(m + 1, device=cuda)).int()
        cp, ri, vt, tperm = ops.csr_transpose(rp, ci, vv, n, m, return_perm=True)
        assert torch.equal(cp, want_cp) and torch.equal(ri, srow[torder]) and torch.equal(vt, sval[torder]), what
        assert torch.equal(tperm.long(), torder), what
        cp, ri, vt = ops.csr_transpose(rp, ci, vv, n, m)
        assert torch.equal(cp, want_cp) and torch.equal(ri, srow[torder]) and torch.equal(vt, sval[torder]), what
        r0, r1 = sorted((rng.randrange(n + 1), rng.randrange(n + 1)))
        c0, c1 = sorted((rng.randrange(m + 1), rng.randrange(m + 1)))
        br, bc, bv = ops.coo_block(srow, scol, sval, r0, r1, c0, c1)
        inside = (srow >= r0) & (srow < r1) & (scol >= c0) & (scol < c1)
        assert torch.equal(br, srow[inside] - r0) and torch.equal(bc, scol[inside] - c0), what
        assert torch.equal(bv, sval[inside]), what
        if n == m:
            lr, lc = ops.add_self_loops(srow, scol, n)
            diag = torch.arange(n, device=cuda)
            allk = torch.unique(torch.cat([srow.long() * n + scol.long(), diag * n + diag]))
            assert torch.equal(lr.long(), allk // n) and torch.equal(lc.long(), allk % n), what
            assert torch.equal(ops.gcn_normalize(lr, lc, n), synth.gcn_normalize(lr.long(), lc.long(), n)), what


@pytest.mark.parametrize("seed", [41])
def test_fused_layer_product_random(cuda, knobs_restored, seed):
    """Z = act((acc + op(A) B) W) in one pass, over random patterns, widths with and without a fused
    form (those must answer None, not compute), sides, accumulators and schedule knobs."""
    from cagnet_amd import ops
    lib = knobs_restored
    rng = random.Random(seed)
    fused = 0
    for case in range(200):
        n = rng.choice([1, 7, 64, 65, 300, 1000, 4097])
        m = rng.choice([1, 5, 64, 129, 1000, 3001])
        dens = rng.choice([0.0, 0.002, 0.02, 0.2, 0.9])
        f = rng.choice([16, 64, 100, 128, 130, 256, 257, 300, 301, 512, 602, 640, 644, 1000, 1300])
        fo = rng.choice([1, 2, 7, 8, 16, 17, 24, 32, 41, 64, 65])
        g = torch.Generator().manual_seed(rng.randrange(1 << 30))
        mask = torch.rand(n, m, generator=g) < dens
        if rng.random() < 0.5 and n > 2:
            mask[rng.randrange(n)] = True
            mask[:, rng.randrange(m)] = True
        dense = torch.where(mask, torch.randn(n, m, generator=g), torch.zeros(()))
        idx = mask.nonzero()
        row, col, val = idx[:, 0].int().to(cuda), idx[:, 1].int().to(cuda), dense[mask].to(cuda)
        values = [rng.choice([0, 64, 100, 512, 1024]), rng.choice([0, 64, 200, 512]), rng.choice([0, 1, 2]),
                  rng.choice([-1, 0, 1, 1]), rng.choice([0, 1, 4, 64]), rng.choice([0, 1, 2, 4, 8]),
                  rng.choice([0, 1, 2, 3, 6]), rng.choice([0, 1, 8, 64])]
        for key, v in zip(SPMM_KNOBS, values):
            assert lib.cg_tune_set(key, v) == 0
        tr, relu, use_acc = rng.random() < 0.3, rng.random() < 0.5, rng.random() < 0.4
        what = f"seed {seed} case {case}: n={n} m={m} nnz={val.numel()} f={f} fo={fo} tr={tr} relu={relu} acc={use_acc} knobs={values}"
        gen = torch.Generator(device=cuda).manual_seed(case)
        rows_b, rows_c = (n, m) if tr else (m, n)
        B = _strided(rows_b, f, rng.choice([0, 0, 4]), gen, cuda)
        W = _strided(f, fo, rng.choice([0, 0, 3]), gen, cuda)
        acc = torch.randn(rows_c, f, device=cuda, generator=gen) if use_acc else None
        A = ops.CsrMatrix(row, col, val, n, m, is_sorted=True, transpose=tr)
        Z = A.spmm_xw(B, W, relu=relu, acc=acc, transpose=tr)
        if Z is None:
            continue
        fused += 1
        assert torch.equal(Z, A.spmm_xw(B, W, relu=relu, acc=acc, transpose=tr)), what
        A64 = dense.double().to(cuda)
        A64 = A64.t() if tr else A64
        inner = A64 @ B.double() + (acc.double() if use_acc else 0)
        inner_mag = A64.abs() @ B.double().abs() + (acc.double().abs() if use_acc else 0)
        ref = inner @ W.double()
        ref = ref.clamp_min(0) if relu else ref
        # two roundings in a row (the row of A B, then its product with W): twice the bound of one
        assert _rel(Z, ref, inner_mag @ W.double().abs()) <= 2 * REL_TOL, what
    assert fused >= 60


@pytest.mark.parametrize("seed", [51])
def test_two_layer_forward_backward_random(cuda, monkeypatch, seed):
    """GCNFunc twice + masked NLL + backward over random graph sizes and densities, feature, hidden and
    class widths, mask fractions (including an empty mask), product orders, fusion and with or without a
    stored transpose, against the fp64 CPU oracle of the same pass."""
    from cagnet_amd import gcn, ops
    from oracle import gcn_oracle as orc
    from tests.util import LOSS_TOL
    rng = random.Random(seed)

    def rel(got, ref64):
        return float((got.detach().cpu().double() - ref64).abs().max()) / max(float(ref64.abs().max()), 1e-30)

    for case in range(40):
        n = rng.choice([33, 100, 257, 1000, 3000])
        nnz = max(n, min(n * n // 2, rng.choice([n, 4 * n, 20 * n, 100 * n])))
        f = rng.choice([1, 3, 16, 64, 100, 128, 300, 301, 602])
        hidden = rng.choice([1, 4, 16, 17, 32, 64])
        classes = rng.choice([2, 7, 8, 24, 41, 64])
        frac = rng.choice([0.0, 0.3, 0.66, 1.0])
        fused, first, tr = rng.random() < 0.5, rng.random() < 0.7, rng.random() < 0.5
        monkeypatch.setattr(gcn, "fused_forward", fused)
        monkeypatch.setattr(gcn, "spmm_first", first)
        what = f"seed {seed} case {case}: n={n} nnz~{nnz} f={f} hidden={hidden} classes={classes} mask={frac} fused={fused} spmm_first={first} transpose={tr}"
        p = synth.make_problem(n=n, target_nnz=nnz, features=f, hidden=hidden, classes=classes, mask_fraction=frac, seed=case)
        A = orc.coo_tensor(p.row, p.col, p.val, p.n, p.n, torch.float64)
        ref = orc.forward_backward(p.x, p.w1, p.w2, [A], p.y, p.train_mask, dtype=torch.float64)
        blk = ops.CsrMatrix(p.row.int().to(cuda), p.col.int().to(cuda), p.val.to(cuda), p.n, p.n, transpose=tr)
        x, w1, w2 = (t.to(cuda).requires_grad_(True) for t in (p.x, p.w1, p.w2))
        h = gcn.GCNFunc.apply(x, w1, p.n, [blk], 0, 1, None, F.relu)
        out = gcn.GCNFunc.apply(h, w2, p.n, [blk], 0, 1, None, F.log_softmax)
        loss = gcn.masked_nll_loss(out, p.y.to(cuda), p.train_mask.to(cuda))
        loss.backward()
        assert abs(float(loss.detach()) - float(ref["loss"])) <= LOSS_TOL, what
        for name, got, want in (("hidden", h, ref["hidden"]), ("outputs", out, ref["outputs"]), ("dw1", w1.grad, ref["dw1"]),
                                ("dw2", w2.grad, ref["dw2"]), ("dx", x.grad, ref["dx"])):
            assert rel(got, want) <= 2e-4, f"{what}: {name}"   # several chained products: relative to the largest entry
