"""Writes the committed golden vectors (tests/golden/*.npz) from the CPU oracle.

    python tests/golden/make_golden.py

The reference holds no golden vectors, known-answer tests or fixtures for this path, and none of
its files can be imported here, so these vectors come from the oracle after it has been pinned
against scipy / torch / closed forms (tests/test_oracle.py).  They freeze its answers so that a
later change to the oracle or to the generator is noticed, and they give the GPU tests inputs and
expected outputs that do not depend on the generator's code at all.
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from cagnet_amd import synth  # noqa: E402
from oracle import gcn_oracle as orc  # noqa: E402

OUT = Path(__file__).resolve().parent


def graph_case(name: str, scale: int, n_edges: int, f: int, seed: int) -> None:
    row, col, n = synth.rmat_graph(scale, n_edges, seed)
    val = synth.gcn_normalize(row, col, n)
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(row.numel(), generator=g)            # shuffled input for the general path
    rp, ci, vv, p = orc.coo2csr(row[perm].numpy(), col[perm].numpy(), val[perm].numpy(), n, n)
    cp, ri, vt, pt = orc.csr_transpose(rp, ci, vv, n, n)
    B = torch.randn(n, f, generator=g)
    C0 = torch.randn(n, f, generator=g)
    out64 = orc.spmm(row, col, val, n, n, B, C0, torch.float64)
    mag = orc.spmm_abs(row, col, val, n, n, B) + C0.double().abs()
    np.savez_compressed(OUT / f"{name}.npz", n=n, row_shuffled=row[perm].numpy().astype(np.int32),
                        col_shuffled=col[perm].numpy().astype(np.int32), val_shuffled=val[perm].numpy(),
                        rowptr=rp, colind=ci, values=vv, perm=p, colptr=cp, rowind=ri, values_t=vt, perm_t=pt,
                        B=B.numpy(), C0=C0.numpy(), C_out_f64=out64.numpy(), magnitude_f64=mag.numpy())


def training_case(name: str) -> None:
    p = synth.make_problem(scale=7, n_edges=1024, features=24, hidden=16, classes=5, mask_fraction=0.66, seed=21)
    A64 = orc.coo_tensor(p.row, p.col, p.val, p.n, p.n, torch.float64)
    fb = orc.forward_backward(p.x, p.w1, p.w2, [A64], p.y, p.train_mask, dtype=torch.float64)
    losses, w1, w2 = orc.train_epochs(p.x, p.w1, p.w2, [A64], p.y, p.train_mask, epochs=20, lr=0.01,
                                      optimizer="sgd", dtype=torch.float64)
    np.savez_compressed(OUT / f"{name}.npz", n=p.n, row=p.row.numpy().astype(np.int32),
                        col=p.col.numpy().astype(np.int32), val=p.val.numpy(), x=p.x.numpy(), y=p.y.numpy(),
                        mask=p.train_mask.numpy(), w1=p.w1.numpy(), w2=p.w2.numpy(), loss0=float(fb["loss"]),
                        outputs_f64=fb["outputs"].numpy(), dw1_f64=fb["dw1"].numpy(), dw2_f64=fb["dw2"].numpy(),
                        dx_f64=fb["dx"].numpy(), sgd_losses_f64=np.array(losses), w1_after=w1.numpy(),
                        w2_after=w2.numpy())


def harness_case(name: str) -> None:
    """Losses of the single-process harness run `bench.py --workload tiny --optimizer sgd --steps 100
    --warmup 0 --seed 0 --print-losses` (scale 12, 32,768 edges, 128 features, hidden 16, 8 classes,
    SGD 0.01), from the fp64 oracle."""
    p = synth.make_problem(scale=12, n_edges=32768, features=128, hidden=16, classes=8, mask_fraction=1.0, seed=0)
    A64 = orc.coo_tensor(p.row, p.col, p.val, p.n, p.n, torch.float64)
    losses, _, _ = orc.train_epochs(p.x, p.w1, p.w2, [A64], p.y, p.train_mask, epochs=100, lr=0.01,
                                    optimizer="sgd", dtype=torch.float64)
    np.savez_compressed(OUT / f"{name}.npz", n=p.n, nnz=p.row.numel(), sgd_losses_f64=np.array(losses))


def prep_case(name: str) -> None:
    """Raw pattern -> self-loops -> normalised values -> one block of a 3 x 3 partition -> blob."""
    rng = np.random.default_rng(41)
    n = 97
    key = np.sort(rng.choice(n * n, size=700, replace=False))
    row, col = (key // n).astype(np.int32), (key % n).astype(np.int32)      # holds a few of the 97 diagonal entries
    lr, lc = orc.add_self_loops(row, col, n)
    val = orc.gcn_normalize(lr, lc, n)
    b = orc.block_bounds_2d(n, 3)
    br, bc, bv = orc.coo_block(lr, lc, val, b[1], b[2], b[2], b[3])
    rp, ci, vv, _ = orc.coo2csr(lr, lc, val, n, n)
    blob = np.frombuffer(orc.blob_write(rp, ci, vv, n, n, True), dtype=np.uint8)
    np.savez_compressed(OUT / f"{name}.npz", n=n, row=row, col=col, loops_row=lr.astype(np.int32),
                        loops_col=lc.astype(np.int32), values=val, bounds=np.array(b), block_row=br.astype(np.int32),
                        block_col=bc.astype(np.int32), block_val=bv, blob=blob)


if __name__ == "__main__":
    only = set(sys.argv[1:])  # optional: names of the cases to (re)write; default all
    cases = {"graph_s6_f5": lambda: graph_case("graph_s6_f5", 6, 400, 5, 31),
             "graph_s8_f41": lambda: graph_case("graph_s8_f41", 8, 2500, 41, 32),
             "train_s7": lambda: training_case("train_s7"),
             "prep_n97": lambda: prep_case("prep_n97"),
             "harness_tiny_sgd": lambda: harness_case("harness_tiny_sgd")}
    for key, make in cases.items():
        if not only or key in only:
            make()
    for f in sorted(OUT.glob("*.npz")):
        print(f.name, f.stat().st_size, "bytes")
    sys.exit(0)
