"""Stand-alone measurements of the sparse kernels on one MI355X.

    python -m cagnet_amd.microbench spmm   [--graph rmat20|reddit|amazon] [--widths 16,64,128,602] [--forward-only]
                                           [--aligned-rows] [--tune KEY=VALUE ...]
    python -m cagnet_amd.microbench grid2d [--grid 4] [--row 1]
    python -m cagnet_amd.microbench prep   [--graph reddit]

`spmm`   builds the CSR (sorted input, unsorted input, transpose) and times A @ H and A^T @ G at
         each width: GFLOP/s = 2 nnz f / t, algorithmic GB/s = (8 nnz + 4 (n+1) + 4 m f + 4 n f) / t.
`grid2d` is one rank's share of the sqrt(P) x sqrt(P) 2D algorithm (gcn_distr_2d.py:333-417) on the
         Reddit-shaped graph: the sparse blocks A(r, 0..q-1) of process row r, each times a resident
         dense block, accumulated over q stages; forward and backward of both layers.
`prep`   times the device-side input preparation on the graph's pattern: self-loop insertion,
         D^-1/2 A D^-1/2 values, and the 16 block extractions of a 4 x 4 partition.
One JSON object per line.  Timing: HIP events on the current stream, median of `--reps`.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import sys
import time

import torch
import torch.nn.functional as F

GRAPHS = {
    "rmat20": dict(scale=20, n_edges=16_777_216),
    "reddit": dict(n=232_965, target_nnz=114_615_892),
    "rmat16": dict(scale=16, n_edges=1_048_576),
    "amazon": dict(n=14_249_639, target_nnz=230_600_000),
}


def _graph(name: str, dev):
    from . import synth

    g = GRAPHS[name]
    if "scale" in g:
        row, col, n = synth.rmat_graph(g["scale"], g["n_edges"], 1, dev)
    else:
        n = g["n"]
        row, col = synth.rmat_graph_target_nnz(n, g["target_nnz"], 1, dev)
    return row, col, synth.gcn_normalize(row, col, n), n


def _time(fn, reps: int) -> float:
    fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    times.sort()
    return times[len(times) // 2]


_SPMM_KERNELS = ("spmm_panel_dense", "spmm_panel", "spmm_panel_add", "spmm_hub_hot", "spmm_rowseg", "spmm_reduce",
                 "spmm_hub_reduce")


def _launched(fn, f: int) -> set:
    """Profiling names of the SpMM kernels one call of fn launches at width f."""
    from ._lib import lib

    torch.cuda.synchronize()
    lib.cg_prof_enable(1)
    fn()
    torch.cuda.synchronize()
    lib.cg_prof_enable(0)
    out = set()
    for k in _SPMM_KERNELS:
        t, c = ctypes.c_double(0.0), ctypes.c_int64(0)
        lib.cg_prof_read(f"{k}/f={f}".encode(), ctypes.byref(t), ctypes.byref(c))
        if c.value:
            out.add(k)
    return out


def run_spmm(args) -> None:
    from . import ops

    dev = torch.device("cuda:0")
    row, col, val, n = _graph(args.graph, dev)
    nnz = int(val.numel())
    r32, c32 = row.int(), col.int()
    torch.cuda.synchronize()

    def build(**kw):
        best, a = float("inf"), None
        for _ in range(3):
            del a
            torch.cuda.synchronize()  # the arguments may still be in the making (permuted copies)
            t0 = time.perf_counter()
            a = ops.CsrMatrix(**kw)
            torch.cuda.synchronize()
            best = min(best, (time.perf_counter() - t0) * 1e3)
        return a, best

    build(row=r32, col=c32, val=val, n=n, m=n)  # first call also grows the scratch buffers
    _, t_sorted = build(row=r32, col=c32, val=val, n=n, m=n)
    A, t_with_t = build(row=r32, col=c32, val=val, n=n, m=n, transpose=True)
    perm = torch.randperm(nnz, device=dev, generator=torch.Generator(device=dev).manual_seed(3))
    _, t_unsorted = build(row=r32[perm], col=c32[perm], val=val[perm], n=n, m=n, is_sorted=False)
    del perm
    print(json.dumps({"what": "csr build", "graph": args.graph, "n": n, "nnz": nnz,
                      "coo2csr_sorted_ms": round(t_sorted, 3), "coo2csr_plus_transpose_ms": round(t_with_t, 3),
                      "coo2csr_unsorted_radix_ms": round(t_unsorted, 3), "max_degree": A.info()["max_row_degree"]}),
          flush=True)
    from ._lib import check, lib
    for item in args.tune:  # tuning keys of cg_tune_set for the products below (measuring runs)
        key, value = item.split("=")
        check(lib.cg_tune_set(key.encode(), int(value)), "cg_tune_set")
    for f in args.widths:
        ld = (f + 31) // 32 * 32 if args.aligned_rows else f  # rows of B a whole number of 128-byte lines apart
        B = torch.randn(n, ld, device=dev)[:, :f]
        C = torch.empty(n, f, device=dev)
        alg = 8 * nnz + 4 * (n + 1) + 4 * n * f + 4 * n * f
        for name, tr in ((("A@H", False),) if args.forward_only else (("A@H", False), ("A^T@G", True))):
            ms = _time(lambda: A.spmm(B, out=C, beta=0.0, transpose=tr), args.reps)
            launched = _launched(lambda: A.spmm(B, out=C, beta=0.0, transpose=tr), f)
            print(json.dumps({"what": "spmm", "graph": args.graph, "product": name, "f": f, "ms": round(ms, 4),
                              "kernels": "+".join(sorted(launched)), "plan": A.plan_signature(f, launched, transpose=tr),
                              "gflops": round(2.0 * nnz * f / ms / 1e6, 1), "algorithmic_gbs": round(alg / ms / 1e6, 1),
                              "pct_of_8TBs": round(alg / ms / 1e6 / 80.0, 2)}), flush=True)
        del B, C


def run_grid2d(args) -> None:
    from . import gcn, ops, synth

    dev = torch.device("cuda:0")
    from ._lib import check, lib
    for item in args.tune:
        key, value = item.split("=")
        check(lib.cg_tune_set(key.encode(), int(value)), "cg_tune_set")
    row, col, val, n = _graph("reddit", dev)
    q, r = args.grid, args.row
    b = synth.block_bounds_2d(n, q)
    rows = b[r + 1] - b[r]
    feats, hidden, classes = 602, 16, 41
    blocks, nnzs = [], []
    for k in range(q):
        rr, cc, vv = synth.coo_block(row, col, val, b[r], b[r + 1], b[k], b[k + 1])
        blocks.append(ops.CsrMatrix(rr.int(), cc.int(), vv, rows, b[k + 1] - b[k]))
        nnzs.append(int(vv.numel()))
    del row, col, val
    gen = torch.Generator(device=dev).manual_seed(11)

    def peers(width):
        return [None if k == r else torch.randn(b[k + 1] - b[k], width, device=dev, generator=gen) for k in range(q)]

    g1 = gcn.ResidentBlocks(peers(feats), peers(hidden))
    g2 = gcn.ResidentBlocks(peers(hidden), peers(classes))
    x = torch.randn(rows, feats, device=dev, generator=gen).requires_grad_(True)
    w1 = synth.glorot_uniform(feats, hidden, 5, dev).requires_grad_(True)
    w2 = synth.glorot_uniform(hidden, classes, 6, dev).requires_grad_(True)
    y = synth.uniform_labels(rows, classes, 3, dev)
    mask = synth.random_mask(rows, 0.66, 4, dev)

    def step():
        h = gcn.GCNFunc.apply(x, w1, rows, blocks, r, q, g1, F.relu)
        out = gcn.GCNFunc.apply(h, w2, rows, blocks, r, q, g2, F.log_softmax)
        loss = gcn.masked_nll_loss(out, y, mask)
        loss.backward()
        x.grad = w1.grad = w2.grad = None

    ms = float("nan") if args.stages_only else _time(step, args.reps)
    # the four accumulate-SpMMs of one stage loop at the input width
    H = [x.detach() if k == r else g1.forward[k] for k in range(q)]
    z = torch.empty(rows, feats, device=dev)

    def stages():
        for k in range(q):
            blocks[k].spmm(H[k], out=z, beta=0.0 if k == 0 else 1.0)

    def fused():  # the library's stage loop: one product of the blocks side by side with the stacked operands
        gcn.broad_func(rows, blocks, x.detach(), r, q, g1.forward, out=z)

    ms_stage = float("nan") if args.stages_only and not args.per_stage else _time(stages, args.reps)
    ms_fused = float("nan") if args.stages_only and args.per_stage else _time(fused, args.reps)
    launched = set() if ms_fused != ms_fused else _launched(fused, feats)
    plan = gcn.stacked_blocks(blocks).plan_signature(feats, launched) if launched else None
    flops = 2.0 * sum(nnzs) * feats
    alg = sum(8 * nz + 4 * (rows + 1) + 4 * (b[k + 1] - b[k]) * feats + 4 * rows * feats * (1 if k == 0 else 2)
              for k, nz in enumerate(nnzs))
    alg_fused = 8 * sum(nnzs) + 4 * (rows + 1) + 4 * n * feats + 4 * rows * feats
    print(json.dumps({"what": "grid2d rank share", "grid": f"{q}x{q}", "process_row": r, "rows": rows, "block_nnz": nnzs,
                      "fwd_bwd_both_layers_ms": None if args.stages_only else round(ms, 3),
                      "stage_loop_f602_ms": round(ms_fused, 3), "stage_loop_f602_one_product_per_stage_ms": round(ms_stage, 3),
                      "stage_loops_run": args.reps + 1, "kernels": "+".join(sorted(launched)), "plan": plan,
                      "stage_loop_gflops": round(flops / ms_fused / 1e6, 1),
                      "stage_loop_algorithmic_gbs": round(alg_fused / ms_fused / 1e6, 1),
                      "one_product_per_stage_algorithmic_gbs": round(alg / ms_stage / 1e6, 1)}), flush=True)


def run_prep(args) -> None:
    from . import ops, synth

    dev = torch.device("cuda:0")
    row, col, _, n = _graph(args.graph, dev)
    r32, c32 = row.int(), col.int()
    nnz = int(r32.numel())
    del row, col

    def wall(fn):
        fn()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(args.reps):
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            best = min(best, (time.perf_counter() - t0) * 1e3)
        return best

    t_loops = wall(lambda: ops.add_self_loops(r32, c32, n))
    t_norm = wall(lambda: ops.gcn_normalize(r32, c32, n))
    val = ops.gcn_normalize(r32, c32, n)
    b = synth.block_bounds_2d(n, 4)

    def blocks():
        for i in range(4):
            for j in range(4):
                ops.coo_block(r32, c32, val, b[i], b[i + 1], b[j], b[j + 1])

    t_blocks = wall(blocks)
    print(json.dumps({"what": "input preparation", "graph": args.graph, "n": n, "nnz": nnz,
                      "add_self_loops_ms": round(t_loops, 3), "gcn_normalize_ms": round(t_norm, 3),
                      "coo_block_4x4_all_16_ms": round(t_blocks, 3)}), flush=True)


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    s = sub.add_parser("spmm")
    s.add_argument("--graph", default="rmat20", choices=sorted(GRAPHS))
    s.add_argument("--widths", default="16,64,128,602", type=lambda t: [int(v) for v in t.split(",")])
    s.add_argument("--reps", type=int, default=5)
    s.add_argument("--forward-only", action="store_true", help="A @ H only")
    s.add_argument("--aligned-rows", action="store_true", help="rows of the dense operand a multiple of 128 bytes apart")
    s.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                   help="a tuning key of cg_tune_set for the products (repeatable), e.g. spmm_panel_qcap=128")
    g = sub.add_parser("grid2d")
    g.add_argument("--grid", type=int, default=4)
    g.add_argument("--row", type=int, default=1)
    g.add_argument("--reps", type=int, default=5)
    g.add_argument("--stages-only", action="store_true",
                   help="run the stage loop only (reps + 1 times): what a counter run of the stage loop profiles")
    g.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                   help="cg_tune_set before the products (repeatable)")
    g.add_argument("--per-stage", action="store_true",
                   help="with --stages-only: the loop as one product per stage instead of the fused one")
    pr = sub.add_parser("prep")
    pr.add_argument("--graph", default="reddit", choices=sorted(GRAPHS))
    pr.add_argument("--reps", type=int, default=3)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        print("microbench: no GPU visible; cagnet_amd has no CPU path", file=sys.stderr)
        return 2
    if args.cmd == "spmm":
        run_spmm(args)
    elif args.cmd == "prep":
        run_prep(args)
    else:
        run_grid2d(args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
