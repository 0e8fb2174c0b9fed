"""Host-side logic that needs no GPU: the synthetic generator, the benchmark's accounting and
its command line."""
import hashlib
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from cagnet_amd import synth

ROOT = Path(__file__).resolve().parents[1]


def _digest(*tensors):
    h = hashlib.sha256()
    for t in tensors:
        h.update(np.ascontiguousarray(t.numpy()).tobytes())
    return h.hexdigest()[:16]


def test_rmat_graph_is_seeded_symmetric_and_self_looped():
    row, col, n = synth.rmat_graph(10, 8192, 1)
    row2, col2, _ = synth.rmat_graph(10, 8192, 1)
    assert _digest(row, col) == _digest(row2, col2)
    assert _digest(row, col) != _digest(*synth.rmat_graph(10, 8192, 2)[:2])
    key = row * n + col
    assert torch.all(key[1:] > key[:-1])                      # sorted by (row, col), duplicate free
    assert torch.equal(torch.sort(col * n + row).values, key)  # symmetric pattern
    assert int((row == col).sum()) == n                        # every self-loop present
    deg = torch.bincount(row, minlength=n)
    assert int(deg.max()) > 20 * int(deg.median())             # power-law: hubs far above the median


def test_rmat_quadrant_probabilities():
    src, dst = synth.rmat_edges(1, 400000, 3)
    frac = [float(((src == s) & (dst == d)).float().mean()) for s, d in ((0, 0), (0, 1), (1, 0), (1, 1))]
    assert all(abs(a - b) < 0.005 for a, b in zip(frac, synth.RMAT_ABCD))


def test_target_nnz_is_met_exactly():
    row, col = synth.rmat_graph_target_nnz(1000, 30001, 5)
    assert row.numel() == 2 * ((30001 - 1000) // 2) + 1000 == 30000   # nnz = 2 * pairs + n: within one of the target
    assert int(row.max()) < 1000 and int((row == col).sum()) == 1000


def test_make_problem_shapes_and_seeds():
    p = synth.make_problem(scale=8, n_edges=1024, features=12, hidden=16, classes=5, mask_fraction=0.66, seed=9)
    assert p.x.shape == (256, 12) and p.w1.shape == (12, 16) and p.w2.shape == (16, 5)
    assert p.y.min() >= 0 and p.y.max() < 5 and p.y.dtype == torch.int64
    assert 0.5 < float(p.train_mask.float().mean()) < 0.8
    bound = (6.0 / (12 + 16)) ** 0.5
    assert float(p.w1.abs().max()) <= bound and float(p.w1.abs().max()) > 0.8 * bound
    assert p.seeds == {"graph": 91, "x": 92, "y": 93, "mask": 94, "w1": 95, "w2": 96}


def test_bench_accounting_and_gpu_count_guard():
    sys.path.insert(0, str(ROOT))
    import bench
    # B_alg = 8 nnz + 4 (n+1) + 4 m f + 4 n f (1 + r)
    assert bench.spmm_alg_bytes(10, 4, 5, 3, False) == 80 + 20 + 60 + 48
    assert bench.spmm_alg_bytes(10, 4, 5, 3, True) == 80 + 20 + 60 + 96
    reddit = bench.spmm_alg_bytes(114_615_891, 232_965, 232_965, 602, False)
    assert abs(reddit - 2.04e9) < 0.01e9
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode != 0 and "ONE GPU" in proc.stderr


@pytest.mark.parametrize("size,c", [(16, 2), (8, 2), (4, 1), (9, 3), (12, 2), (20, 2)])
def test_stage_schedule_15d_covers_every_block_once(size, c):
    """Over the c replicas of a block row the stages cover the P/c block columns exactly once, the
    source of a stage sits in the stage's block row and the rank's replica column, and the host
    schedule equals the oracle's restatement (gcn_distr_15d.py:194-208)."""
    from cagnet_amd import gcn
    from oracle import gcn_oracle as orc
    for row in range(size // c):
        seen = []
        for col in range(c):
            rank = row * c + col
            sched = gcn.stage_schedule_15d(rank, size, c)
            assert sched == orc.stage_schedule_15d(rank, size, c)
            for q, block in sched:
                assert q // c == block and q % c == col
            seen += [b for _, b in sched]
        assert sorted(seen) == list(range(size // c))
    with pytest.raises(ValueError):
        gcn.stage_schedule_15d(0, 6, 4)


def test_tile_kernels_keep_their_accumulators_in_registers():
    """spmm_tile_kernel holds 80 accumulators in the physical registers v48..v127 and names them as tied operands of
    its inline-asm statements; the scheme stands only while the register allocator neither spills nor needs scratch
    in any instantiation (a spill around the asm statements would move the accumulators through memory)."""
    from cagnet_amd import build
    res = build.kernel_resources("spmm.hip", "spmm_tile_kernel")
    assert len(res) >= 6, sorted(res)
    for name, r in res.items():
        assert r["vgpr_count"] == 128, (name, r)
        assert r["vgpr_spill_count"] == 0 and r["private_segment_fixed_size"] == 0, (name, r)


def test_recorded_traffic_is_reported_only_for_the_same_kernels_on_the_same_plan():
    """profiles/spmm_traffic.txt: every record names its kernels, its plan signature and the commit it was measured
    at; bench.py hands a record out only to a run that launched those kernels on a plan of that signature."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_for_test", ROOT / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    table = bench.load_traffic()
    lines = [l for l in (ROOT / "profiles" / "spmm_traffic.txt").read_text().splitlines() if l and not l.startswith("#")]
    assert len(table) == len(lines) >= 5
    for (workload, f), rec in table.items():
        assert rec["read"] > 0 and rec["write"] > 0 and len(rec["commit"]) >= 7
        assert rec["plan"] == "rowwise" or rec["plan"].split(":")[0] in ("panel", "tile", "narrow", "hub")
        assert bench.traffic_of(table, workload, f, set(rec["kernels"]), rec["plan"]) == rec["read"] + rec["write"]
        assert bench.traffic_of(table, workload, f, set(rec["kernels"]), rec["plan"] + "x") is None
        assert bench.traffic_of(table, workload, f, set(rec["kernels"]) | {"spmm_hub_hot"}, rec["plan"]) is None
    assert bench.traffic_of(table, "reddit", 600, {"spmm_panel"}, "rowwise") is None
