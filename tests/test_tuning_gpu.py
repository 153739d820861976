"""The launch-parameter sweep (bitsknn/tuning.py) on a tiny grid: it runs, keeps the fastest
configuration per problem and writes a file the lookup can read."""
import os

import pytest

pytestmark = pytest.mark.gpu


def test_small_sweep_round_trip(bk, dev, tmp_path):
    from bitsknn import tuning
    rows = list(tuning.sweep(repeats=2, point_count=32 * 1024, query_counts=(64, 256), k_values=(16, 300),
                             block_sizes=(128, 256), batch_sizes=(1, 8)))
    assert len(rows) == 2 * 2 * 2 * 2 * 2          # q x k x algorithm x block x batch
    assert all(r["time"] > 0 for r in rows)
    rows += list(tuning.sweep_partial_bitonic(repeats=1, problem_size=1 << 22, query_counts=(64,),
                                              k_values=(32,), block_sizes=(64, 512)))
    best = tuning.optima(rows)
    assert len(best) == 2 * 2 * 2 + 1
    for r in best:
        same = [x for x in rows if all(x[c] == r[c] for c in ("algorithm", "query_count", "k"))]
        assert r["time"] == min(x["time"] for x in same)
    path = os.path.join(tmp_path, "optima.csv")
    tuning.write_optima(best, path, hostname="testbox")
    block, deg, batch, _, _ = tuning.config_algorithm("bits", 200, 200, hostname="testbox", optima_file=path)
    chosen = [r for r in best if r["algorithm"] == "bits" and r["query_count"] == 256 and r["k"] == 300][0]
    assert (block, deg, batch) == (chosen["block_size"], 1, chosen["items_per_thread"])
    assert tuning.config_algorithm("partial-bitonic-regs", 64, 32, hostname="testbox", optima_file=path)[0] in (64, 512)


def test_bits_sq_and_fused_sweeps(bk, dev, oracle, tmp_path):
    """The row-splitting sweep gives the oracle's result for every number of parts, and its rows
    and the fused-cache rows land in a file the lookup reads (deg and the three item counts)."""
    import numpy as np
    import torch
    from bitsknn import tuning
    m = oracle.uniform_matrix(5, 3, 1 << 15)
    ed, el = oracle.topk(m, 100)
    for deg in (2, 4, 16):
        od, ol = tuning.bits_sq(torch.from_numpy(m).to(dev), 100, deg, 128, 8)
        torch.cuda.synchronize()
        assert np.array_equal(od.cpu().numpy(), ed) and np.array_equal(ol.cpu().numpy(), el), deg
    rows = list(tuning.sweep_bits_sq(repeats=1, point_count=1 << 15, query_counts=(64,), k_values=(16,),
                                     block_sizes=(128,), batch_sizes=(8,), degrees=(2, 8)))
    assert [r["deg"] for r in rows] == [2, 8] and all(r["algorithm"] == "bits-sq" for r in rows)
    rows += list(tuning.sweep_fused(repeats=1, shapes=((256, 1 << 14),), dims=(8,), k_values=(16,)))
    path = os.path.join(tmp_path, "optima.csv")
    tuning.write_optima(tuning.optima(rows), path, hostname="testbox")
    block, deg, batch, _, _ = tuning.config_algorithm("bits-sq", 64, 16, hostname="testbox", optima_file=path)
    assert block == 128 and deg in (2, 8) and batch == 8
    assert tuning.config_algorithm("fused-cache", 256, 16, 8, hostname="testbox", optima_file=path) == (1, 1, 8, 4, 2)
