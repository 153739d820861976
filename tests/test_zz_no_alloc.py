"""The fused entry point that allocates nothing (bitsknn_fused_l2_topk_f32_static): its partial
lists live in a static device array inside the library.  Checked against
bitsknn_fused_l2_topk_f32_ws with a caller-allocated workspace, bit for bit, on consecutive calls
that share the array -- the second one smaller, so that it meets the first one's leftovers."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(bk, dev, oracle, seed, n, q, d, k, workspace):
    import torch
    points, queries = oracle.generate(seed, n, q, d)
    pd = torch.from_numpy(np.ascontiguousarray(points.T)).to(dev)
    qd = torch.from_numpy(np.ascontiguousarray(queries.T)).to(dev)
    od, ol = bk.fused_l2_topk(qd, pd, k, workspace=workspace)
    torch.cuda.synchronize()
    return od.cpu().numpy(), ol.cpu().numpy()


def test_static_scratch_matches_the_workspace_entry_point(bk, dev, oracle):
    import torch
    limit = bk.fused_static_scratch_bytes()
    assert limit == 32 << 20
    # (points, queries, dim, k): the first call cuts the points into many ranges, the second is a
    # smaller problem with fewer and shorter partial lists, the third needs no ranges at all
    cases = [(200000, 700, 16, 32), (50000, 130, 8, 16), (3000, 40, 8, 4)]
    for seed, (n, q, d, k) in enumerate(cases):
        need = bk.fused_workspace_bytes(q, n, k)
        assert need <= limit
        want_d, want_l = _run(bk, dev, oracle, 50 + seed, n, q, d, k, "auto")
        before = torch.cuda.memory_allocated(dev)
        got_d, got_l = _run(bk, dev, oracle, 50 + seed, n, q, d, k, "static")
        assert torch.cuda.memory_allocated(dev) == before
        assert np.array_equal(got_d, want_d) and np.array_equal(got_l, want_l), (n, q, d, k)
    sizes = [bk.fused_workspace_bytes(q, n, k) for n, q, d, k in cases]
    assert sizes[0] > sizes[1] > sizes[2] == 0
    # against the oracle as well (the first case again, after the smaller ones used the array)
    n, q, d, k = cases[0]
    got_d, got_l = _run(bk, dev, oracle, 50, n, q, d, k, "static")
    points, queries = oracle.generate(50, n, q, d)
    exp_d, exp_l = oracle.topk(oracle.dist(queries, points, "partial"), k)
    recall = np.mean([len(set(a) & set(b)) / k for a, b in zip(got_l, exp_l)])
    assert recall >= 0.999
    scale = np.abs(exp_d[:, k - 1]) + (queries.astype(np.float64) ** 2).sum(1)
    assert np.max(np.abs(got_d[:, k - 1] - exp_d[:, k - 1]) / scale) <= 1e-5


def test_static_scratch_call_replayed_from_a_graph(bk, dev, oracle):
    """The call is meant for code under HIP graph capture: after one eager call on the device (which
    looks up the array's address and sets the kernels' LDS sizes), the same call is captured into a
    graph and replayed several times with eager work and synchronisations in between; every replay
    must give the workspace entry point's result bit for bit.  An allocation inside the library
    (hipMalloc is not allowed while a stream is being captured) would fail the capture."""
    import torch
    n, q, d, k = 120000, 500, 16, 32
    assert 0 < bk.fused_workspace_bytes(q, n, k) <= bk.fused_static_scratch_bytes()
    points, queries = oracle.generate(77, n, q, d)
    pd = torch.from_numpy(np.ascontiguousarray(points.T)).to(dev)
    qd = torch.from_numpy(np.ascontiguousarray(queries.T)).to(dev)
    want_d, want_l = bk.fused_l2_topk(qd, pd, k, workspace="auto")
    torch.cuda.synchronize()
    out_d = torch.empty((q, k), dtype=torch.float32, device=dev)
    out_l = torch.empty((q, k), dtype=torch.int32, device=dev)
    bk.fused_l2_topk(qd, pd, k, workspace="static", out_dist=out_d, out_label=out_l)  # eager warm-up
    torch.cuda.synchronize()
    assert torch.equal(out_d, want_d) and torch.equal(out_l, want_l)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        bk.fused_l2_topk(qd, pd, k, workspace="static", out_dist=out_d, out_label=out_l)
    for replay in range(3):
        out_d.fill_(-1.0)
        out_l.fill_(-1)
        # eager work on the same scratch memory between the replays: a smaller problem
        bk.fused_l2_topk(qd[:, :100].contiguous(), pd[:, :50000].contiguous(), 16, workspace="static")
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_d, want_d) and torch.equal(out_l, want_l), replay
    bk.fused_status()


def test_static_scratch_rejects_problems_beyond_its_size(bk, dev):
    import torch
    q, n, k = 8192, 1 << 17, 256
    assert bk.fused_workspace_bytes(q, n, k) > bk.fused_static_scratch_bytes()
    qd = torch.zeros((8, q), device=dev)
    pd = torch.zeros((8, n), device=dev)
    with pytest.raises(bk.BitsKnnError, match="scratch memory holds 33554432"):
        bk.fused_l2_topk(qd, pd, k, workspace="static")
    with pytest.raises(bk.BitsKnnError, match="Unsupported k value: 5"):
        bk.fused_l2_topk(qd, pd, 5, workspace="static")
