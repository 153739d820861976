"""Parity of the distance kernels (through the C ABI) with the CPU oracle.

Bars: BITSKNN_DIST_L2 bit-exact (sequential fused multiply-add, the reference's default
distance); the MFMA kernels within 1e-5 of the oracle's partial distance relative to the
magnitude of the terms that cancel in it (||p||^2 and 2|q.p|), the k-th neighbour distance of
every query to the contract's bar (tests/parity.py), and the completed distance within the
reference test's own tolerances (tests/distance/dist_test.hpp:93-115, 164-186).
"""
import numpy as np
import pytest

from parity import assert_kth_distance

pytestmark = pytest.mark.gpu


def _dm(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a.T)).to(dev)


def _gpu_dist(bk, dev, queries, points, op):
    import torch
    out = bk.distances(_dm(queries, dev), _dm(points, dev), op)
    torch.cuda.synchronize()
    return out.cpu().numpy()


# shapes of the reference's distance tests (tests/distance/magma_dist_test.cpp:7-96,
# cublas_dist_test.cpp:6-64): (points, queries, dim)
REF_SHAPES = [(32, 32, 16), (128, 1, 16), (32, 32, 9), (1024, 32, 32), (23 * 1024, 1, 17), (64, 32, 2)]
OUR_SHAPES = [(1000, 37, 1), (4097, 130, 3), (257, 129, 64), (5000, 200, 33), (300, 260, 100), (129, 5, 8)]


@pytest.mark.parametrize("n,q,d", REF_SHAPES + OUR_SHAPES)
def test_l2_is_bit_exact(bk, dev, oracle, n, q, d):
    p, s = oracle.generate(42, n, q, d)
    got = _gpu_dist(bk, dev, s, p, bk.DIST_L2)
    exp = oracle.dist(s, p, "l2")
    assert np.array_equal(got.view(np.uint32), exp.view(np.uint32))


def test_l2_unaligned_strides(bk, dev, oracle):
    import torch
    p, s = oracle.generate(7, 1003, 45, 5)
    pd = torch.zeros((5, 1009), device=dev)
    qd = torch.zeros((5, 47), device=dev)
    pd[:, 1:1004] = torch.from_numpy(np.ascontiguousarray(p.T)).to(dev)
    qd[:, 2:47] = torch.from_numpy(np.ascontiguousarray(s.T)).to(dev)
    out = torch.full((45, 1005), -1.0, device=dev)
    bk.distances(qd[:, 2:47], pd[:, 1:1004], bk.DIST_L2, out=out[:, 1:1004])
    torch.cuda.synchronize()
    exp = oracle.dist(s, p, "l2")
    assert np.array_equal(out[:, 1:1004].cpu().numpy(), exp)
    assert (out[:, 0] == -1).all() and (out[:, 1004] == -1).all()


@pytest.mark.parametrize("op", ["partial", "expanded"])
@pytest.mark.parametrize("n,q,d", REF_SHAPES + OUR_SHAPES)
def test_mfma_distances(bk, dev, oracle, n, q, d, op):
    p, s = oracle.generate(42, n, q, d)
    got = _gpu_dist(bk, dev, s, p, bk.DIST_PARTIAL_L2 if op == "partial" else bk.DIST_EXPANDED)
    exp = oracle.dist(s, p, "partial")
    truth = oracle.dist(s, p, "f64-partial")
    # the terms that cancel in an entry: ||p||^2 and 2|q.p| (exact values)
    p64, s64 = p.astype(np.float64), s.astype(np.float64)
    scale = (p64 ** 2).sum(1)[None, :] + 2.0 * np.abs(s64 @ p64.T)
    assert np.max(np.abs(got - exp) / scale) < 1e-5
    assert np.max(np.abs(got - truth) / scale) < 1e-5
    # the k-th neighbour distance of every query (k = 16, or all points when there are fewer)
    kk = min(16, n)
    assert_kth_distance(s, np.sort(exp, axis=1)[:, kk - 1], np.sort(got, axis=1)[:, kk - 1], d, (n, q, d, op))
    # the reference's own check: add ||q||^2 on the CPU, compare with the plain triple loop at 1e-3
    full = got.astype(np.float64) + (s.astype(np.float64) ** 2).sum(1)[:, None]
    ref_full = oracle.dist(s, p, "f64")
    assert np.allclose(full, ref_full, rtol=1e-3, atol=1e-5)


def test_mfma_operand_orientation(bk, dev, oracle):
    # one-hot vectors make every entry of q.p identify its (query, point, dimension): a transposed
    # or mis-tiled operand cannot pass
    n, q, d = 300, 200, 40
    rng = np.random.default_rng(0)
    p = np.zeros((n, d), dtype=np.float32)
    s = np.zeros((q, d), dtype=np.float32)
    p[np.arange(n), rng.integers(0, d, n)] = np.arange(1, n + 1, dtype=np.float32)
    s[np.arange(q), rng.integers(0, d, q)] = np.arange(1, q + 1, dtype=np.float32) / 4
    got = _gpu_dist(bk, dev, s, p, bk.DIST_PARTIAL_L2)
    assert np.array_equal(got, oracle.dist(s, p, "partial"))  # all products exact in fp32


def test_knn_through_both_distances_meets_the_recall_bar(bk, dev, oracle):
    """GEMM distance + bits top-k (k = 64, d = 64): k-th neighbour distance within 1e-5 relative,
    recall@k >= 0.999 against the reference arithmetic."""
    import torch
    n, q, d, k = 1 << 16, 256, 64, 64
    p, s = oracle.generate(24, n, q, d)
    dist = bk.distances(_dm(s, dev), _dm(p, dev), bk.DIST_PARTIAL_L2)
    gd, gl = bk.topk_bits(dist, k, 256, 8)
    torch.cuda.synchronize()
    ed, el = oracle.topk(oracle.dist(s, p, "partial"), k)
    gd, gl = gd.cpu().numpy(), gl.cpu().numpy()
    recall = np.mean([len(set(a) & set(b)) / k for a, b in zip(gl, el)])
    assert recall >= 0.999, recall
    completed, _, _ = assert_kth_distance(s, ed[:, -1], gd[:, -1], d, "gemm + bits")
    assert completed < 1e-5
    # and the top-k of the device matrix itself is bit-exact
    od, ol = oracle.topk(dist.cpu().numpy(), k)
    assert np.array_equal(gd, od) and np.array_equal(gl, ol)


def test_golden_fused_run_checksums_via_two_phase(bk, dev, oracle, golden):
    """Reference-held checksums of the fused runs (data/fused-*.err) reproduced by the two-phase
    path on the device: exact L2 distances + bits top-k, query 0."""
    import torch
    checked = 0
    for n, q, d in ((131072, 8192, 4), (131072, 8192, 8), (131072, 8192, 16), (262144, 4096, 16)):
        p, s = oracle.generate(24, n, q, d)
        dist = bk.distances(_dm(s[:8], dev), _dm(p, dev), bk.DIST_L2)
        part = bk.distances(_dm(s[:8], dev), _dm(p, dev), bk.DIST_PARTIAL_L2)
        for rec in golden:
            if rec["family"] != "fused" or (rec["n"], rec["q"], rec["d"]) != (n, q, d):
                continue
            for m in (dist, part):
                _, gl = bk.topk_bits(m, rec["k"], 256, 8)
                torch.cuda.synchronize()
                assert str(oracle.checksum(gl[0].cpu().numpy())) in rec["checksums"], rec
            checked += 1
    assert checked >= 24


def test_dist_errors(bk, dev):
    import torch
    a = torch.zeros((4, 10), device=dev)
    with pytest.raises(bk.BitsKnnError, match="Unsupported distance"):
        bk.distances(a, a, 7)


@pytest.mark.parametrize("d", [8, 16, 32, 48, 64, 100, 128])
def test_pipelined_and_plain_kernels_give_the_same_bits(bk, dev, d):
    """Whole 128-query blocks x whole stages take the pipelined kernel, everything else (here: the
    same problem written into a matrix whose rows are not 16-byte aligned) the plain one.  Both
    add the same products in the same order."""
    import torch
    gen = torch.Generator(device=dev)
    gen.manual_seed(d)
    q, n = 384, 4096 * 2 + 640 + 37          # interior + a ragged last stage + ragged columns
    queries = torch.rand((d, q), device=dev, generator=gen) - 0.5
    points = torch.rand((d, n), device=dev, generator=gen) - 0.5
    out_a = torch.full((q, n + 3), -7.0, device=dev)
    assert (n + 3) % 4 == 0
    bk.distances(queries, points, bk.DIST_PARTIAL_L2, out=out_a[:, :n])       # row stride n+3: aligned
    out_b = torch.full((q, n + 2), -7.0, device=dev)
    bk.distances(queries, points, bk.DIST_PARTIAL_L2, out=out_b[:, :n])       # row stride n+2: unaligned
    torch.cuda.synchronize()
    assert torch.equal(out_a[:, :n].view(torch.int32), out_b[:, :n].view(torch.int32))
    assert (out_a[:, n:] == -7.0).all() and (out_b[:, n:] == -7.0).all()
    # ragged query count: the last 5 queries go through the plain kernel
    out_c = torch.full((q + 5, n + 3), -7.0, device=dev)
    more = torch.cat([queries, queries[:, :5]], dim=1).contiguous()
    bk.distances(more, points, bk.DIST_PARTIAL_L2, out=out_c[:, :n])
    torch.cuda.synchronize()
    assert torch.equal(out_c[:q, :n], out_a[:, :n]) and torch.equal(out_c[q:, :n], out_a[:5, :n])


def test_config_4_full_size_samples(bk, dev):
    """The 4096 x 2^20 x 64 distance matrix (16 GiB): a million sampled entries against float64
    arithmetic on the same inputs (1e-5 of the scale of the cancelling terms), and whole rows
    against the plain kernel on an unaligned copy of the problem (bit for bit)."""
    import torch
    gen = torch.Generator(device=dev)
    gen.manual_seed(4)
    q, n, d = 4096, 1 << 20, 64
    queries = torch.rand((d, q), device=dev, generator=gen)
    points = torch.rand((d, n), device=dev, generator=gen)
    out = bk.distances(queries, points, bk.DIST_PARTIAL_L2)
    torch.cuda.synchronize()
    qi = torch.randint(0, q, (1 << 20,), device=dev, generator=gen)
    pj = torch.randint(0, n, (1 << 20,), device=dev, generator=gen)
    qs = queries.double()[:, qi]
    ps = points.double()[:, pj]
    exact = (ps * ps).sum(0) - 2.0 * (qs * ps).sum(0)
    scale = 2.0 * (ps * ps).sum(0) + (qs * qs).sum(0)
    got = out[qi, pj].double()
    assert float(((got - exact).abs() / scale).max()) < 1e-5
    # first and last 128-query block, a slice of columns that starts inside a stage
    sub = points[:, 5000:5000 + 8192 + 77].contiguous()
    for q0 in (0, q - 128):
        ref = torch.empty((128, sub.shape[1] + 1), device=dev)
        bk.distances(queries[:, q0:q0 + 128].contiguous(), sub, bk.DIST_PARTIAL_L2, out=ref[:, :sub.shape[1]])
        torch.cuda.synchronize()
        assert torch.equal(ref[:, :sub.shape[1]], out[q0:q0 + 128, 5000:5000 + sub.shape[1]])


def test_random_shapes_and_strides_against_the_oracle(bk, dev, oracle):
    """40 random problems: all three operations, dimensions on both sides of every padded size,
    padded and offset views of queries, points and the output matrix (aligned and unaligned rows,
    which select between the pipelined kernel, the plain kernel and their store variants)."""
    import torch
    rng = np.random.default_rng(31)
    dims = [1, 2, 3, 5, 8, 9, 16, 17, 31, 32, 33, 63, 64, 65, 100, 128, 129, 200, 256]
    codes = {"l2": bk.DIST_L2, "partial": bk.DIST_PARTIAL_L2, "expanded": bk.DIST_EXPANDED}
    for case in range(40):
        d = int(rng.choice(dims))
        n = int(rng.choice([rng.integers(1, 300), rng.integers(300, 9000), rng.integers(9000, 50000)]))
        q = int(rng.choice([rng.integers(1, 140), rng.integers(128, 600), rng.integers(256, 1200)]))
        q = max(1, min(q, int(2e9 / (n * d))))
        op = ["l2", "partial", "expanded"][case % 3]
        qpad, ppad, opad, off = (int(rng.choice(c)) for c in ([0, 0, 1, 3, 4], [0, 0, 1, 4, 5],
                                                              [0, 0, 1, 4, 28, 32], [0, 0, 1, 4]))
        p, s = oracle.generate(700 + case, n, q, d)
        pd = torch.zeros((d, n + ppad + off), device=dev)
        qd = torch.zeros((d, q + qpad + off), device=dev)
        pd[:, off:off + n] = torch.from_numpy(np.ascontiguousarray(p.T)).to(dev)
        qd[:, off:off + q] = torch.from_numpy(np.ascontiguousarray(s.T)).to(dev)
        out = torch.full((q, n + opad + off), -7.0, device=dev)
        bk.distances(qd[:, off:off + q], pd[:, off:off + n], codes[op], out=out[:, off:off + n])
        torch.cuda.synchronize()
        what = (case, n, q, d, op, qpad, ppad, opad, off)
        got = out[:, off:off + n].cpu().numpy()
        assert (out[:, :off] == -7).all() and (out[:, off + n:] == -7).all(), what
        if op == "l2":
            assert np.array_equal(got.view(np.uint32), oracle.dist(s, p, "l2").view(np.uint32)), what
        else:
            exp = oracle.dist(s, p, "partial")
            scale = (p.astype(np.float64) ** 2).sum(1)[None, :] * 2 + (s.astype(np.float64) ** 2).sum(1)[:, None]
            assert np.max(np.abs(got - exp) / np.maximum(scale, 1e-30)) < 1e-5, what


# ---- BITSKNN_DIST_PARTIAL_L2_BF16X3: products from three bf16 pieces per operand (dimensions 33 .. 64) ----

@pytest.mark.parametrize("n,q,d", [(1000, 37, 33), (4097, 130, 40), (257, 129, 64), (5000, 200, 48), (129, 5, 63),
                                   (16385, 129, 64), (70000, 300, 50), (32, 32, 16), (1024, 32, 32), (300, 7, 100)])
def test_bf16x3_distances(bk, dev, oracle, n, q, d):
    """Same bar as the fp32 matrix instructions (1e-5 of the cancelling terms, measured: a few
    1e-7), including the dimensions and shapes for which the operation falls back to them."""
    p, s = oracle.generate(77, n, q, d)
    got = _gpu_dist(bk, dev, s, p, bk.DIST_PARTIAL_L2_BF16X3)
    fp32 = _gpu_dist(bk, dev, s, p, bk.DIST_PARTIAL_L2)
    truth = oracle.dist(s, p, "f64-partial")
    scale = (p.astype(np.float64) ** 2).sum(1)[None, :] * 2 + (s.astype(np.float64) ** 2).sum(1)[:, None]
    err = np.max(np.abs(got - truth) / scale)
    err32 = np.max(np.abs(fp32 - truth) / scale)
    assert err < 1e-6 and err < 4 * err32 + 1e-7
    if d <= 32 or d > 64:
        assert np.array_equal(got, fp32)


def test_bf16x3_distances_views_and_ragged_ends(bk, dev, oracle):
    """Padded and offset views: aligned rows take the bf16x3 kernel (whole and ragged last tiles,
    rows beyond the last query of a wave), unaligned ones the fp32 kernels; nothing outside the
    view is written."""
    import torch
    for case, (n, q, opad, off) in enumerate([(1003, 45, 1, 0), (1003, 45, 5, 4), (2050, 130, 2, 0), (64, 33, 0, 0),
                                              (16384 + 37, 100, 3, 0), (999, 45, 0, 1)]):
        d = 33 + 7 * case
        p, s = oracle.generate(17 + case, n, q, d)
        out = torch.full((q, n + opad + off), -7.0, device=dev)
        bk.distances(_dm(s, dev), _dm(p, dev), bk.DIST_PARTIAL_L2_BF16X3, out=out[:, off:off + n])
        torch.cuda.synchronize()
        assert (out[:, :off] == -7).all() and (out[:, off + n:] == -7).all()
        exp = oracle.dist(s, p, "partial")
        scale = (p.astype(np.float64) ** 2).sum(1)[None, :] * 2 + (s.astype(np.float64) ** 2).sum(1)[:, None]
        assert np.max(np.abs(out[:, off:off + n].cpu().numpy() - exp) / scale) < 1e-5, (n, q, d, opad, off)


@pytest.mark.parametrize("op", ["l2", "partial", "expanded"])
@pytest.mark.parametrize("q,n,d", [(37, 1000, 5), (130, 4097, 32), (64, 300, 100), (1, 1, 1), (33, 129, 64)])
def test_the_four_layout_combinations(bk, dev, oracle, op, q, n, d):
    """bitsknn_dist_layout_f32: points and queries in either layout of the reference's knn_args
    (src/distance/cublas_distance.cu:122-149 serves the four combinations); every combination must
    give the matrix of the dim-major entry point bit for bit."""
    import torch
    code = {"l2": bk.DIST_L2, "partial": bk.DIST_PARTIAL_L2, "expanded": bk.DIST_EXPANDED}[op]
    points, queries = oracle.generate(q + n + d, n, q, d)
    p_rows = torch.from_numpy(points).to(dev)
    q_rows = torch.from_numpy(queries).to(dev)
    p_dm = p_rows.t().contiguous()
    q_dm = q_rows.t().contiguous()
    want = bk.distances(q_dm, p_dm, code)
    torch.cuda.synchronize()
    for q_layout, q_in in ((bk.LAYOUT_ROW_MAJOR, q_rows), (bk.LAYOUT_COLUMN_MAJOR, q_dm)):
        for p_layout, p_in in ((bk.LAYOUT_ROW_MAJOR, p_rows), (bk.LAYOUT_COLUMN_MAJOR, p_dm)):
            got = bk.distances_layout(q_in, q_layout, p_in, p_layout, code)
            torch.cuda.synchronize()
            assert torch.equal(got, want), (q_layout, p_layout)
    if op == "l2":
        assert np.array_equal(want.cpu().numpy(), oracle.dist(queries, points, "l2"))


def test_layout_entry_point_validation(bk, dev):
    import torch
    a = torch.zeros((10, 4), device=dev)
    square = torch.zeros((4, 4), device=dev)
    with pytest.raises(bk.BitsKnnError, match="unknown layout 7"):
        bk.distances_layout(square, 7, square, bk.LAYOUT_ROW_MAJOR)
    L = bk.lib()
    assert L.bitsknn_dist_layout_workspace_bytes(4, 10, 10, bk.LAYOUT_COLUMN_MAJOR, bk.LAYOUT_COLUMN_MAJOR) == 0
    assert L.bitsknn_dist_layout_workspace_bytes(4, 10, 13, bk.LAYOUT_ROW_MAJOR, bk.LAYOUT_ROW_MAJOR) == 4 * (12 + 16) * 4
    out = torch.empty((10, 10), device=dev)
    status = L.bitsknn_dist_layout_f32(bk.DIST_L2, 4, 10, 10, a.data_ptr(), bk.LAYOUT_ROW_MAJOR, 4, a.data_ptr(),
                                       bk.LAYOUT_ROW_MAJOR, 4, out.data_ptr(), 10, None, 0, None)
    assert status == bk.ERR_INVALID and b"workspace" in L.bitsknn_last_error()
