"""Parity of bits-fused (distance + top-k in one kernel, through the C ABI) with the CPU oracle.

In every dimension the plain entry points report distances computed with the reference's own
arithmetic (sequential fused multiply-adds over the dimensions in order, norm - 2 dot), found
through a filter on the matrix instructions (bf16 up to 128 dimensions, fp32 from 129 to 256) that
is guaranteed never to drop a candidate, and by a plain kernel above 256 dimensions: the result
must equal the oracle's BIT FOR BIT, values and labels, equal distances by lower index ("default"
below).  With the distances taken from the fp32 matrix instructions ("mfma": BITSKNN_FUSED_FP32, on
request, up to 256 dimensions) or from bf16x3 products they are not
bit-identical to the reference's; the bar there (the stated tolerance of this path) is the k-th
neighbour distance within 1e-5 relative of the oracle's -- of the completed distance
(value + ||q||^2) for dim >= 16, of the reported partial distance below that, see tests/parity.py --
and recall@k >= 0.999 against the oracle's neighbour sets.  Structure is checked exactly in every
mode: ascending order, distinct in-range labels, and every reported distance equal to the oracle's
distance of the reported label (to 1e-5 of the magnitude of the terms that cancel in it).
"""
import numpy as np
import pytest

from parity import REL, assert_kth_distance

pytestmark = pytest.mark.gpu


def _dm(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a.T)).contiguous().to(dev)


def _fused(bk, dev, points, queries, k, params=(8, 4, 2), bqd=1, dim_mult=1, workspace=None, arithmetic=None):
    import torch
    pd = _dm(points, dev).reshape(points.shape[1], points.shape[0])
    qd = _dm(queries, dev).reshape(queries.shape[1], queries.shape[0])
    if arithmetic == "image":
        # the default arithmetic with the stages cut once into the workspace (forced: the library
        # itself only does it from a few thousand queries on), ranges as the library chooses
        od, ol = bk.fused_l2_topk(qd, pd, k, workspace="image", tuning=(0, 0, 1))
        bk.fused_status()
        return od.cpu().numpy(), ol.cpu().numpy()
    if arithmetic == "big":
        # the default arithmetic in workgroups of 256 queries (forced: the library itself takes them
        # where they fill the chip), ranges as the library chooses ("one-range": a single one)
        od, ol = bk.fused_l2_topk(qd, pd, k, workspace=None if workspace == "one-range" else "auto",
                                  tuning=(0, 0, 0, 256))
        bk.fused_status()
        return od.cpu().numpy(), ol.cpu().numpy()
    od, ol = bk.fused_l2_topk(qd, pd, k, params, bqd, dim_mult, workspace=workspace, arithmetic=arithmetic)
    bk.fused_status()  # synchronises; raises if a wave gave up a wait for a stage
    return od.cpu().numpy(), ol.cpu().numpy()


MODES = ["default", "mfma"]
MODES_AND_IMAGE = ["default", "mfma", "image", "big"]


def _arith(bk, mode):
    """C-ABI arithmetic of a test mode: None = the plain entry points; "image" = the default
    arithmetic through bitsknn_fused_l2_topk_f32_tuned with the stage image, "big" = the same in
    workgroups of 256 queries (see _fused)"""
    return {"default": None, "mfma": bk.FUSED_FP32, "bf16x3": bk.FUSED_BF16X3, "image": "image", "big": "big"}[mode]


def _bits(mode, dim):
    """whether the result of this mode must equal the oracle's bit for bit"""
    return mode in ("default", "image", "big") or dim > 256


def _check(oracle, points, queries, k, gd, gl, min_recall=0.999, bar_dim=None, bits=False):
    n = points.shape[0]
    part = oracle.dist(queries, points, "partial")
    ed, el = oracle.topk(part, k)
    if bits:
        kk = min(k, n)
        assert np.array_equal(gd[:, :kk].view(np.uint32), ed[:, :kk].view(np.uint32)), "values differ from the oracle's"
        assert np.array_equal(gl[:, :kk], el[:, :kk]), "labels differ from the oracle's"
        if k > n:
            assert np.all(np.isinf(gd[:, n:]))
        return 1.0
    qn = (queries.astype(np.float64) ** 2).sum(1)[:, None]
    kk = min(k, n)
    # structure
    assert np.all(gd[:, 1:kk] >= gd[:, :kk - 1]), "not ascending"
    assert gl[:, :kk].min() >= 0 and gl[:, :kk].max() < n
    for row in gl[:, :kk]:
        assert len(set(row.tolist())) == kk, "duplicate labels"
    # every reported distance is the distance of the reported label
    ref_at = np.take_along_axis(part, gl[:, :kk].astype(np.int64), axis=1)
    scale = np.abs(ref_at) + qn
    assert np.max(np.abs(gd[:, :kk] - ref_at) / scale) <= REL
    # k-th neighbour distance and recall
    # (bar_dim: data whose distances cancel harder than uniform points' do take the bar of few dimensions)
    assert_kth_distance(queries, ed[:, kk - 1], gd[:, kk - 1], bar_dim or points.shape[1], (n, queries.shape[0], k))
    recall = np.mean([len(set(a[:kk]) & set(b[:kk])) / kk for a, b in zip(gl, el)])
    if recall < min_recall:
        # Neighbours closer together than fp32 resolves (many points on a line, say): which of
        # them a correct kernel reports depends on its rounding order.  A reported label then
        # counts when its exact distance lies within the tolerance of the exact k-th distance.
        truth = oracle.dist(queries, points, "f64-partial")
        kth = np.sort(truth, axis=1)[:, kk - 1]
        at = np.take_along_axis(truth, gl[:, :kk].astype(np.int64), axis=1)
        recall = np.mean(at <= (kth + REL * (np.abs(kth) + qn[:, 0]))[:, None])
    assert recall >= min_recall, recall
    # where the oracle's neighbour gaps are far above the rounding noise the sets must be identical
    if n > kk:
        nxt = np.sort(part, axis=1)[:, kk]
        clear = (nxt - ed[:, kk - 1]) > 1e-4 * (np.abs(nxt) + qn[:, 0])
        for r in np.nonzero(clear)[0]:
            assert set(gl[r, :kk]) == set(el[r, :kk])
    if k > n:
        assert np.all(np.isinf(gd[:, n:]))
    return recall


# the reference's own fused-cache test cases (tests/topk/fused_cache_kernel_test.cu:12-82):
# (dim, k, points, queries) with items {8,4,2}, block 4, deg 2
@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("d,k,n,q", [(8, 32, 1024, 32), (16, 32, 1024, 1), (37, 32, 997, 43), (9, 16, 25, 7)])
def test_reference_unit_test_shapes(bk, dev, oracle, d, k, n, q, mode):
    p, s = oracle.generate(42, n, q, d)
    gd, gl = _fused(bk, dev, p, s, k, (8, 4, 2), 4, 2, arithmetic=_arith(bk, mode))
    _check(oracle, p, s, k, gd, gl, bits=_bits(mode, d))


@pytest.mark.parametrize("mode", MODES_AND_IMAGE)
@pytest.mark.parametrize("k", [4, 8, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("d", [4, 8, 16, 32, 64, 128, 192])
def test_all_k_values(bk, dev, oracle, k, d, mode):
    p, s = oracle.generate(100 + k + d, 20000, 150, d)
    gd, gl = _fused(bk, dev, p, s, k, arithmetic=_arith(bk, mode))
    _check(oracle, p, s, k, gd, gl, bits=_bits(mode, d))


@pytest.mark.parametrize("mode", MODES_AND_IMAGE)
@pytest.mark.parametrize("d", [1, 2, 3, 5, 7, 9, 15, 17, 31, 33, 48, 49, 63, 64, 65, 100, 113, 200, 256, 257, 300, 520])
def test_dimensions(bk, dev, oracle, d, mode):
    p, s = oracle.generate(d, 3000, 70, d)
    gd, gl = _fused(bk, dev, p, s, 16, (2, 4, 1), 1, 1, arithmetic=_arith(bk, mode))
    _check(oracle, p, s, 16, gd, gl, bits=_bits(mode, d))


@pytest.mark.parametrize("mode", MODES_AND_IMAGE)
@pytest.mark.parametrize("n,q", [(1, 1), (31, 5), (32, 33), (33, 127), (255, 128), (257, 129), (1000, 300), (5001, 1)])
def test_ragged_counts(bk, dev, oracle, n, q, mode):
    for d in (8, 24, 72, 200):
        p, s = oracle.generate(n + q + d, n, q, d)
        for k in (4, 32):
            gd, gl = _fused(bk, dev, p, s, k, arithmetic=_arith(bk, mode))
            _check(oracle, p, s, k, gd, gl, bits=_bits(mode, d))


# points per stage by padded dimension.  fp32 matrix instructions: 256 up to 16 dimensions, 128 / 64
# / 32 for 32 / 64 / 128; the exact arithmetic and bf16x3: 128 up to 16 dimensions, 64 / 32 for 32 / 64
# (the exact arithmetic in workgroups of 256 queries: twice that, and 32 in 65 .. 128 dimensions,
# which have this shape only)
@pytest.mark.parametrize("d", [8, 16, 32, 64, 100, 200])
@pytest.mark.parametrize("mode", ["default", "mfma", "bf16x3", "image", "big"])
def test_point_counts_around_whole_stages(bk, dev, oracle, d, mode):
    # one to five stages, each count one short of, at and one past a whole stage: the ring of three
    # stage buffers starts, wraps around and ends at every position
    if mode == "bf16x3" and not 9 <= d <= 64:
        pytest.skip("bf16x3 products serve 9 to 64 dimensions")
    if mode == "image" and d > 64:
        pytest.skip("the stage image serves up to 64 dimensions")
    if mode == "big":
        stage = {8: 256, 16: 256, 32: 128, 64: 64, 100: 32, 200: 32}[d]
    elif mode == "mfma" or d > 64:
        stage = {8: 256, 16: 256, 32: 128, 64: 64, 100: 32, 200: 32}[d]
    else:
        stage = {8: 128, 16: 128, 32: 64, 64: 32}[d]
    q = 130
    for stages in (1, 2, 3, 4, 5):
        for n in (stages * stage - 1, stages * stage, stages * stage + 1):
            p, s = oracle.generate(1000 * stages + n + d, n, q, d)
            gd, gl = _fused(bk, dev, p, s, 16, arithmetic=_arith(bk, mode))
            _check(oracle, p, s, 16, gd, gl, bits=_bits(mode, d))


@pytest.mark.parametrize("n,q,d,k", [(20000, 150, 8, 32), (70001, 300, 16, 16), (300000, 33, 32, 4),
                                     (9000, 1000, 8, 64), (131072, 1024, 5, 128), (40000, 128, 8, 256),
                                     (50000, 200, 16, 256), (33000, 77, 13, 128)])
def test_point_split_variant_with_workspace(bk, dev, oracle, n, q, d, k):
    """The workspace entry point cuts the points into ranges when queries are few; its result must
    equal the plain entry point's bit for bit (same distances, canonical ties), also where the
    kernel over ranges has another geometry (64-slot buffers and smaller stages for lists of 128
    and more in up to 16 dimensions)."""
    import torch
    p, s = oracle.generate(n + q + d, n, q, d)
    # the workspace holds partial lists only, whatever the list length: never the distance matrix
    need = bk.fused_workspace_bytes(q, n, k)
    assert need % (8 * q * k) == 0 and 0 < need <= 8 * q * 64 * k
    gd, gl = _fused(bk, dev, p, s, k, workspace="auto")
    _check(oracle, p, s, k, gd, gl, bits=True)
    pd, pl = _fused(bk, dev, p, s, k)
    assert np.array_equal(gd, pd) and np.array_equal(gl, pl)
    # the same through the fp32 matrix instructions (the kernel over ranges has another geometry there)
    md, ml = _fused(bk, dev, p, s, k, workspace="auto", arithmetic=bk.FUSED_FP32)
    _check(oracle, p, s, k, md, ml)
    pd, pl = _fused(bk, dev, p, s, k, arithmetic=bk.FUSED_FP32)
    assert np.array_equal(md, pd) and np.array_equal(ml, pl)


def test_smaller_workspace_means_fewer_ranges(bk, dev, oracle):
    """A workspace below what bitsknn_fused_workspace_bytes asks for is not an error: the call uses
    the ranges that fit (down to none) and returns the same lists bit for bit."""
    import torch
    n, q, d, k = 100000, 256, 8, 32
    p, s = oracle.generate(11, n, q, d)
    need = bk.fused_workspace_bytes(q, n, k)
    assert need >= 4 * 8 * q * k
    want = _fused(bk, dev, p, s, k)
    for size in (need, need - 8, need // 2, need // 4 + 8, 8 * q * k, 16):
        gd, gl = _fused(bk, dev, p, s, k, workspace=torch.empty(size, dtype=torch.uint8, device=dev))
        assert np.array_equal(gd, want[0]) and np.array_equal(gl, want[1]), size


def test_duplicate_points_are_ordered_by_index(bk, dev, oracle):
    # every point appears 4 times: equal distances must come out by ascending index
    base, s = oracle.generate(5, 500, 64, 8)
    p = np.concatenate([base, base, base, base])
    part = oracle.dist(s, p, "partial")
    ed, el = oracle.topk(part, 32)
    for arithmetic in (None, bk.FUSED_FP32):
        gd, gl = _fused(bk, dev, p, s, 32, arithmetic=arithmetic)
        assert np.array_equal(gl, el)
        if arithmetic is None:
            assert np.array_equal(gd.view(np.uint32), ed.view(np.uint32))


@pytest.mark.parametrize("mode", MODES_AND_IMAGE)
@pytest.mark.parametrize("d,k", [(8, 32), (16, 4), (16, 32), (32, 32), (64, 16), (16, 64), (100, 32)])
def test_points_that_come_ever_closer(bk, dev, oracle, d, k, mode):
    # Every point is nearer to every query than all points before it, so every tile brings each
    # query 32 candidates: more than a query buffer of 24 slots holds even when it is empty (the
    # geometries with three stages in LDS), which has such a tile appended in two halves.  Small
    # integer coordinates keep the arithmetic exact, so the result must equal the oracle's bit for
    # bit.
    n, q = 2000, 200
    rng = np.random.default_rng(d * 100 + k)
    s = rng.integers(-2, 3, size=(q, d)).astype(np.float32)
    p = np.zeros((n, d), dtype=np.float32)
    p[:, 0] = 20 + (n - 1 - np.arange(n))         # 2019, 2018, ..., 20 along the first axis
    p[:, 1:3] = rng.integers(-1, 2, size=(n, 2))  # (a step along it outweighs what these can add)
    part = oracle.dist(s, p, "partial")
    assert np.all(np.diff(part, axis=1) < 0), "the points must approach every query"
    gd, gl = _fused(bk, dev, p, s, k, arithmetic=_arith(bk, mode))
    ed, el = oracle.topk(part, k)
    assert np.array_equal(gd, ed) and np.array_equal(gl, el)


def test_exact_arithmetic_is_bit_exact(bk, dev, oracle):
    # small integers: every product and sum is exact in fp32, so the fused result must equal the
    # oracle bit for bit, labels included (heavy ties)
    rng = np.random.default_rng(3)
    p = rng.integers(-8, 9, size=(4000, 12)).astype(np.float32)
    s = rng.integers(-8, 9, size=(100, 12)).astype(np.float32)
    ed, el = oracle.topk(oracle.dist(s, p, "partial"), 64)
    for arithmetic in (None, bk.FUSED_FP32, bk.FUSED_BF16X3):
        gd, gl = _fused(bk, dev, p, s, 64, arithmetic=arithmetic)
        assert np.array_equal(gd, ed) and np.array_equal(gl, el)


@pytest.mark.parametrize("d", [5, 8, 16, 24, 32, 64, 72, 100, 128, 160, 256])
@pytest.mark.parametrize("kind", ["tiny", "huge", "signs", "near", "ranges-of-magnitude", "subnormal", "constant"])
def test_the_filter_never_drops_a_neighbour(bk, dev, oracle, d, kind):
    """The filter of the default arithmetic promises a lower bound of every distance (bf16 pieces,
    an error budget relative to ||q||^2 + 2 ||p||^2): a neighbour it dropped would show as a
    difference from the oracle.  Inputs chosen against that budget: values near the ends of the
    fp32 range, mixed signs, points so near the queries that norm and dot product cancel almost
    completely (nearly every value then ties within the slack and is looked at exactly), coordinates
    spread over eight orders of magnitude, subnormal coordinates, and constant vectors.  Bit for bit
    against the oracle."""
    n, q, k = 6000, 140, 32
    rng = np.random.default_rng(d * 7 + len(kind))
    p = rng.random((n, d), dtype=np.float32)
    s = rng.random((q, d), dtype=np.float32)
    if kind == "tiny":
        p, s = p * np.float32(1e-18), s * np.float32(1e-18)
    elif kind == "huge":
        p, s = p * np.float32(3e17), s * np.float32(3e17)
    elif kind == "signs":
        p, s = (p - 0.5) * 100, (s - 0.5) * 100
    elif kind == "near":
        centre = (rng.random(d, dtype=np.float32) * 2000 - 1000).astype(np.float32)
        p = centre + (p - 0.5) * np.float32(0.01)
        s = centre + (s - 0.5) * np.float32(0.01)
    elif kind == "ranges-of-magnitude":
        scale = np.float32(10.0) ** rng.integers(-4, 5, size=d).astype(np.float32)
        p, s = (p - 0.3) * scale, (s - 0.3) * scale
    elif kind == "subnormal":
        p[:, ::2] *= np.float32(1e-41)
        s[:, ::2] *= np.float32(1e-41)
    else:
        p[:] = np.float32(0.7)
        s[:] = np.float32(0.3)
        p[::3, 0] = np.float32(0.25)
    p = np.ascontiguousarray(p, dtype=np.float32)
    s = np.ascontiguousarray(s, dtype=np.float32)
    gd, gl = _fused(bk, dev, p, s, k)
    ed, el = oracle.topk(oracle.dist(s, p, "partial"), k)
    assert np.array_equal(gd.view(np.uint32), ed.view(np.uint32)), "values differ from the oracle's"
    assert np.array_equal(gl, el), "labels differ from the oracle's"
    if kind in ("signs", "near"):
        wd, wl = _fused(bk, dev, p, s, k, workspace="auto")
        assert np.array_equal(gd, wd) and np.array_equal(gl, wl)
    # the same through the stage image (the launch that writes it cuts the points the same way) and in
    # workgroups of 256 queries
    for other in ("image", "big"):
        wd, wl = _fused(bk, dev, p, s, k, arithmetic=other)
        assert np.array_equal(gd.view(np.uint32), wd.view(np.uint32)) and np.array_equal(gl, wl), other


# reference-held checksums of the fused runs (data/fused-*.err), query 0
@pytest.mark.parametrize("n,q", [(131072, 8192), (262144, 4096)])
def test_golden_fused_checksums(bk, dev, oracle, golden, n, q):
    checked = 0
    for d in (4, 8, 16):
        p, s = oracle.generate(24, n, q, d)
        part0 = oracle.dist(s[:64], p, "partial")
        for rec in golden:
            if rec["family"] != "fused" or (rec["n"], rec["q"], rec["d"]) != (n, q, d):
                continue
            k = rec["k"]
            gd, gl = _fused(bk, dev, p, s, k)
            assert str(oracle.checksum(gl[0])) in rec["checksums"], (rec, oracle.checksum(gl[0]))
            _check(oracle, p, s[:64], k, gd[:64], gl[:64], bits=True)
            checked += 1
    assert checked >= 18


def test_parameter_validation(bk, dev):
    import torch
    qd = torch.zeros((8, 4), device=dev)
    pd = torch.zeros((8, 100), device=dev)
    for args, msg in (((qd, pd, 5), "Unsupported k value: 5"),
                      ((qd, pd, 32, (3, 4, 2)), "Unsupported queries_reg value: 3"),
                      ((qd, pd, 32, (8, 5, 2)), "Unsupported db_reg value: 5"),
                      ((qd, pd, 32, (8, 4, 3)), "Unsupported dim_reg value: 3"),
                      ((qd, pd, 32, (8, 4, 2), 3), "Unsupported query_block_size value: 3"),
                      ((qd, pd, 32, (8, 4, 2), 1, 3), "Unsupported dim_mult value: 3"),
                      ((qd, pd, 32, (8, 4, 4), 1, 4), "Dimension of vectors must not be lower than 16, but is 8")):
        with pytest.raises(bk.BitsKnnError, match=msg):
            bk.fused_l2_topk(*args)


@pytest.mark.parametrize("k", [16, 128])
@pytest.mark.parametrize("d", [256, 128, 64])
def test_point_matrix_of_2_gib_takes_the_plain_loads(bk, dev, oracle, k, d):
    """dim * n * 4 bytes >= 2 GiB: the staging falls back from buffer loads (32-bit offsets) to
    ordinary loads (k = 128: also in the launch over a sample of the points).  Checked against the
    GEMM distance kernel + bits top-k on the same inputs: k-th distance within 1e-5 of the scale of
    the cancelling terms, recall >= 0.999; the lists of the first queries also bit for bit against
    the oracle."""
    import torch
    gen = torch.Generator(device=dev)
    gen.manual_seed(9)
    q, n = 128, 2_200_000 * 256 // d
    assert d * n * 4 >= 1 << 31
    queries = torch.rand((d, q), device=dev, generator=gen)
    points = torch.rand((d, n), device=dev, generator=gen)
    fd, fl = bk.fused_l2_topk(queries, points, k)
    dist = bk.distances(queries, points, bk.DIST_PARTIAL_L2)
    gd, gl = bk.topk_bits(dist, k, 256, 8)
    torch.cuda.synchronize()
    scale = (queries.double() ** 2).sum(0)[:, None] + gd.double().abs()
    assert float(((fd.double() - gd.double()).abs() / scale).max()) < 1e-5
    same = sum(len(set(a.tolist()) & set(b.tolist())) for a, b in zip(fl.cpu(), gl.cpu())) / (q * k)
    assert same >= 0.999
    # and the reported distances belong to the reported labels
    at = torch.gather(dist, 1, fl.long())
    assert float(((fd.double() - at.double()).abs() / scale).max()) < 1e-5
    if True:
        first = 4
        del dist, gd, gl, at
        points_h = np.ascontiguousarray(points.cpu().numpy().T)
        queries_h = np.ascontiguousarray(queries[:, :first].cpu().numpy().T)
        ed, el = oracle.topk(oracle.dist(queries_h, points_h, "partial"), k)
        assert np.array_equal(fd[:first].cpu().numpy().view(np.uint32), ed.view(np.uint32))
        assert np.array_equal(fl[:first].cpu().numpy(), el)


@pytest.mark.parametrize("n,q,d,k,workspace,mode", [(5000, 130, 300, 32, None, "default"), (20000, 300, 512, 16, None, "default"),
                                                    (3000, 70, 1000, 4, None, "default"), (25, 7, 260, 16, None, "default"),
                                                    (10, 300, 290, 128, None, "default"), (9000, 150, 384, 256, None, "default"),
                                                    (5000, 130, 300, 64, None, "mfma"), (5000, 130, 300, 8, None, "bf16x3"),
                                                    (70001, 300, 300, 16, "auto", "default"),
                                                    (131072, 100, 257, 128, "auto", "default")])
def test_more_than_256_dimensions(bk, dev, oracle, n, q, d, k, workspace, mode):
    """Above 256 dimensions every arithmetic takes the plain kernel with one query per thread, in the
    reference's arithmetic: bit for bit against the oracle, with and without ranges of points."""
    p, s = oracle.generate(n + d + k, n, q, d)
    gd, gl = _fused(bk, dev, p, s, k, arithmetic=_arith(bk, mode), workspace=workspace)
    _check(oracle, p, s, k, gd, gl, bits=True)


@pytest.mark.parametrize("k", [4, 32, 128])
def test_more_than_256_dimensions_with_equal_distances(bk, dev, oracle, k):
    """Many copies of few points: equal distances are reported by lower index, and lists whose largest
    entries tie are kept right (the plain kernel tracks the largest entries of a list in registers)."""
    rng = np.random.default_rng(k)
    n, q, d = 4000, 90, 270
    few = rng.random((12, d), dtype=np.float32)
    p = np.ascontiguousarray(few[rng.integers(0, 12, size=n)])
    p[::7] = rng.random((len(p[::7]), d), dtype=np.float32)
    s = rng.random((q, d), dtype=np.float32)
    for workspace in (None, "auto"):
        gd, gl = _fused(bk, dev, p, s, k, workspace=workspace)
        _check(oracle, p, s, k, gd, gl, bits=True)


@pytest.mark.parametrize("k", [128, 256])
def test_long_lists_stay_in_the_fused_kernel(bk, dev, oracle, k):
    """k >= 128: the workspace the library asks for holds partial lists only (never the q x n
    matrix), and with or without it the result is the fused kernel's."""
    n, q, d = 20000, 300, 24
    points, queries = oracle.generate(77, n, q, d)
    assert 0 < bk.fused_workspace_bytes(q, n, k) <= 8 * q * 64 * k and bk.fused_workspace_bytes(q, n, k) < q * n * 4
    gd, gl = _fused(bk, dev, points, queries, k, workspace="auto")
    _check(oracle, points, queries, k, gd, gl, bits=True)
    fd, fl = _fused(bk, dev, points, queries, k)
    assert np.array_equal(gd, fd) and np.array_equal(gl, fl)


def _sampled_points(n, d, small_stages, scale):
    """Points the launch over a sample visits (on at least 2^17 points, lists of 128 and more,
    or of 64 and more when the points are cut into ranges, start from radii taken from
    it): every `scale`-th stage, the one in the middle of its group.  small_stages: the stage sizes
    of the exact arithmetic and of bf16x3 products."""
    if small_stages:
        stage = 128 if d <= 16 else (64 if d <= 32 else 32)
    else:
        stage = 256 if d <= 16 else (128 if d <= 32 else (64 if d <= 64 else 32))
    stages = n // (stage * scale)
    half = scale // 2
    return np.concatenate([np.arange((s * scale + half) * stage, (s * scale + half + 1) * stage)
                           for s in range(stages)])


@pytest.mark.parametrize("d,k,mode,ranges", [(8, 64, "default", False), (8, 128, "mfma", False), (8, 256, "mfma", False),
                                             (32, 256, "mfma", False), (100, 128, "default", False), (200, 128, "default", False),
                                             (128, 64, "default", True),
                                             (8, 128, "default", False), (8, 256, "default", False),
                                             (32, 256, "default", False), (64, 128, "default", False),
                                             (16, 256, "bf16x3", False), (48, 128, "bf16x3", False),
                                             (8, 64, "mfma", True), (8, 256, "mfma", True),
                                             (16, 128, "mfma", True), (32, 64, "mfma", True),
                                             (8, 64, "default", True), (8, 256, "default", True),
                                             (16, 128, "default", True), (32, 64, "default", True),
                                             (24, 128, "bf16x3", True),
                                             (8, 64, "big", False), (16, 128, "big", False), (32, 256, "big", False),
                                             (64, 128, "big", False), (8, 256, "big", True), (32, 64, "big", True),
                                             (64, 64, "big", True)])
def test_first_radius_from_a_sample(bk, dev, oracle, d, k, mode, ranges):
    """Lists on many points start from radii that a launch over a sample of the points
    estimates, and workgroups with a query whose estimate proved too low repeat their pass; the
    result must not depend on either.  Uniform points (the estimates hold), and points whose
    sampled stages hold the only near ones, more than k of them (every estimate is too low).
    `ranges`: with a workspace, so that the few queries search the points in ranges."""
    n, q = (1 << 17) + 777, 200
    rng = np.random.default_rng(d * k)
    queries = rng.random((q, d), dtype=np.float32)
    points = rng.random((n, d), dtype=np.float32)
    arithmetic = _arith(bk, mode)
    bits = _bits(mode, d)
    workspace = "auto" if ranges else None
    if mode == "big" and not ranges:
        workspace = "one-range"
    if ranges:
        assert bk.fused_workspace_bytes(q, n, k) > 0
    gd, gl = _fused(bk, dev, points, queries, k, arithmetic=arithmetic, workspace=workspace)
    _check(oracle, points, queries, k, gd, gl, bits=bits)
    assert not np.isnan(gd).any()
    # (over ranges the sample has about 2048 points: one stage in every 64 .. 256)
    # (the workgroups of 256 queries have the stage sizes of the fp32 matrix instructions)
    sample = _sampled_points(n, d, mode == "bf16x3" or (bits and mode != "big"),
                             max(64, min(256, n // 2048)) if ranges else 64)
    assert sample.size >= 2 * 32
    points = rng.random((n, d), dtype=np.float32)
    points[:, :4] += 1.0                    # all points a step away in four dimensions ...
    points[sample] = rng.random((sample.size, d), dtype=np.float32)    # ... but the sampled ones
    queries[::2, :4] += 1.0                 # every other query sits among the far points
    gd, gl = _fused(bk, dev, points, queries, k, arithmetic=arithmetic, workspace=workspace)
    _check(oracle, points, queries, k, gd, gl, bar_dim=8, bits=bits)   # norms twice those of uniform points
    assert not np.isnan(gd).any()


@pytest.mark.parametrize("mode", MODES + ["big"])
def test_random_shapes_against_the_oracle(bk, dev, oracle, mode):
    """40 random problems over dimensions on both sides of every padded size, all list lengths,
    ragged point and query counts, with the plain entry point, the workspace the library asks for
    and a workspace that only holds partial lists."""
    import torch
    rng = np.random.default_rng(77)
    dims = [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 24, 31, 32, 33, 40, 63, 64, 65, 100, 128, 129, 200, 256, 257, 300, 511]
    for case in range(40):
        d = int(rng.choice(dims))
        k = int(rng.choice([4, 8, 16, 32, 64, 128, 256]))
        n = int(rng.choice([rng.integers(1, 300), rng.integers(300, 5000), rng.integers(5000, 30000)]))
        q = int(rng.choice([rng.integers(1, 40), rng.integers(40, 300), rng.integers(300, 600)]))
        q = max(1, min(q, int(1.5e9 / (n * d))))
        kind = case % 3
        workspace = None
        if kind == 1:
            workspace = "auto"
        elif kind == 2:
            workspace = torch.empty(max(8, 8 * q * 64 * k), dtype=torch.uint8, device=dev)
        p, s = oracle.generate(3000 + case, n, q, d)
        arithmetic = _arith(bk, mode)
        if mode == "big":
            workspace = "one-range" if kind == 0 else "auto"
        gd, gl = _fused(bk, dev, p, s, k, (2, 4, 1), 1, 1, workspace=workspace, arithmetic=arithmetic)
        try:
            _check(oracle, p, s, k, gd, gl, bits=_bits(mode, d))
        except AssertionError as e:
            raise AssertionError((case, n, q, d, k, kind)) from e


# ---- products from three bf16 pieces per operand (BITSKNN_FUSED_BF16X3, dimensions 9 .. 64) --------

@pytest.fixture
def bf16x3(bk):
    """The arithmetic argument of bitsknn_fused_l2_topk_f32_ex (chosen per call)."""
    return bk.FUSED_BF16X3


@pytest.mark.parametrize("k", [4, 8, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("d", [9, 16, 17, 32, 33, 64])
def test_bf16x3_all_k_values(bk, dev, oracle, bf16x3, k, d):
    p, s = oracle.generate(200 + k + d, 20000, 150, d)
    gd, gl = _fused(bk, dev, p, s, k, arithmetic=bf16x3)
    _check(oracle, p, s, k, gd, gl)


@pytest.mark.parametrize("n,q", [(1, 1), (31, 5), (32, 33), (63, 127), (64, 128), (65, 129), (129, 3), (1000, 300), (5001, 1)])
def test_bf16x3_ragged_counts(bk, dev, oracle, bf16x3, n, q):
    for d in (12, 31, 50):
        p, s = oracle.generate(n + q + d, n, q, d)
        for k in (4, 32):
            gd, gl = _fused(bk, dev, p, s, k, (2, 4, 1), 1, 1, arithmetic=bf16x3)
            _check(oracle, p, s, k, gd, gl)


@pytest.mark.parametrize("n,q,d,k", [(20000, 150, 12, 32), (70001, 300, 16, 16), (300000, 33, 32, 4),
                                     (9000, 1000, 24, 64), (30000, 100, 64, 32)])
def test_bf16x3_point_split_variant_with_workspace(bk, dev, oracle, bf16x3, n, q, d, k):
    p, s = oracle.generate(n + q + d, n, q, d)
    gd, gl = _fused(bk, dev, p, s, k, workspace="auto", arithmetic=bf16x3)
    _check(oracle, p, s, k, gd, gl)
    pd, pl = _fused(bk, dev, p, s, k, arithmetic=bf16x3)
    assert np.array_equal(gd, pd) and np.array_equal(gl, pl)


def test_bf16x3_random_shapes_against_the_oracle(bk, dev, oracle, bf16x3):
    import torch
    rng = np.random.default_rng(99)
    for case in range(30):
        d = int(rng.integers(9, 65))
        k = int(rng.choice([4, 8, 16, 32, 64, 128, 256]))
        n = int(rng.choice([rng.integers(1, 300), rng.integers(300, 5000), rng.integers(5000, 30000)]))
        q = int(rng.choice([rng.integers(1, 40), rng.integers(40, 300), rng.integers(300, 600)]))
        workspace = None if case % 2 == 0 else torch.empty(max(8, 8 * q * 64 * k), dtype=torch.uint8, device=dev)
        p, s = oracle.generate(4000 + case, n, q, d)
        gd, gl = _fused(bk, dev, p, s, k, (2, 4, 1), 1, 1, workspace=workspace, arithmetic=bf16x3)
        try:
            _check(oracle, p, s, k, gd, gl)
        except AssertionError as e:
            raise AssertionError((case, n, q, d, k)) from e


def test_bf16x3_is_as_accurate_as_the_fp32_matrix_instructions(bk, dev, oracle):
    """Error of the reported distances against the exact (fp64) ones, relative to the magnitude of
    the cancelling terms, for both arithmetics on the same inputs: the split products must stay at
    the level of fp32 rounding (far inside the 1e-5 bar) and within a small factor of the fp32
    matrix instructions' own error."""
    err = {}
    for d in (16, 32, 64):
        p, s = oracle.generate(900 + d, 30000, 200, d)
        truth = oracle.dist(s, p, "f64-partial")
        qn = (s.astype(np.float64) ** 2).sum(1)[:, None]
        for mode in (bk.FUSED_FP32, bk.FUSED_BF16X3):
            gd, gl = _fused(bk, dev, p, s, 64, arithmetic=mode)
            at = np.take_along_axis(truth, gl.astype(np.int64), axis=1)
            err[(d, mode)] = float(np.max(np.abs(gd - at) / (np.abs(at) + qn)))
        assert err[(d, bk.FUSED_BF16X3)] < 1e-6
        assert err[(d, bk.FUSED_BF16X3)] < 4 * err[(d, bk.FUSED_FP32)] + 1e-7


GIVE_UP_SCRIPT = r"""
import sys
sys.path[:0] = [{root!r}, {pkg!r}]
import numpy as np
import torch
import bitsknn
dev = torch.device("cuda:0")
rng = np.random.default_rng(5)
n, q, d, k = 100000, 1024, 8, 32
points = torch.from_numpy(rng.random((d, n), dtype=np.float32)).to(dev)
queries = torch.from_numpy(rng.random((d, q), dtype=np.float32)).to(dev)
print("status before any call", flush=True)
bitsknn.fused_status()
print("fused call with a poll limit of 0", flush=True)
od, ol = bitsknn.fused_l2_topk(queries, points, k)
try:
    bitsknn.fused_status()
except bitsknn.BitsKnnError as error:
    assert error.code == bitsknn.ERR_INTERNAL, error.code
    assert "ran out of polls" in str(error), str(error)
else:
    raise SystemExit("no wait gave up although the poll limit is 0")
kth = od[:, k - 1].cpu().numpy()
assert np.isnan(kth).any(), "no list is marked"
print("marked lists:", int(np.isnan(kth).sum()), "of", q, flush=True)
bitsknn.fused_status()  # the check has cleared the word
print("ok", flush=True)
"""


def test_a_wait_that_gives_up_is_reported(bk, dev):
    """The failure path of the ring of stages, forced from the host: with BITSKNN_FUSED_POLL_LIMIT=0
    (read once per process, hence the child process) every wait that finds its stage incomplete
    gives up at once.  Every kernel still ends normally; the lists of the waves concerned end in
    NaN, bitsknn_fused_status reports BITSKNN_ERR_INTERNAL once and is clear afterwards."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pkg = os.path.join(root, "bits-knn-jpdc2024_amd")
    env = dict(os.environ, BITSKNN_FUSED_POLL_LIMIT="0")
    done = subprocess.run([sys.executable, "-u", "-c", GIVE_UP_SCRIPT.format(root=root, pkg=pkg)], env=env,
                          capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, (done.stdout, done.stderr)
    assert done.stdout.strip().endswith("ok"), done.stdout
    bk.fused_status()  # this process, with the default limit, has seen no wait give up


def test_tuned_entry_point(bk, dev, oracle):
    """bitsknn_fused_l2_topk_f32_tuned: the number of ranges and the sample for the first radii are
    the caller's; the result is the same whatever they are (bit for bit in the default arithmetic),
    and values outside their ranges are rejected."""
    import torch
    n, q, d, k = (1 << 17) + 300, 260, 12, 64
    p, s = oracle.generate(404, n, q, d)
    pd = torch.from_numpy(np.ascontiguousarray(p.T)).to(dev)
    qd = torch.from_numpy(np.ascontiguousarray(s.T)).to(dev)
    ed, el = oracle.topk(oracle.dist(s, p, "partial"), k)
    space = torch.empty(8 * q * 64 * k, dtype=torch.uint8, device=dev)
    for ranges, first_radius in [(0, 0), (1, -1), (1, 64), (2, -1), (8, 256), (64, 64), (3, 32), (64, 4096)]:
        od, ol = bk.fused_l2_topk(qd, pd, k, workspace=space, tuning=(ranges, first_radius))
        bk.fused_status()
        assert np.array_equal(od.cpu().numpy().view(np.uint32), ed.view(np.uint32)), (ranges, first_radius)
        assert np.array_equal(ol.cpu().numpy(), el), (ranges, first_radius)
    # the fp32 matrix instructions through the same entry point, to the tolerance
    od, ol = bk.fused_l2_topk(qd, pd, k, workspace=space, tuning=(4, 64), arithmetic=bk.FUSED_FP32)
    bk.fused_status()
    _check(oracle, p, s, k, od.cpu().numpy(), ol.cpu().numpy())
    # without a workspace there is one range whatever is asked for
    od, ol = bk.fused_l2_topk(qd, pd, k, tuning=(16, -1))
    bk.fused_status()
    assert np.array_equal(ol.cpu().numpy(), el)
    for bad, message in (((65, 0), "ranges must be"), ((-1, 0), "ranges must be"), ((0, 1), "first_radius must be"),
                         ((0, -2), "first_radius must be"), ((0, 5000), "first_radius must be"),
                         ((0, 0, 0, 64), "workgroup must be")):
        with pytest.raises(bk.BitsKnnError, match=message):
            bk.fused_l2_topk(qd, pd, k, workspace=space, tuning=bad)


def test_stage_image(bk, dev, oracle):
    """The stage image: bitsknn_fused_image_bytes more bytes in the workspace, behind the partial
    lists, and the points are cut into the stages of the default arithmetic once per call.  Same
    result bit for bit with one range and several, with first radii from a sample, with a workspace
    that is too small for it (no image then) and through the plain workspace entry point, which
    writes it from 4096 queries on."""
    import torch
    assert bk.fused_image_bytes(32, 1 << 20) == (1 << 20) // 64 * (32 * 64 * 4 + 9 * 64 * 16)
    assert bk.fused_image_bytes(8, 1000) == 8 * (8 * 128 * 4 + 3 * 128 * 16)
    assert bk.fused_image_bytes(65, 1000) == 0 and bk.fused_image_bytes(64, 1 << 23) == 0
    n, q, d, k = (1 << 17) + 300, 260, 24, 64
    p, s = oracle.generate(405, n, q, d)
    pd = torch.from_numpy(np.ascontiguousarray(p.T)).to(dev)
    qd = torch.from_numpy(np.ascontiguousarray(s.T)).to(dev)
    ed, el = oracle.topk(oracle.dist(s, p, "partial"), k)
    lists = 8 * q * 64 * k
    space = torch.empty((lists + 255) // 256 * 256 + bk.fused_image_bytes(d, n), dtype=torch.uint8, device=dev)
    for tuning in [(1, -1, 1), (1, 64, 1), (8, -1, 1), (64, 64, 1), (3, 32, 1), (0, 0, 1), (0, 0, 0), (4, 0, -1)]:
        space.fill_(0xFF)
        od, ol = bk.fused_l2_topk(qd, pd, k, workspace=space, tuning=tuning)
        bk.fused_status()
        assert np.array_equal(od.cpu().numpy().view(np.uint32), ed.view(np.uint32)), tuning
        assert np.array_equal(ol.cpu().numpy(), el), tuning
    # a workspace with room for the lists of 4 ranges only: ranges, no image
    od, ol = bk.fused_l2_topk(qd, pd, k, workspace=space[:8 * q * 4 * k + 1000], tuning=(4, 0, 1))
    bk.fused_status()
    assert np.array_equal(ol.cpu().numpy(), el)
    # many queries: the plain workspace entry point writes the image by itself
    n, q, d, k = 30000, 4500, 8, 16
    p, s = oracle.generate(406, n, q, d)
    ed, el = oracle.topk(oracle.dist(s, p, "partial"), k)
    gd, gl = _fused(bk, dev, p, s, k, workspace="image")
    assert np.array_equal(gd.view(np.uint32), ed.view(np.uint32)) and np.array_equal(gl, el)
    with pytest.raises(bk.BitsKnnError, match="image must be"):
        bk.fused_l2_topk(qd, pd, 64, workspace=space, tuning=(0, 0, 2))
