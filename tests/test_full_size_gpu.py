"""The benchmark's workloads at their full sizes, checked on samples against the CPU oracle.

The oracle cannot redo a 4 GiB matrix or 2^36 pairs in a test, so every case runs the kernel on the
whole problem, checks size-independent properties on the whole result and compares a sample of
rows or queries with the oracle: top-k bit for bit, distances to the bar of tests/parity.py.  The
instantiations are the ones the benchmark times (workgroup size, values per thread, plain or
prefetching variant) and the ones the shipped optima file names.

Counterparts in the reference: tests/topk/bits_knn_test.cpp:7-63 and
tests/topk/fused_cache_kernel_test.cu:12-82 (small shapes only).
"""
import numpy as np
import pytest

from parity import MIN_RECALL, assert_kth_distance

pytestmark = pytest.mark.gpu


def _sample(count, samples):
    step = max(1, count // samples)
    return list(range(step // 2, count, step))[:samples]


def _topk_properties(torch, m, od, ol, k):
    # ascending; every value is the matrix entry its label points to; equal values by ascending
    # label; distinct labels; nothing smaller left behind
    assert bool((od[:, 1:] >= od[:, :-1]).all())
    assert torch.equal(torch.gather(m, 1, ol.long()), od)
    same = od[:, 1:] == od[:, :-1]
    assert bool((ol[:, 1:][same] > ol[:, :-1][same]).all())
    sorted_labels = torch.sort(ol, dim=1).values
    assert bool((sorted_labels[:, 1:] != sorted_labels[:, :-1]).all())
    # at most k - 1 entries of a row are below its k-th value, at least k are not above it
    kth = od[:, -1:]
    assert bool(((m < kth).sum(dim=1) <= k - 1).all())
    assert bool(((m <= kth).sum(dim=1) >= k).all())


def _check_topk_sample(torch, oracle, cache, m, sample, od, ol, k):
    if "rows" not in cache:
        cache["rows"] = m[sample].cpu().numpy()
    if k not in cache:
        cache[k] = oracle.topk(cache["rows"], k)
    ed, el = cache[k]
    assert np.array_equal(od[sample].cpu().numpy().view(np.uint32), ed.view(np.uint32)), "values differ"
    assert np.array_equal(ol[sample].cpu().numpy(), el), "labels differ"


# ---- config 1: the CPU reference's own case, 1024 x 65,536 from seed 24, k = 32 ----------------

@pytest.mark.parametrize("block,batch,prefetch", [(256, 8, False), (128, 16, False), (512, 4, True)])
def test_the_cpu_reference_matrix_through_the_hip_path(bk, dev, oracle, block, batch, prefetch):
    """The matrix the CPU baseline is timed on (seeded generator of the reference, 1024 x 65,536,
    k = 32) through bitsknn_topk_bits_f32, against the canonical oracle and against the restated
    serial (reference src/topk/serial_knn.cpp:35-54: full sort of every row) and parallel
    (src/topk/parallel_knn.cpp:30-65: OpenMP heap) selections.  Values bit for bit with all three;
    labels bit for bit with the canonical oracle everywhere, and with the two restated CPU
    selections on every row whose k + 1 smallest values are distinct (they order by distance
    alone, so equal values may come out in either order there)."""
    import torch
    rows, cols, k = 1024, 65536, 32
    m = oracle.uniform_matrix(24, rows, cols)
    od, ol = bk.topk_bits(torch.from_numpy(m).to(dev), k, block, batch, prefetch)
    torch.cuda.synchronize()
    gd, gl = od.cpu().numpy(), ol.cpu().numpy()
    ed, el = oracle.topk(m, k)
    assert np.array_equal(gd.view(np.uint32), ed.view(np.uint32)), "values differ from the canonical oracle"
    assert np.array_equal(gl, el), "labels differ from the canonical oracle"
    sd, sl = oracle.topk_serial(m, k)
    pd, pl, _ = oracle.topk_parallel(m, k, 8)
    assert np.array_equal(gd.view(np.uint32), sd.view(np.uint32)), "values differ from serial_knn"
    assert np.array_equal(gd.view(np.uint32), pd.view(np.uint32)), "values differ from parallel_knn"
    smallest = np.sort(np.partition(m, k + 1, axis=1)[:, :k + 1], axis=1)
    distinct = np.all(smallest[:, 1:] != smallest[:, :-1], axis=1)
    assert distinct.sum() >= rows - 8, "seeded uniform rows should hardly ever tie among their smallest values"
    assert np.array_equal(gl[distinct], sl[distinct]), "labels differ from serial_knn"
    assert np.array_equal(gl[distinct], pl[distinct]), "labels differ from parallel_knn"
    # the driver's checksum of query 0 (reference src/main.cpp:410-417)
    assert oracle.checksum(gl[0]) == oracle.checksum(sl[0]) == oracle.checksum(pl[0])


# ---- config 2: 1024 x 2^20 uniform rows -------------------------------------------------------

@pytest.fixture(scope="module")
def uniform_matrix(dev):
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(24)
    m = torch.rand((1024, 1 << 20), device=dev, generator=g)
    yield m, {}
    del m
    torch.cuda.empty_cache()


def _tuned(name, rows, k):
    from bitsknn import tuning
    block, _, batch, _, _ = tuning.config_algorithm(name, rows, k)
    return block, batch


# (k, block, values per thread, prefetching variant): the benchmark's headline instantiation, its
# sweep (k x block with 16 / 8 / 4 values per thread), other depths
SWEEP_ITEMS = {128: 16, 256: 8, 512: 4}
CONFIG2 = [(32, 256, 8, False)] + \
          [(k, block, SWEEP_ITEMS[block], False) for k in (16, 32, 128, 512, 2048) for block in (128, 256, 512)
           if k // block <= 16 and (k, block) != (32, 256)] + \
          [(32, 128, 8, False), (32, 512, 8, False), (16, 128, 12, False), (128, 128, 8, True), (2048, 512, 8, False)]


@pytest.mark.parametrize("k,block,batch,prefetch", CONFIG2)
def test_uniform_rows_at_full_size(bk, dev, oracle, uniform_matrix, k, block, batch, prefetch):
    import torch
    m, cache = uniform_matrix
    od, ol = bk.topk_bits(m, k, block, batch, prefetch)
    torch.cuda.synchronize()
    _topk_properties(torch, m, od, ol, k)
    _check_topk_sample(torch, oracle, cache, m, _sample(1024, 16), od, ol, k)


@pytest.mark.parametrize("k", [16, 32, 128, 512, 2048])
@pytest.mark.parametrize("name", ["bits", "bits-prefetch"])
def test_uniform_rows_with_the_tuned_configuration(bk, dev, oracle, uniform_matrix, name, k):
    import torch
    m, cache = uniform_matrix
    block, batch = _tuned(name, 1024, k)
    od, ol = bk.topk_bits(m, k, block, batch, name == "bits-prefetch")
    torch.cuda.synchronize()
    _check_topk_sample(torch, oracle, cache, m, _sample(1024, 16), od, ol, k)


# ---- config 3: 16,384 x 65,536 hard rows ------------------------------------------------------

@pytest.fixture(scope="module")
def hard_matrices(dev):
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(24)
    rows, cols = 16384, 65536
    base = torch.rand((rows, cols), device=dev, generator=g)
    asc = torch.sort(base, dim=1).values
    out = {"ascending": (asc, {}), "descending": (torch.flip(asc, dims=[1]).contiguous(), {}),
           "256-values": (torch.floor(base * 256) / 256, {})}
    del base
    yield out
    out.clear()
    torch.cuda.empty_cache()


@pytest.mark.parametrize("k", [32, 256])
@pytest.mark.parametrize("kind", ["ascending", "descending", "256-values"])
def test_hard_rows_at_full_size(bk, dev, oracle, hard_matrices, kind, k):
    import torch
    m, cache = hard_matrices[kind]
    sample = _sample(m.shape[0], 32)
    tuned = _tuned("bits", m.shape[0], k)
    for block, batch in {(128, 16), (128, 8), tuned}:
        od, ol = bk.topk_bits(m, k, block, batch)
        torch.cuda.synchronize()
        _check_topk_sample(torch, oracle, cache, m, sample, od, ol, k)
    # properties of the whole result (heavy ties included: equal values by ascending label)
    assert bool((od[:, 1:] >= od[:, :-1]).all())
    assert torch.equal(torch.gather(m, 1, ol.long()), od)
    same = od[:, 1:] == od[:, :-1]
    assert bool((ol[:, 1:][same] > ol[:, :-1][same]).all())
    if kind == "ascending":
        # (equal neighbours of a sorted row keep their order; a descending row's do not)
        assert torch.equal(ol, torch.arange(k, dtype=torch.int32, device=dev).expand_as(ol))


# ---- neighbours against the oracle on sampled queries ------------------------------------------

def _check_neighbours(oracle, points_dm, queries_dm, sample, got_d, got_l, k, what, bits=False):
    """points_dm / queries_dm: dim-major device tensors; got_*: the results of the sampled queries.
    bits: the result must equal the oracle's bit for bit."""
    points = np.ascontiguousarray(points_dm.cpu().numpy().T)
    queries = np.ascontiguousarray(queries_dm[:, sample].cpu().numpy().T)
    part = oracle.dist(queries, points, "partial")
    exp_d, exp_l = oracle.topk(part, k)
    if bits:
        assert np.array_equal(got_d.view(np.uint32), exp_d.view(np.uint32)), (what, "values differ from the oracle's")
        assert np.array_equal(got_l, exp_l), (what, "labels differ from the oracle's")
        return
    assert np.all(got_d[:, 1:] >= got_d[:, :-1])
    assert got_l.min() >= 0 and got_l.max() < points.shape[0]
    for row in got_l:
        assert len(set(row.tolist())) == k
    # the reported distances are the distances of the reported points
    at = np.take_along_axis(part, got_l.astype(np.int64), axis=1)
    qn = (queries.astype(np.float64) ** 2).sum(1)[:, None]
    assert np.max(np.abs(got_d - at) / (np.abs(at) + qn)) <= 1e-5
    assert_kth_distance(queries, exp_d[:, -1], got_d[:, -1], points.shape[1], what)
    # recall; a reported point outside the oracle's list counts when its exact distance is within
    # the tolerance of the k-th distance (neighbours closer together than fp32 resolves)
    hits = 0
    for row in range(len(sample)):
        want = set(exp_l[row].tolist())
        for label in got_l[row].tolist():
            if label in want:
                hits += 1
                continue
            p64 = points[label].astype(np.float64)
            exact = float((p64 * p64).sum() - 2.0 * (p64 * queries[row].astype(np.float64)).sum())
            hits += exact <= exp_d[row, -1] + 1e-5 * (abs(exp_d[row, -1]) + qn[row, 0])
    assert hits / (len(sample) * k) >= MIN_RECALL, (what, hits / (len(sample) * k))


# config 5: 1,048,576 points x 65,536 queries (2^36 pairs per launch).  The default arithmetic
# (the reference's, behind the filter) bit for bit against the oracle on the sampled queries; the
# fp32 matrix instructions to the tolerance.
@pytest.mark.parametrize("d,k,mode", [(8, 4, "default"), (16, 16, "default"), (32, 32, "default"),
                                      (8, 32, "default"), (32, 4, "default"), (32, 32, "mfma"), (8, 4, "mfma"),
                                      (64, 32, "default"), (100, 16, "default"), (128, 32, "default"), (192, 16, "default")])
def test_fused_at_full_size(bk, dev, oracle, d, k, mode):
    import torch
    q, n = 65536, 1 << 20
    g = torch.Generator(device=dev)
    g.manual_seed(100 + d)
    points = torch.rand((d, n), device=dev, generator=g)
    queries = torch.rand((d, q), device=dev, generator=g)
    od, ol = bk.fused_l2_topk(queries, points, k, arithmetic=None if mode == "default" else bk.FUSED_FP32)
    bk.fused_status()
    # whole result: ascending, labels in range and distinct per query
    assert bool((od[:, 1:] >= od[:, :-1]).all())
    assert int(ol.min()) >= 0 and int(ol.max()) < n
    sorted_labels = torch.sort(ol, dim=1).values
    assert bool((sorted_labels[:, 1:] != sorted_labels[:, :-1]).all())
    sample = _sample(q, 64)
    _check_neighbours(oracle, points, queries, sample, od[sample].cpu().numpy(), ol[sample].cpu().numpy(), k,
                      ("fused", d, k, mode), bits=mode == "default")


# config 4: 1,048,576 points x 4,096 queries, d = 64 -> a 16 GiB matrix, then bits top-k, k = 64
def test_gemm_distance_and_bits_at_full_size(bk, dev, oracle):
    import torch
    q, n, d, k = 4096, 1 << 20, 64, 64
    g = torch.Generator(device=dev)
    g.manual_seed(64)
    points = torch.rand((d, n), device=dev, generator=g)
    queries = torch.rand((d, q), device=dev, generator=g)
    dist = bk.distances(queries, points, bk.DIST_PARTIAL_L2)
    od, ol = bk.topk_bits(dist, k, 256, 8)
    torch.cuda.synchronize()
    sample = _sample(q, 16)
    got_d, got_l = od[sample].cpu().numpy(), ol[sample].cpu().numpy()
    # the selection is exact on the matrix it was given
    sel_d, sel_l = oracle.topk(dist[sample].cpu().numpy(), k)
    assert np.array_equal(got_d.view(np.uint32), sel_d.view(np.uint32)) and np.array_equal(got_l, sel_l)
    assert torch.equal(torch.gather(dist, 1, ol.long()), od)
    _check_neighbours(oracle, points, queries, sample, got_d, got_l, k, ("gemm + bits", d, k))
    # the bf16x3 arithmetic writes the same matrix to fp32 rounding: same neighbours
    dist2 = bk.distances(queries, points, bk.DIST_PARTIAL_L2_BF16X3, out=dist)
    od, ol = bk.topk_bits(dist2, k, 256, 8)
    torch.cuda.synchronize()
    _check_neighbours(oracle, points, queries, sample, od[sample].cpu().numpy(), ol[sample].cpu().numpy(), k,
                      ("gemm bf16x3 + bits", d, k))
    del dist, dist2
    torch.cuda.empty_cache()
