"""Parity of the bits top-k HIP kernel (through the C ABI) with the CPU oracle.

Bar: bit-exact values and labels, equal values ordered by lower label.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(bk, dev, matrix, k, block=256, batch=16, prefetch=False, labels=None, offsets=None):
    import torch
    d = torch.from_numpy(matrix).to(dev)
    lab = torch.from_numpy(labels).to(dev) if labels is not None else None
    off = torch.from_numpy(offsets).to(dev) if offsets is not None else None
    od, ol = bk.topk_bits(d, k, block, batch, prefetch, in_label=lab, label_offsets=off)
    torch.cuda.synchronize()
    return od.cpu().numpy(), ol.cpu().numpy()


def _check(bk, dev, oracle, matrix, k, **kw):
    gd, gl = _run(bk, dev, matrix, k, **kw)
    ed, el = oracle.topk(matrix, k, labels=kw.get("labels"), label_offsets=kw.get("offsets"))
    assert np.array_equal(gd.view(np.uint32), ed.view(np.uint32)), "values differ"
    assert np.array_equal(gl, el), "labels differ"


# the reference's own unit-test shapes (tests/topk/bits_knn_test.cpp:7-63): seed 42, d = 10
@pytest.mark.parametrize("n,k", [(128, 128), (1024, 256)])
@pytest.mark.parametrize("batch", [1, 7, 16])
def test_reference_unit_test_shapes(bk, dev, oracle, n, k, batch):
    p, q = oracle.generate(42, n, 1, 10)
    dist = oracle.dist(q, p, "l2")
    _check(bk, dev, oracle, dist, k, block=128, batch=batch)


@pytest.mark.parametrize("block", [128, 256, 512])
@pytest.mark.parametrize("k", [1, 16, 32, 64, 100, 128, 256, 512, 1024, 2048])
def test_uniform_rows_all_k_and_blocks(bk, dev, oracle, block, k):
    m = oracle.uniform_matrix(1000 + k + block, 6, 40000)
    _check(bk, dev, oracle, m, k, block=block, batch=8)


@pytest.mark.parametrize("batch,prefetch", [(1, False), (4, False), (5, False), (9, False), (12, False),
                                            (16, False), (1, True), (8, True), (12, True), (16, True)])
def test_batch_sizes_and_prefetch(bk, dev, oracle, batch, prefetch):
    m = oracle.uniform_matrix(77 + batch, 5, 70001)
    _check(bk, dev, oracle, m, 128, block=256, batch=batch, prefetch=prefetch)
    _check(bk, dev, oracle, m, 2048, block=256, batch=batch, prefetch=prefetch)


@pytest.mark.parametrize("cols", [1, 2, 15, 16, 17, 127, 128, 129, 255, 256, 257, 511, 513, 1000, 4095,
                                  4096, 4097, 12289, 16385])
def test_ragged_row_lengths(bk, dev, oracle, cols):
    m = oracle.uniform_matrix(cols, 3, cols)
    for k in (1, 16, 32, 300):
        _check(bk, dev, oracle, m, k, block=128, batch=7)
        _check(bk, dev, oracle, m, k, block=512, batch=16)


def test_rows_not_16_byte_aligned(bk, dev, oracle):
    import torch
    # a row stride that is not a multiple of 4 floats, and a base offset of one float
    big = oracle.uniform_matrix(5, 9, 30011)
    t = torch.from_numpy(big).to(dev)
    for view, ref in ((t[:, 1:20000], big[:, 1:20000]), (t[:, 3:30011], big[:, 3:30011]), (t[:, :30008], big[:, :30008])):
        od, ol = bk.topk_bits(view, 64, 256, 16)
        torch.cuda.synchronize()
        ed, el = oracle.topk(ref, 64)
        assert np.array_equal(od.cpu().numpy(), ed) and np.array_equal(ol.cpu().numpy(), el)


@pytest.mark.parametrize("kind", ["ascending", "descending", "256-values", "constant", "two-values"])
@pytest.mark.parametrize("k", [32, 256, 2048])
def test_hard_inputs(bk, dev, oracle, kind, k):
    rows, cols = 4, 65536
    base = oracle.uniform_matrix(99, rows, cols)
    if kind == "ascending":
        m = np.sort(base, axis=1)
    elif kind == "descending":
        m = np.sort(base, axis=1)[:, ::-1].copy()
    elif kind == "256-values":
        m = (np.floor(base * 256) / 256).astype(np.float32)
    elif kind == "constant":
        m = np.full((rows, cols), 0.25, dtype=np.float32)
    else:
        m = (base > 0.5).astype(np.float32)
    for block in (128, 256, 512):
        if k // block > 16:
            continue
        _check(bk, dev, oracle, m, k, block=block, batch=16)


def test_rows_long_enough_for_the_sampled_radius(bk, dev, oracle):
    """Rows of at least 128 x block size values start from a radius that the kernel takes from a
    sample of both ends of the row; the result must not depend on it."""
    rng = np.random.default_rng(5)
    rows, cols = 8, 70000
    m = oracle.uniform_matrix(321, rows, cols, -3.0, 3.0)
    m[0, :3000] = np.inf                      # nothing finite in the sampled parts
    m[0, -3000:] = np.inf
    m[1, :] = np.inf                          # fewer finite values than k, none of them sampled
    m[1, 30000:30040] = rng.random(40, dtype=np.float32)
    m[2, :4096] = -7.0                        # more equal values than k inside the sample
    m[3, 20000:20300] = -7.0                  # the smallest values tie and lie outside the sample
    m[4] = np.round(m[4] * 8) / 8             # few distinct values
    m[5, :2048] = np.sort(m[5, :2048])        # sampled parts sorted towards the middle
    m[5, -2048:] = np.sort(m[5, -2048:])[::-1]
    m[6, 1::2] = -0.0                         # both zeros, everywhere
    m[6, 0::2] = 0.0
    m[7] = (rng.permutation(cols).astype(np.uint32) + 1).view(np.float32)  # subnormal values only
    for block in (128, 256, 512):
        for k in (1, 5, 100, 127, 128, 129, 256, 257, 512, 1024):
            if k // block > 16:
                continue
            gd, gl = _run(bk, dev, m, k, block=block, batch=8)
            ed, el = oracle.topk(m, k)
            assert np.array_equal(gd, ed) and np.array_equal(gl, el), (block, k)
    # rows that do not start on a 16-byte boundary take 4-byte loads, the sample included
    import torch
    t = torch.from_numpy(m).to(dev)
    for view, ref in ((t[:, 1:], m[:, 1:]), (t[:, 2:69999], m[:, 2:69999])):
        for block, k in ((128, 100), (256, 256), (512, 2048)):
            od, ol = bk.topk_bits(view, k, block, 8)
            torch.cuda.synchronize()
            ed, el = oracle.topk(np.ascontiguousarray(ref), k)
            assert np.array_equal(od.cpu().numpy(), ed) and np.array_equal(ol.cpu().numpy(), el), (block, k)
    # explicit labels with the extreme values on tied entries, and label offsets
    labels = np.stack([rng.permutation(cols) for _ in range(rows)]).astype(np.int32)
    labels[4, :4] = [np.iinfo(np.int32).max, np.iinfo(np.int32).min, -1, 0]
    offsets = (np.arange(rows) * 1000003).astype(np.int32)
    short, short_labels = np.ascontiguousarray(m[:, :66000]), np.ascontiguousarray(labels[:, :66000])
    for matrix, k, block, batch, lab, off in ((short, 300, 128, 8, short_labels, None),
                                              (m, 64, 256, 4, None, offsets),
                                              (m, 512, 512, 3, labels, offsets)):
        gd, gl = _run(bk, dev, matrix, k, block=block, batch=batch, labels=lab, offsets=off)
        ed, el = oracle.topk(matrix, k, labels=lab, label_offsets=off)
        assert np.array_equal(gd, ed) and np.array_equal(gl, el), (k, block)


def _estimate_sample_columns(cols, block):
    """Columns of the evenly spread sample that long lists estimate their first radius from (rows
    of at least 256 x block size values)."""
    pieces = min(4096 // block, cols // (256 * block))
    segment = (cols // pieces) & ~3
    offset = (segment // 2 - 2 * block) & ~3
    return np.concatenate([np.arange(p * segment + offset, p * segment + offset + 4 * block)
                           for p in range(pieces)])


@pytest.mark.parametrize("block,k,batch", [(128, 1024, 8), (128, 2048, 16), (256, 600, 8), (256, 2048, 8),
                                           (256, 2048, 12), (512, 513, 4), (512, 1024, 8), (512, 2047, 8),
                                           (512, 2048, 16), (128, 200, 16), (128, 256, 8), (128, 500, 16),
                                           (256, 300, 8), (256, 512, 16)])
def test_rows_long_enough_for_the_estimated_radius(bk, dev, oracle, block, k, batch):
    """Long lists (two and more entries per thread from 256 entries on, all from 1024 on) on long
    rows start from an estimate of the k-th smallest value and repeat the row when the estimate
    proves too low; the result must not depend on either.  Rows where the estimate holds, rows where it cannot hold (the sampled columns hold
    the only small values, fewer than k of them), ties at the estimate, sorted rows, rows with
    few finite values."""
    rng = np.random.default_rng(block + k)
    rows, cols = 12, 1 << 18
    sample = _estimate_sample_columns(cols, block)
    m = oracle.uniform_matrix(77 + k, rows, cols, -2.0, 2.0)
    m[1] = np.sort(m[1])
    m[2] = np.sort(m[2])[::-1]
    m[3] = 5.0 + rng.random(cols, dtype=np.float32)          # small values only where the sample looks:
    m[3, sample] = rng.random(sample.size, dtype=np.float32)  # more than k of them
    m[4] = 5.0 + rng.random(cols, dtype=np.float32)
    few = rng.choice(sample, size=k // 2, replace=False)      # fewer than k of them
    m[4, few] = rng.random(few.size, dtype=np.float32)
    m[5] = 5.0                                                # ties above the few small values
    m[5, few] = rng.random(few.size, dtype=np.float32)
    m[6] = np.round(m[6] * 4) / 4                             # 17 distinct values
    m[7] = np.inf                                             # fewer finite values than k, all sampled
    m[7, few[:100]] = rng.random(100, dtype=np.float32)
    m[8] = np.inf                                             # nothing finite in the sample
    rest = np.setdiff1d(np.arange(cols), sample)
    m[8, rest[::3]] = rng.random(rest[::3].size, dtype=np.float32)
    m[9, sample] = np.nan                                     # a sample of NaNs
    m[10, sample] = -3.0                                      # the sample is one value, below the rest
    m[11] = m[11, 0]                                          # constant row
    want = np.where(np.isnan(m), np.float32(np.inf), m)       # a NaN counts as +inf
    gd, gl = _run(bk, dev, m, k, block=block, batch=batch)
    ed, el = oracle.topk(want, k)
    assert np.array_equal(gd, ed) and np.array_equal(gl, el)
    # rows that do not start on a 16-byte boundary (4-byte loads, the sample too), explicit labels
    import torch
    t = torch.from_numpy(m).to(dev)
    od, ol = bk.topk_bits(t[:, 3:], k, block, batch)
    torch.cuda.synchronize()
    ed, el = oracle.topk(np.ascontiguousarray(want[:, 3:]), k)
    assert np.array_equal(od.cpu().numpy(), ed) and np.array_equal(ol.cpu().numpy(), el)
    labels = np.stack([rng.permutation(cols) for _ in range(rows)]).astype(np.int32)
    offsets = (np.arange(rows) * 7919).astype(np.int32)
    gd, gl = _run(bk, dev, m, k, block=block, batch=batch, labels=labels, offsets=offsets)
    ed, el = oracle.topk(want, k, labels=labels, label_offsets=offsets)
    assert np.array_equal(gd, ed) and np.array_equal(gl, el)


def test_negative_values_and_infinities(bk, dev, oracle):
    m = oracle.uniform_matrix(3, 4, 20000, -5.0, 5.0)
    m[0, 17] = -np.inf
    m[1, 5] = np.inf
    m[2, :] = np.inf
    m[2, 100] = 1.0
    _check(bk, dev, oracle, m, 64, block=256, batch=16)
    _check(bk, dev, oracle, m, 1024, block=128, batch=3)


def test_negative_zero_is_returned_as_positive_zero(bk, dev, oracle):
    # documented deviation: -0.0 ties with +0.0 (as for the oracle) but is written back as +0.0
    m = oracle.uniform_matrix(4, 1, 5000, 1.0, 2.0)
    m[0, 10] = -0.0
    m[0, 4000] = 0.0
    gd, gl = _run(bk, dev, m, 16)
    assert list(gl[0, :2]) == [10, 4000]
    assert gd[0, 0] == 0.0 and gd[0, 1] == 0.0 and not np.signbit(gd[0, 0])


def test_nans_count_as_plus_infinity(bk, dev, oracle):
    """A NaN of either sign is treated as +inf everywhere (first values of a row, streamed part,
    sampled row ends) and is written back as +inf: the result equals the oracle's on the matrix
    with every NaN replaced by +inf, ties by lower label included."""
    pos_nan = np.array([0x7FC00000], dtype=np.uint32).view(np.float32)[0]
    neg_nan = np.array([0xFFC00000], dtype=np.uint32).view(np.float32)[0]   # what 0/0 gives on x86
    sig_nan = np.array([0x7F800001], dtype=np.uint32).view(np.float32)[0]
    rng = np.random.default_rng(8)
    for cols in (3000, 70000):                      # without and with a sampled first radius
        m = oracle.uniform_matrix(900 + cols, 6, cols, -2.0, 2.0)
        m[0, :40:3] = neg_nan                       # among the first values of the row
        m[0, 5] = pos_nan
        m[1, cols // 2:cols // 2 + 50:2] = neg_nan  # in the streamed part
        m[1, cols - 7:] = pos_nan                   # at the very end (sampled when the row is long)
        m[2, rng.permutation(cols)[:cols // 3]] = neg_nan   # a third of the row
        m[2, rng.permutation(cols)[:cols // 5]] = sig_nan
        m[3, :] = neg_nan                           # nothing but NaNs ...
        m[3, 100:110] = np.arange(10, dtype=np.float32)     # ... and ten numbers
        m[4, :] = pos_nan                           # NaNs, infinities and five numbers: fewer than k
        m[4, 1::2] = np.inf
        m[4, [7, 77, 777, 1777, 2777]] = [3.0, -1.0, 2.0, 0.0, 1.0]
        m[5, :] = neg_nan                           # nothing at all
        want = np.where(np.isnan(m), np.float32(np.inf), m)
        for block, batch in ((128, 3), (256, 8), (512, 16)):
            for k in (1, 16, 40, 256, 1024):
                gd, gl = _run(bk, dev, m, k, block=block, batch=batch)
                ed, el = oracle.topk(want, k)
                assert not np.isnan(gd).any()
                assert np.array_equal(gd, ed) and np.array_equal(gl, el), (cols, block, batch, k)
    # the unfiltered baseline builds the same keys
    import torch
    gd, gl = bk.topk_partial_bitonic(torch.from_numpy(m).to(dev), 64, 256)
    torch.cuda.synchronize()
    ed, el = oracle.topk(want, 64)
    assert np.array_equal(gd.cpu().numpy(), ed) and np.array_equal(gl.cpu().numpy(), el)


def test_k_larger_than_row(bk, dev, oracle):
    m = oracle.uniform_matrix(8, 3, 20)
    _check(bk, dev, oracle, m, 32, block=128, batch=1)


def test_explicit_labels_and_offsets(bk, dev, oracle):
    rng = np.random.default_rng(1)
    m = (np.floor(oracle.uniform_matrix(12, 6, 9000) * 64) / 64).astype(np.float32)
    labels = np.stack([rng.permutation(9000) for _ in range(6)]).astype(np.int32)
    offsets = (np.arange(6) * 9000).astype(np.int32)
    _check(bk, dev, oracle, m, 200, block=256, batch=16, labels=labels)
    _check(bk, dev, oracle, m, 200, block=256, batch=16, offsets=offsets)
    _check(bk, dev, oracle, m, 200, block=128, batch=5, labels=labels, offsets=offsets)


def test_row_split_like_bits_sq(bk, dev, oracle):
    """One long row split into parts, then merged with explicit labels
    (reference src/topk/singlepass/bits_knn.cu:132-186)."""
    import torch
    n, deg, k = 1 << 18, 8, 64
    row = oracle.uniform_matrix(21, 1, n)
    t = torch.from_numpy(row).to(dev)
    cols = n // deg
    offs = bk.label_offsets(1, deg, cols, dev)
    assert offs.cpu().tolist() == [i * cols for i in range(deg)]
    pd, pl = bk.topk_bits(t.view(deg, cols), k, 256, 16, True, label_offsets=offs)
    fd, fl = bk.topk_bits(pd.view(1, deg * k), k, 256, 16, True, in_label=pl.view(1, deg * k))
    torch.cuda.synchronize()
    ed, el = oracle.topk(row, k)
    assert np.array_equal(fd.cpu().numpy(), ed) and np.array_equal(fl.cpu().numpy(), el)


@pytest.mark.parametrize("rows,n,parts,k,block,batch", [
    (1, 1 << 18, 8, 64, 256, 16), (3, 1 << 16, 16, 32, 128, 4), (64, 1 << 15, 4, 16, 128, 8),
    (5, 40960, 5, 100, 256, 8), (7, 30000, 3, 7, 512, 4), (2, 1 << 17, 32, 256, 512, 12),
    (4, 1 << 16, 2, 2048, 512, 4), (9, 9 * 1001, 7, 33, 256, 16), (130, 4096, 2, 4, 128, 16),
    (2, 1 << 19, 32, 2, 128, 4), (300, 1 << 14, 4, 8, 128, 8), (512, 8192, 2, 16, 256, 4)])
def test_rows_cut_into_parts_in_one_launch(bk, dev, oracle, rows, n, parts, k, block, batch):
    """bitsknn_topk_bits_parts_f32 (bits-sq: reference src/topk/singlepass/bits_knn.cu:132-186) against
    the oracle's top-k of the whole rows, bit for bit, three calls in a row on the same scratch
    memory (the counters must come back to zero).  Shapes with 16-byte loads and one launch, with
    parts * k not a multiple of four or more than 1024 parts in all (second pass as its own launch)
    and with parts that are not a multiple of four values (4-byte loads)."""
    import torch
    m = oracle.uniform_matrix(rows + parts + k, rows, n)
    m[:, ::97] = m[:, 5:6]     # ties across the parts
    t = torch.from_numpy(m).to(dev)
    ed, el = oracle.topk(m, k)
    scratch = {}
    for call in range(3):
        od, ol = bk.topk_bits_parts(t, k, parts, block, batch, scratch=scratch)
        torch.cuda.synchronize()
        assert np.array_equal(od.cpu().numpy().view(np.uint32), ed.view(np.uint32)), call
        assert np.array_equal(ol.cpu().numpy(), el), call
    (_, _, counters), = scratch.values()
    assert int(counters.abs().sum()) == 0


def test_rows_cut_into_parts_validation(bk, dev):
    import torch
    t = torch.zeros((2, 1000), device=dev)
    with pytest.raises(bk.BitsKnnError, match="multiple of the parts"):
        bk.topk_bits_parts(t, 4, 3)
    with pytest.raises(bk.BitsKnnError, match="Unsupported block size: 64"):
        bk.topk_bits_parts(t, 4, 2, 64)
    with pytest.raises(bk.BitsKnnError, match="Unsupported k value: 4096"):
        bk.topk_bits_parts(t, 4096, 2)


def test_strided_output(bk, dev, oracle):
    import torch
    m = oracle.uniform_matrix(31, 5, 10000)
    od = torch.full((5, 100), -1.0, device=dev)
    ol = torch.full((5, 100), -1, dtype=torch.int32, device=dev)
    bk.topk_bits(torch.from_numpy(m).to(dev), 40, 256, 16, out_dist=od, out_label=ol)
    torch.cuda.synchronize()
    ed, el = oracle.topk(m, 40)
    assert np.array_equal(od[:, :40].cpu().numpy(), ed) and np.array_equal(ol[:, :40].cpu().numpy(), el)
    assert (od[:, 40:] == -1).all() and (ol[:, 40:] == -1).all()


def test_fill_and_errors_on_device(bk, dev):
    import torch
    t = torch.zeros(100003, device=dev)
    bk.fill(t, 2.5)
    torch.cuda.synchronize()
    assert (t == 2.5).all()
    with pytest.raises(bk.BitsKnnError, match="Unsupported block size: 64"):
        bk.topk_bits(torch.zeros((2, 100), device=dev), 16, 64, 1)


# reference-held checksums of query 0 (data/kselection-*.err), distances by the oracle
@pytest.mark.parametrize("n,q", [(1 << 20, 1024), (1 << 18, 4096)])
def test_golden_kselection_checksums(bk, dev, oracle, golden, n, q):
    p, qq = oracle.generate(24, n, q, 1)
    dist = oracle.dist(qq[:4], p, "l2")
    checked = 0
    for rec in golden:
        if rec["family"] != "kselection" or rec["n"] != n or rec["q"] != q:
            continue
        for block in (128, 256, 512):
            if rec["k"] // block > 16:
                continue
            gd, gl = _run(bk, dev, dist, rec["k"], block=block, batch=16)
            assert str(oracle.checksum(gl[0])) in rec["checksums"], (rec, block)
            ed, el = oracle.topk(dist, rec["k"])
            assert np.array_equal(gd, ed) and np.array_equal(gl, el)
            checked += 1
    assert checked >= 7


def test_full_size_properties(bk, dev):
    """1024 x 2^20 uniform rows (4 GiB): size-independent properties against torch.topk values."""
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(24)
    rows, cols = 1024, 1 << 20
    m = torch.rand((rows, cols), device=dev, generator=g)
    for k, block in ((32, 256), (512, 512), (2048, 256)):
        od, ol = bk.topk_bits(m, k, block, 16, True)
        torch.cuda.synchronize()
        # ascending
        assert bool((od[:, 1:] >= od[:, :-1]).all())
        # every value is the matrix entry its label points to
        assert torch.equal(torch.gather(m, 1, ol.long()), od)
        # equal values come out by ascending label, labels are distinct
        same = od[:, 1:] == od[:, :-1]
        assert bool((ol[:, 1:][same] > ol[:, :-1][same]).all())
        assert bool((torch.sort(ol, dim=1).values[:, 1:] != torch.sort(ol, dim=1).values[:, :-1]).all())
        # the k smallest: bit-equal to torch's sorted top-k values on a sample of rows
        sample = torch.arange(0, rows, 37, device=dev)
        tv = torch.topk(m[sample], k, dim=1, largest=False, sorted=True).values
        assert torch.equal(tv, od[sample])
        # nothing smaller was left behind
        kth = od[:, -1:]
        assert bool(((m < kth).sum(dim=1) <= k - 1).all())
    del m
    torch.cuda.empty_cache()


def test_random_shapes_against_the_oracle(bk, dev, oracle):
    """150 random problems: ragged lengths around every chunk boundary, all block and batch sizes,
    uniform / heavily tied / sorted rows, with and without the prefetching variant."""
    rng = np.random.default_rng(2024)
    for case in range(150):
        block = int(rng.choice([128, 256, 512]))
        batch = int(rng.integers(1, 17))
        k = int(rng.choice([1, 7, 16, 32, 100, 256, 512, 1000, 2048]))
        if k // block > 16:
            k = block * 16
        rows = int(rng.integers(1, 5))
        kind = case % 5
        cols = int(rng.integers(1, 150000)) if kind else int(block * 4 * ((batch + 3) // 4) * rng.integers(1, 9) + rng.integers(-2, 3) + max(k, block))
        cols = max(cols, 1)
        m = oracle.uniform_matrix(5000 + case, rows, cols)
        if kind == 1:
            m = (np.floor(m * 8) / 8).astype(np.float32)
        elif kind == 2:
            m = np.sort(m, axis=1)
        elif kind == 3:
            m = np.ascontiguousarray(np.sort(m, axis=1)[:, ::-1])
        gd, gl = _run(bk, dev, m, k, block=block, batch=batch, prefetch=bool(case & 1))
        ed, el = oracle.topk(m, k)
        assert np.array_equal(gd.view(np.uint32), ed.view(np.uint32)), (case, block, batch, k, rows, cols, kind)
        assert np.array_equal(gl, el), (case, block, batch, k, rows, cols, kind)
