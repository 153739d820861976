"""CPU tests that pin the oracle (tests/ is the only consumer of oracle/ besides smoke and the
CPU-baseline leg of bench.py)."""
import ctypes

import numpy as np
import pytest

F32P = ctypes.POINTER(ctypes.c_float)


def _p(a):
    return a.ctypes.data_as(F32P)


# ---------------------------------------------------------------------------------------------
# generator / preprocessors / parsers against the reference's own headers (oracle/_ref)
# ---------------------------------------------------------------------------------------------

def test_generator_known_first_values(oracle):
    # first values of the seed-24 stream (d = 1, n = 2^20): points[0], points[1], queries[0]
    p, q = oracle.generate(24, 1 << 20, 4, 1)
    assert p[0, 0] == np.float32(0.773905456)
    assert p[1, 0] == np.float32(0.0291313827)
    assert q[0, 0] == np.float32(0.882071555)


def test_generator_is_minstd_rand0_spec(oracle):
    # the C++ standard fixes the 10000th value of a default-constructed minstd_rand0: 1043618065
    L = oracle.lib()
    state = 1
    state = L.oracle_engine_skip(state, 10000)
    assert state == 1043618065
    # skip-ahead is a homomorphism
    assert L.oracle_engine_skip(L.oracle_engine_skip(7, 123), 877) == L.oracle_engine_skip(7, 1000)
    # init = seed, then discard 4096
    assert L.oracle_engine_init(24) == L.oracle_engine_skip(24, 4096)


@pytest.mark.parametrize("seed,n,q,d,lo,hi", [(24, 5000, 77, 1, 0.0, 1.0), (42, 1024, 32, 8, 0.0, 1.0),
                                              (5, 333, 10, 3, -2.0, 3.5), (1, 100000, 3, 16, 0.0, 1.0)])
def test_uniform_generator_matches_reference_header(oracle, seed, n, q, d, lo, hi):
    R = oracle.ref()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree not mounted)")
    p, s = oracle.generate(seed, n, q, d, "uniform", (lo, hi))
    rp, rs = np.empty_like(p), np.empty_like(s)
    R.ref_uniform_generate(seed, lo, hi, n, q, d, _p(rp), _p(rs))
    assert np.array_equal(p.view(np.uint32), rp.view(np.uint32))
    assert np.array_equal(s.view(np.uint32), rs.view(np.uint32))


@pytest.mark.parametrize("seed,mean,std", [(7, 0.0, 1.0), (24, 0.5, 2.0)])
def test_normal_generator_matches_reference_header(oracle, seed, mean, std):
    R = oracle.ref()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree not mounted)")
    p, s = oracle.generate(seed, 4097, 33, 3, "normal", (mean, std))
    rp, rs = np.empty_like(p), np.empty_like(s)
    R.ref_normal_generate(seed, mean, std, 4097, 33, 3, _p(rp), _p(rs))
    assert np.array_equal(p.view(np.uint32), rp.view(np.uint32))
    assert np.array_equal(s.view(np.uint32), rs.view(np.uint32))


def test_large_fill_equals_serial_fill(oracle):
    # the OpenMP skip-ahead path (> 2^20 values) must equal the one-by-one path
    L = oracle.lib()
    n = (1 << 21) + 12345
    big = np.empty(n, dtype=np.float32)
    st = L.oracle_engine_init(24)
    end_big = L.oracle_uniform_fill(st, 0.0, 1.0, _p(big), n)
    small = np.empty(n, dtype=np.float32)
    s = st
    step = 1 << 19
    for off in range(0, n, step):
        cnt = min(step, n - off)
        s = L.oracle_uniform_fill(s, 0.0, 1.0, _p(small[off:off + cnt]), cnt)
    assert s == end_big
    assert np.array_equal(big, small)


@pytest.mark.parametrize("descending", [0, 1])
def test_ordering_preprocessor_matches_reference_header(oracle, descending):
    R = oracle.ref()
    if R is None:
        pytest.skip("oracle/_ref not built (reference tree not mounted)")
    p, s = oracle.generate(24, 3000, 17, 4)
    p2, s2 = p.copy(), s.copy()
    oracle.lib().oracle_preprocess_ordering(_p(p), p.size, _p(s), s.size, descending)
    R.ref_preprocess_ordering(_p(p2), p2.size, _p(s2), s2.size, 4, descending)
    assert np.array_equal(p, p2) and np.array_equal(s, s2)
    assert not s.any()
    flat = p.ravel()
    assert np.all(flat[:-1] >= flat[1:]) if descending else np.all(flat[:-1] <= flat[1:])


@pytest.mark.parametrize("text", ["0", "1", "17", "1k", "3K", "2m", "5M", "1g", "2G", "", "12x", "k", "007"])
def test_parse_number_matches_reference_header(oracle, text):
    expected = {"1k": 1024, "3K": 3072, "2m": 2 << 20, "1g": 1 << 30, "17": 17, "": 0}
    if text in expected:
        assert oracle.parse_number(text) == expected[text]
    R = oracle.ref()
    if R is not None:
        assert oracle.parse_number(text) == R.ref_parse_number(text.encode())


@pytest.mark.parametrize("text", ["1", "8,4,2", "16,1", "1k,2,3,4", ",,", "4,,2"])
def test_parse_dim3_matches_reference_header(oracle, text):
    R = oracle.ref()
    if R is None:
        pytest.skip("oracle/_ref not built")
    out = (ctypes.c_uint64 * 3)()
    R.ref_parse_dim3(text.encode(), out)
    assert oracle.parse_dim3(text) == tuple(out)


# ---------------------------------------------------------------------------------------------
# distances
# ---------------------------------------------------------------------------------------------

def test_dist_l2_against_fp64_and_d1_closed_form(oracle):
    p, q = oracle.generate(42, 700, 9, 10)
    d32 = oracle.dist(q, p, "l2")
    d64 = oracle.dist(q, p, "f64")
    assert np.allclose(d32, d64, rtol=2e-6, atol=0)
    # d = 1: exactly fl((q-p)^2) with the subtraction rounded first
    p1, q1 = oracle.generate(24, 1000, 5, 1)
    d1 = oracle.dist(q1, p1, "l2")
    diff = (q1[:, None, 0] - p1[None, :, 0]).astype(np.float32)
    assert np.array_equal(d1, (diff * diff).astype(np.float32))
    # asymmetry check: swapping the operands transposes the matrix (catches swapped q/p indexing)
    assert np.array_equal(oracle.dist(p[:50], q, "l2"), oracle.dist(q, p[:50], "l2").T)


def test_dist_partial_l2_identity(oracle):
    p, q = oracle.generate(42, 500, 7, 17)
    part = oracle.dist(q, p, "partial").astype(np.float64)
    full = oracle.dist(q, p, "f64")
    qn = (q.astype(np.float64) ** 2).sum(axis=1)[:, None]
    assert np.allclose(part + qn, full, rtol=0, atol=2e-5)
    assert np.allclose(part, oracle.dist(q, p, "f64-partial"), rtol=0, atol=2e-5)
    # not symmetric: it contains ||p||^2 but not ||q||^2
    z = np.zeros((1, 17), dtype=np.float32)
    assert np.allclose(oracle.dist(z, p, "partial")[0], (p.astype(np.float64) ** 2).sum(axis=1), rtol=1e-6)


# ---------------------------------------------------------------------------------------------
# top-k
# ---------------------------------------------------------------------------------------------

def _brute(matrix, k, labels=None):
    rows, cols = matrix.shape
    out_d = np.full((rows, k), np.inf, dtype=np.float32)
    out_l = np.full((rows, k), np.iinfo(np.int32).max, dtype=np.int32)
    for r in range(rows):
        lab = labels[r] if labels is not None else np.arange(cols, dtype=np.int32)
        order = np.lexsort((lab, matrix[r]))[:k]
        out_d[r, :len(order)] = matrix[r, order]
        out_l[r, :len(order)] = lab[order]
    return out_d, out_l


@pytest.mark.parametrize("rows,cols,k", [(5, 100, 7), (3, 64, 64), (4, 1000, 16), (2, 10, 16), (1, 1, 1)])
def test_topk_vs_brute_force_with_ties(oracle, rows, cols, k):
    rng = np.random.default_rng(rows * 1000 + cols)
    m = (rng.integers(0, 13, size=(rows, cols)) / 8.0).astype(np.float32)  # heavy ties
    d, l = oracle.topk(m, k)
    bd, bl = _brute(m, k)
    assert np.array_equal(d, bd) and np.array_equal(l, bl)


def test_topk_labels_and_offsets(oracle):
    rng = np.random.default_rng(3)
    m = (rng.integers(0, 5, size=(4, 200)) / 4.0).astype(np.float32)
    labels = rng.permutation(800).astype(np.int32).reshape(4, 200)
    d, l = oracle.topk(m, 9, labels=labels)
    bd, bl = _brute(m, 9, labels)
    assert np.array_equal(d, bd) and np.array_equal(l, bl)
    offs = np.array([0, 200, 400, 600], dtype=np.int32)
    d2, l2 = oracle.topk(m, 9, label_offsets=offs)
    bd2, bl2 = _brute(m, 9)
    assert np.array_equal(d2, bd2) and np.array_equal(l2, bl2 + offs[:, None])


def test_serial_and_parallel_restatements_agree_on_tie_free_input(oracle):
    m = oracle.uniform_matrix(7, 16, 4096)
    d, l = oracle.topk(m, 32)
    sd, sl = oracle.topk_serial(m, 32)
    pd, pl, used = oracle.topk_parallel(m, 32, 2)
    assert used == 2
    assert np.array_equal(d, sd) and np.array_equal(d, pd)
    # rows of distinct values: labels must agree as well
    distinct = np.array([len(np.unique(m[r])) == m.shape[1] for r in range(m.shape[0])])
    assert distinct.any()
    assert np.array_equal(l[distinct], sl[distinct]) and np.array_equal(l[distinct], pl[distinct])


def test_checksum_and_closed_forms(oracle):
    # ascending preprocessor, d = 1: every query is 0 and the points are sorted, so the k nearest
    # are columns 0..k-1 -> k(k-1)/2; descending -> the last k columns
    for k in (32, 256, 2048):
        n = 4096
        p, q = oracle.generate(24, n, 2, 1, preprocessor="ascending")
        dist = oracle.dist(q, p, "l2")
        _, l = oracle.topk(dist, k)
        assert oracle.checksum(l[0]) == k * (k - 1) // 2
        p, q = oracle.generate(24, n, 2, 1, preprocessor="descending")
        dist = oracle.dist(q, p, "l2")
        _, l = oracle.topk(dist, k)
        assert oracle.checksum(l[0]) == sum(range(n - k, n)) % (1 << 32)
    assert oracle.checksum(np.array([2**31 - 1, 2**31 - 1, 5], dtype=np.int32)) == (2**32 - 2 + 5) % 2**32


# ---------------------------------------------------------------------------------------------
# golden checksums held by the reference (data/*.err), query 0 only
# ---------------------------------------------------------------------------------------------

def _golden_cases(records, family, max_pairs):
    for rec in records:
        if rec["family"] != family or rec["preprocessor"] != "identity":
            continue
        if rec["n"] * rec["d"] > max_pairs:
            continue
        yield rec


def test_golden_kselection_checksums(oracle, golden):
    checked = 0
    cache = {}
    for rec in _golden_cases(golden, "kselection", 1 << 22):
        key = (rec["n"], rec["q"])
        if key not in cache:
            p, q = oracle.generate(24, rec["n"], rec["q"], 1)
            cache[key] = oracle.dist(q[:1], p, "l2")
        _, l = oracle.topk(cache[key], rec["k"])
        got = str(oracle.checksum(l[0]))
        # on rows where the reference itself printed several values (a tie at the k-th place),
        # the canonical (value, index) order must produce one of them
        assert got in rec["checksums"], (rec["n"], rec["q"], rec["k"], got, rec["checksums"])
        checked += 1
    assert checked >= 21


def test_golden_fused_checksums(oracle, golden):
    checked = 0
    cache = {}
    for rec in _golden_cases(golden, "fused", 1 << 24):
        key = (rec["n"], rec["q"], rec["d"])
        if key not in cache:
            p, q = oracle.generate(24, rec["n"], rec["q"], rec["d"])
            cache[key] = (oracle.dist(q[:1], p, "l2"), oracle.dist(q[:1], p, "partial"))
        for kind in (0, 1):
            _, l = oracle.topk(cache[key][kind], rec["k"])
            assert str(oracle.checksum(l[0])) in rec["checksums"], (rec, kind)
        checked += 1
    assert checked >= 72


def test_golden_buffer_closed_forms(golden):
    for rec in golden:
        if rec["family"] != "buffer" or rec["preprocessor"] == "identity":
            continue
        n, k = rec["n"], rec["k"]
        expect = k * (k - 1) // 2 if rec["preprocessor"] == "ascending" else sum(range(n - k, n)) % (1 << 32)
        assert list(rec["checksums"]) == [str(expect)]


# ---------------------------------------------------------------------------------------------
# verify() restatement: hand cases
# ---------------------------------------------------------------------------------------------

def test_verify_restatement(oracle):
    d = np.array([[0.1, 0.2, 0.3, 0.3]], dtype=np.float32)
    l = np.array([[5, 6, 7, 9]], dtype=np.int32)
    assert oracle.verify(d, l, d, l, 4) == (True, 0)
    # a different member of a tie group that runs to the end of the row is tolerated
    l_tie = np.array([[5, 6, 7, 11]], dtype=np.int32)
    assert oracle.verify(d, l, d, l_tie, 4)[0]
    # permutation inside a tie group is normalised away
    l_perm = np.array([[5, 6, 9, 7]], dtype=np.int32)
    assert oracle.verify(d, l, d, l_perm, 4) == (True, 0)
    # a real mismatch is reported
    l_bad = np.array([[5, 8, 7, 9]], dtype=np.int32)
    ok, bad = oracle.verify(d, l, d, l_bad, 4)
    assert not ok and bad == 1
