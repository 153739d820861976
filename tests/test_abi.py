"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol, and rejects
unsupported parameters with the reference's messages before touching the GPU."""
import ctypes
import json
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "bitsknn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bitsknn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(bk):
    L = bk.lib()
    declared = _declared_symbols()
    assert len(declared) >= 7
    assert set(declared) == set(bk.EXPORTS)
    for name in declared:
        assert getattr(L, name) is not None


def test_version_and_error_string(bk):
    assert bk.version().startswith("bitsknn")
    assert isinstance(bk.lib().bitsknn_last_error(), bytes)


def _topk_status(bk, k, block, batch):
    # parameter validation happens before any pointer is looked at or any HIP call is made
    L = bk.lib()
    st = L.bitsknn_topk_bits_f32(None, 0, None, 0, None, 0, 0, None, None, 0, k, block, batch, 0, None)
    return st, L.bitsknn_last_error().decode()


# messages of the reference dispatch (src/topk/singlepass/bits_knn.cu:52-62)
@pytest.mark.parametrize("k,block,batch,msg", [
    (32, 100, 1, "Unsupported block size: 100"),
    (32, 1024, 1, "Unsupported block size: 1024"),
    (32, 256, 0, "Unsupported batch size: 0"),
    (32, 256, 17, "Unsupported batch size: 17"),
    (0, 256, 1, "Unsupported k value: 0"),
    (2049, 256, 1, "Unsupported k value: 2049"),
    (4096, 128, 16, "Unsupported k value: 4096"),
])
def test_topk_rejects_unsupported_parameters(bk, k, block, batch, msg):
    st, text = _topk_status(bk, k, block, batch)
    assert st == bk.ERR_UNSUPPORTED
    assert text == msg


def _fused_ex_status(bk, k, arithmetic, params=(8, 4, 2)):
    # validation only: q = 0 returns before any pointer is looked at or any HIP call is made
    L = bk.lib()
    st = L.bitsknn_fused_l2_topk_f32_ex(None, None, 8, 0, 0, None, None, k, params[0], params[1], params[2],
                                        1, 1, arithmetic, None, 0, None)
    return st, L.bitsknn_last_error().decode()


def test_fused_arithmetic_is_a_call_argument(bk):
    assert _fused_ex_status(bk, 32, bk.FUSED_FP32) == (bk.OK, "")
    assert _fused_ex_status(bk, 32, bk.FUSED_BF16X3) == (bk.OK, "")
    st, text = _fused_ex_status(bk, 32, 7)
    assert st == bk.ERR_INVALID and "unknown arithmetic 7" in text
    st, text = _fused_ex_status(bk, 5, bk.FUSED_BF16X3)
    assert st == bk.ERR_UNSUPPORTED and text == "Unsupported k value: 5"
    # nothing process-wide is left behind by a call: the library exports no mode setter
    assert not hasattr(bk, "fused_set_arithmetic")
    with pytest.raises(AttributeError):
        bk.lib().bitsknn_fused_set_arithmetic


def test_two_threads_with_different_arithmetics(bk):
    """Two host threads validate calls with different arithmetics and different mistakes at the
    same time: every thread sees its own status and its own (thread-local) message."""
    import threading
    failures = []

    def worker(arithmetic, bad_k, rounds=2000):
        for i in range(rounds):
            if i % 2 == 0:
                got = _fused_ex_status(bk, 32, arithmetic)
                want = (bk.OK, "")
            else:
                got = _fused_ex_status(bk, bad_k, arithmetic)
                want = (bk.ERR_UNSUPPORTED, "Unsupported k value: %d" % bad_k)
            if got != want:
                failures.append((arithmetic, i, got))
                return

    threads = [threading.Thread(target=worker, args=(bk.FUSED_FP32, 5)),
               threading.Thread(target=worker, args=(bk.FUSED_BF16X3, 7))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures[:3]


def test_topk_accepts_reference_parameter_lists_with_zero_rows(bk):
    # rows == 0 is a no-op that returns before any launch: every supported combination is accepted
    for block in (128, 256, 512):
        for batch in range(1, 17):
            for k in (1, 16, 17, 32, 64, 128, 256, 512, 1024, 2048):
                st, text = _topk_status(bk, k, block, batch)
                assert st == bk.OK, (block, batch, k, text)


# messages of the reference dispatch (src/topk/singlepass/partial_bitonic.cu:341-358)
@pytest.mark.parametrize("k,block,msg", [
    (32, 100, "Unsupported block size: 100"),
    (32, 1024, "Unsupported block size: 1024"),
    (0, 256, "Unsupported k value: 0"),
    (4096, 64, "Unsupported k value: 4096"),
])
def test_partial_bitonic_rejects_unsupported_parameters(bk, k, block, msg):
    L = bk.lib()
    st = L.bitsknn_topk_partial_bitonic_f32(None, 0, 0, 0, None, None, 0, k, block, None)
    assert st == bk.ERR_UNSUPPORTED
    assert L.bitsknn_last_error().decode() == msg
    for good_block in (64, 128, 256, 512):
        for good_k in (1, 16, 100, 2048):
            assert L.bitsknn_topk_partial_bitonic_f32(None, 0, 0, 0, None, None, 0, good_k, good_block,
                                                      None) == bk.OK


def _load_tuning():
    import importlib.util
    path = os.path.join(ROOT, "bits-knn-jpdc2024_amd", "bitsknn", "tuning.py")
    spec = importlib.util.spec_from_file_location("bitsknn_tuning", path)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def test_config_lookup_matches_reference_script():
    """config_algorithm() against what the reference's awk lookup (scripts/config.sh:97-200)
    printed for the same requests on tests/golden/optima_sample.csv (vectors written by
    tests/golden/make_config_vectors.py)."""
    tuning = _load_tuning()
    golden = os.path.join(ROOT, "tests", "golden")
    with open(os.path.join(golden, "config_vectors.json")) as handle:
        vectors = json.load(handle)
    assert len(vectors) >= 40
    for vec in vectors:
        def arg(x):
            return None if x == "None" else x
        got = tuning.config_algorithm(vec["algorithm"], arg(vec["query_count"]), arg(vec["k"]),
                                      arg(vec["dim"]), arg(vec["hostname"]),
                                      optima_file=os.path.join(golden, "optima_sample.csv"))
        want = tuple(None if w == "" else int(w) for w in vec["answer"])
        assert got == want, (vec, got)


def test_shipped_optima_file():
    """The MI355X optima file has the reference's columns (scripts/optima.csv, line 1) and a row
    for every (algorithm, q, k) of the reference's search grid (scripts/run-opt-ipt.sh:38-47),
    for bits-sq on the query counts that leave compute units idle, and for fused-cache."""
    import csv
    tuning = _load_tuning()
    with open(tuning.DEFAULT_OPTIMA, newline="") as handle:
        rows = list(csv.DictReader(handle))
    assert tuple(rows[0].keys()) == tuning.OPTIMA_COLUMNS
    seen = {(r["algorithm"], int(r["query_count"]), int(r["k"])) for r in rows}
    for name, _ in tuning.ALGORITHMS:
        for q in tuning.QUERY_COUNTS:
            for k in tuning.K_VALUES:
                assert (name, q, k) in seen
    # and the rows for many short rows, measured on their own shape
    for name, _ in tuning.ALGORITHMS:
        for k in tuning.K_VALUES:
            short = [r for r in rows if r["algorithm"] == name and int(r["k"]) == k and
                     int(r["query_count"]) == tuning.SHORT_ROWS_QUERY_COUNT]
            assert len(short) == 1 and int(short[0]["point_count"]) == tuning.SHORT_ROWS_POINT_COUNT
    assert sum(r["algorithm"] == "partial-bitonic-regs" for r in rows) == 28
    for r in rows:
        assert float(r["time"]) > 0
        if r["algorithm"] in ("bits", "bits-prefetch", "bits-sq"):
            # only values per thread that are kernels of their own (whole 16-byte loads)
            assert int(r["block_size"]) in (128, 256, 512) and int(r["items_per_thread"]) in tuning.BATCH_SIZES
        if r["algorithm"] == "partial-bitonic-regs":
            assert int(r["block_size"]) in (64, 128, 256, 512)
    block, deg, batch, _, _ = tuning.config_algorithm("bits", 1024, 32)
    assert block in (128, 256, 512) and deg == 1 and batch in tuning.BATCH_SIZES
    # bits-sq: every (q, k) of its grid, with the number of parts in the deg column; cutting the
    # rows must pay where one row per workgroup leaves most of the GPU idle
    plain = {(int(r["query_count"]), int(r["k"])): float(r["time"]) for r in rows if r["algorithm"] == "bits"}
    for q in tuning.SQ_QUERY_COUNTS:
        for k in tuning.K_VALUES:
            mine = [r for r in rows if r["algorithm"] == "bits-sq" and int(r["query_count"]) == q and int(r["k"]) == k]
            assert len(mine) == 1 and int(mine[0]["deg"]) in tuning.SQ_DEGREES
            if q == 64:
                assert float(mine[0]["time"]) < plain[(q, k)]
    block, deg, batch, _, _ = tuning.config_algorithm("bits-sq", 64, 32)
    assert deg in tuning.SQ_DEGREES
    # fused-cache: the reference's fixed parameters (they do not steer the kernel) for every
    # (shape, dim, k) of the grid; the lookup by (q, k, dim) returns them
    fused = [r for r in rows if r["algorithm"] == "fused-cache"]
    assert len(fused) == len(tuning.FUSED_SHAPES) * len(tuning.FUSED_DIMS) * len(tuning.FUSED_K_VALUES)
    assert tuning.config_algorithm("fused-cache", 8192, 32, 16) == (1, 1, 8, 4, 2)


def test_entry_points_never_allocate_device_memory():
    """The C ABI's contract: every entry point works on the caller's memory and allocates and frees
    nothing (bitsknn_fused_l2_topk_f32_static in particular, which exists for callers that cannot
    allocate).  No source of the library may name an allocating or freeing runtime call, and the
    sources behind the static entry point no memset either (a memset node recorded into a captured
    graph is not replayed reliably)."""
    import glob
    import re
    csrc = os.path.join(ROOT, "bits-knn-jpdc2024_amd", "csrc")
    sources = sorted(glob.glob(os.path.join(csrc, "*.hip")) + glob.glob(os.path.join(csrc, "*.hpp")))
    assert len(sources) >= 10
    forbidden = re.compile(r"\bhip(Malloc|Free|HostMalloc|HostFree|ExtMalloc|MallocAsync|FreeAsync|MallocManaged)\w*")
    memset = re.compile(r"\bhipMemset\w*")
    for path in sources:
        with open(path) as handle:
            text = handle.read()
        assert forbidden.search(text) is None, (path, forbidden.search(text).group(0))
        name = os.path.basename(path)
        if name.startswith("fused") or name.startswith("topk_bits") or name in ("common.hpp", "bitonic_net.hpp"):
            assert memset.search(text) is None, (path, memset.search(text).group(0))
