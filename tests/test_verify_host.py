"""host/verify.cpp -- the comparison behind `knn -v ALG` -- on hand-built results: a real mismatch
is reported, ties are tolerated exactly where the reference tolerates them
(src/verify.cpp:17-112), and the CPU oracle's restatement gives the same verdict on the same pairs.
The function is compiled into a small driver (tests/verify_driver.cpp) and run on the CPU."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "bits-knn-jpdc2024_amd", "host")


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("verify") / "verify_driver")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    subprocess.run(["g++", "-O1", "-std=c++20", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROOT, "include"),
                    "-I" + HOST, "-I" + os.path.join(rocm, "include"), "-o", out,
                    os.path.join(ROOT, "tests", "verify_driver.cpp"), os.path.join(HOST, "verify.cpp")], check=True)
    return out


def _verify(driver, expected, actual, k):
    lines = [f"{k} {len(expected)}"]
    for result in (expected, actual):
        lines += [f"{float(d)!r} {int(i)}" for d, i in result]
    p = subprocess.run([driver], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=60)
    assert p.returncode == 0, p.stderr
    return p.stdout.strip() == "1", p.stderr


def _both(driver, oracle, expected, actual, k):
    ok, report = _verify(driver, expected, actual, k)
    o_ok, o_bad = oracle.verify([d for d, _ in expected], [i for _, i in expected],
                                [d for d, _ in actual], [i for _, i in actual], k)
    assert ok == o_ok, (ok, o_ok, report)
    assert report.count("Difference at index") == o_bad
    return ok, report


def test_identical_results_are_accepted(driver, oracle):
    result = [(0.1, 5), (0.2, 7), (0.3, 1), (0.05, 2), (0.6, 9), (0.7, 4)]
    assert _both(driver, oracle, result, result, 3) == (True, "")


def test_a_real_mismatch_is_reported(driver, oracle):
    expected = [(0.1, 5), (0.2, 7), (0.3, 1), (0.05, 2), (0.6, 9), (0.7, 4)]
    actual = list(expected)
    actual[4] = (0.65, 8)          # another point at another distance, second query
    ok, report = _both(driver, oracle, expected, actual, 3)
    assert not ok
    assert "Difference at index 4 (expected: 9, actual: 8)" in report
    assert "- expected distance: 0.6" in report and "- actual distance: 0.65" in report
    # a wrong neighbour at the same distance in the middle of a list is a mismatch too: the
    # entries after it are not all at that distance
    actual = list(expected)
    actual[0] = (0.1, 6)
    ok, report = _both(driver, oracle, expected, actual, 3)
    assert not ok and "Difference at index 0 (expected: 5, actual: 6)" in report


def test_equal_distances_may_come_in_any_order(driver, oracle):
    expected = [(0.1, 5), (0.2, 7), (0.2, 3), (0.2, 11), (0.9, 1)]
    actual = [(0.1, 5), (0.2, 11), (0.2, 7), (0.2, 3), (0.9, 1)]
    assert _both(driver, oracle, expected, actual, 5) == (True, "")
    # ... and within the relative tolerance of 1e-3 as well
    actual = [(0.1, 5), (0.20001, 11), (0.2, 7), (0.19999, 3), (0.9, 1)]
    assert _both(driver, oracle, expected, actual, 5)[0]


def test_a_tie_at_the_end_of_a_list_may_hold_other_members(driver, oracle):
    # four points at distance 0.5 compete for the last two places of the first query's list
    expected = [(0.1, 5), (0.5, 20), (0.5, 21), (0.3, 1), (0.4, 2), (0.6, 3)]
    actual = [(0.1, 5), (0.5, 22), (0.5, 23), (0.3, 1), (0.4, 2), (0.6, 3)]
    assert _both(driver, oracle, expected, actual, 3) == (True, "")
    # the same swap is a mismatch when the list goes on with a larger distance
    expected = [(0.1, 5), (0.5, 20), (0.7, 21), (0.3, 1), (0.4, 2), (0.6, 3)]
    actual = [(0.1, 5), (0.5, 22), (0.7, 21), (0.3, 1), (0.4, 2), (0.6, 3)]
    ok, report = _both(driver, oracle, expected, actual, 3)
    assert not ok and "Difference at index 1 (expected: 20, actual: 22)" in report


def test_random_results_with_injected_faults(driver, oracle):
    rng = np.random.default_rng(9)
    k, queries = 8, 50
    for case in range(20):
        dist = np.sort(np.round(rng.random((queries, k)) * 20) / 20, axis=1).astype(np.float32)  # many ties
        idx = rng.permutation(queries * k).reshape(queries, k).astype(np.int32)
        expected = list(zip(dist.ravel().tolist(), idx.ravel().tolist()))
        actual_d, actual_i = dist.copy(), idx.copy()
        if case % 2:
            row, col = int(rng.integers(queries)), int(rng.integers(k))
            actual_i[row, col] = 10_000 + case
            actual_d[row, col] += 0.5
            actual_d[row] = np.sort(actual_d[row])
        actual = list(zip(actual_d.ravel().tolist(), actual_i.ravel().tolist()))
        ok, _ = _both(driver, oracle, expected, actual, k)
        if case % 2 == 0:
            assert ok
