import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "bits-knn-jpdc2024_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import binding
    binding.lib()
    return binding


@pytest.fixture(scope="session")
def golden():
    import json
    with open(os.path.join(ROOT, "tests", "golden", "checksums.json")) as f:
        return json.load(f)["records"]


@pytest.fixture(scope="session")
def bk():
    """The product library behind its C ABI (no fallback: fails if it is not built)."""
    import bitsknn
    bitsknn.lib()
    return bitsknn


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    return torch.device("cuda:0")


def pytest_sessionfinish(session, exitstatus):
    """The largest k-th-neighbour distance errors the floating-point parity checks met (pytest -s)."""
    try:
        import parity
    except ImportError:
        return
    for key, seen in sorted(parity.margins.items()):
        print("\nparity margin %s: %s" % (key, ", ".join(
            ("%s %d" if isinstance(kv[1], int) else "%s %.3g") % kv for kv in sorted(seen.items()))))
