"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol, and rejects
unsupported parameters with the reference's messages before touching the GPU."""
import ctypes
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


def test_topk_accepts_reference_parameter_lists_with_zero_rows(bk):
    # rows == 0 is a no-op that returns before any launch: every supported combination is accepted
    for block in (128, 256, 512):
        for batch in range(1, 17):
            for k in (1, 16, 17, 32, 64, 128, 256, 512, 1024, 2048):
                st, text = _topk_status(bk, k, block, batch)
                assert st == bk.OK, (block, batch, k, text)
