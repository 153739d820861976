"""The register sorting networks (csrc/bitonic_net.hpp) driven directly by test-only kernels
(tests/net_kernels.hip, built into tests/libnettest.so): full sorts and bitonic merges of random
and heavily tied 64-bit keys, compared with numpy's sort, over workgroup-wide and in-wave group
sizes, both exchange flavours below 64 lanes (vector moves / LDS crossbar) and both LDS exchange
schemes (one region / two alternating regions).

Counterpart of the reference's tests/bitonic_sort_regs_test.cu:21-160, which sorts
(items per thread, block size) in {(1,32), (1,64), (1,128), (1,1024), (2,32), (4,32), (8,64),
(2,1024)} and checks that the output is monotonic; here the output must equal the sorted input.
"""
import ctypes
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
XBAR_NONE, XBAR_4_16_32 = 0, 4 | 16 | 32

# (lanes or threads per group, keys per thread, crossbar set, two LDS regions)
IN_WAVE = [(8, 4, XBAR_NONE, 0), (16, 4, XBAR_NONE, 0), (32, 4, XBAR_NONE, 0), (64, 4, XBAR_NONE, 0),
           (16, 2, XBAR_NONE, 0), (32, 1, XBAR_NONE, 0), (32, 2, XBAR_NONE, 0), (64, 1, XBAR_NONE, 0),
           (64, 2, XBAR_NONE, 0), (64, 8, XBAR_NONE, 0), (64, 4, XBAR_4_16_32, 0), (32, 4, XBAR_4_16_32, 0)]
WORKGROUP = [(128, 1, XBAR_4_16_32, 1), (128, 2, XBAR_4_16_32, 1), (128, 16, XBAR_4_16_32, 1),
             (256, 1, XBAR_4_16_32, 1), (256, 8, XBAR_4_16_32, 1), (512, 1, XBAR_4_16_32, 1),
             (512, 4, XBAR_4_16_32, 1), (128, 1, XBAR_NONE, 0), (128, 4, XBAR_NONE, 0), (256, 2, XBAR_NONE, 0),
             (512, 4, XBAR_NONE, 0), (128, 8, XBAR_NONE, 1), (256, 4, XBAR_4_16_32, 0), (1024, 1, XBAR_NONE, 0),
             (1024, 2, XBAR_4_16_32, 1)]


@pytest.fixture(scope="module")
def nettest():
    path = os.path.join(HERE, "libnettest.so")
    if not os.path.exists(path):
        pytest.fail(f"{path} is missing: build it with `make -C bits-knn-jpdc2024_amd nettest`")
    import torch  # noqa: F401  (the process's HIP runtime is torch's)
    lib = ctypes.CDLL(path)
    lib.nettest_run.restype = ctypes.c_int
    lib.nettest_run.argtypes = [ctypes.c_int] * 6 + [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    return lib


def _keys(rng, groups, n, kind):
    if kind == "random":
        return rng.integers(0, 1 << 63, size=(groups, n), dtype=np.uint64) * np.uint64(2) + \
            rng.integers(0, 2, size=(groups, n), dtype=np.uint64)
    if kind == "tied":      # a handful of distinct keys: every compare-exchange meets equal keys
        return rng.integers(0, 5, size=(groups, n), dtype=np.uint64) << np.uint64(40)
    if kind == "high-word":  # keys that differ in the upper 32 bits only / in the lower 32 bits only
        a = rng.integers(0, 1 << 32, size=(groups, n), dtype=np.uint64)
        return np.where(rng.integers(0, 2, size=(groups, n)) == 0, a << np.uint64(32), a + (np.uint64(7) << np.uint64(32)))
    return np.tile(np.arange(n, dtype=np.uint64)[::-1], (groups, 1))  # reversed ramp


def _run(nettest, dev, keys, bs, ipt, xbar, pp, desc, op):
    import torch
    t = torch.from_numpy(keys.view(np.int64).copy()).to(dev)
    status = nettest.nettest_run(bs, ipt, xbar, pp, desc, op, ctypes.c_void_p(t.data_ptr()), keys.shape[0],
                                 ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert status == 0, ("nettest_run", status, bs, ipt, xbar, pp)
    torch.cuda.synchronize()
    return t.cpu().numpy().view(np.uint64)


@pytest.mark.parametrize("desc", [0, 1])
@pytest.mark.parametrize("bs,ipt,xbar,pp", IN_WAVE + WORKGROUP)
def test_full_sort(nettest, dev, bs, ipt, xbar, pp, desc):
    rng = np.random.default_rng(bs * 100 + ipt)
    n = bs * ipt
    groups = 16 if bs < 64 else 3   # whole waves of in-wave groups
    for kind in ("random", "tied", "high-word", "ramp"):
        keys = _keys(rng, groups, n, kind)
        got = _run(nettest, dev, keys, bs, ipt, xbar, pp, desc, 0)
        want = np.sort(keys, axis=1)
        if desc:
            want = want[:, ::-1]
        assert np.array_equal(got, want), (kind, bs, ipt, xbar, pp, desc)


@pytest.mark.parametrize("desc", [0, 1])
@pytest.mark.parametrize("bs,ipt,xbar,pp", IN_WAVE + WORKGROUP)
def test_merge_of_a_bitonic_sequence(nettest, dev, bs, ipt, xbar, pp, desc):
    """The last phase alone: an ascending run followed by a descending one (the element-wise
    minimum of an ascending list and a descending buffer is such a sequence) comes out sorted."""
    rng = np.random.default_rng(bs * 100 + ipt + 7)
    n = bs * ipt
    groups = 16 if bs < 64 else 3
    for kind in ("random", "tied"):
        keys = _keys(rng, groups, n, kind)
        for split in (n // 2, n // 4, n - 1, 1):
            bitonic = np.concatenate([np.sort(keys[:, :split], axis=1), np.sort(keys[:, split:], axis=1)[:, ::-1]],
                                     axis=1)
            got = _run(nettest, dev, np.ascontiguousarray(bitonic), bs, ipt, xbar, pp, desc, 1)
            want = np.sort(keys, axis=1)
            if desc:
                want = want[:, ::-1]
            assert np.array_equal(got, want), (kind, split, bs, ipt, xbar, pp, desc)
