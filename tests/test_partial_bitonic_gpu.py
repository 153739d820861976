"""Parity of the partial-bitonic-regs HIP kernel (through the C ABI) with the CPU oracle.

Bar: bit-exact values and labels, equal values ordered by lower label (the reference's kernel,
src/topk/singlepass/partial_bitonic.cu:217-294, compares values only and leaves the order of
equal values open; the canonical order is one of its valid results).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _check(bk, dev, oracle, matrix, k, block):
    import torch
    od, ol = bk.topk_partial_bitonic(torch.from_numpy(matrix).to(dev), k, block)
    torch.cuda.synchronize()
    ed, el = oracle.topk(matrix, k)
    assert np.array_equal(od.cpu().numpy().view(np.uint32), ed.view(np.uint32)), "values differ"
    assert np.array_equal(ol.cpu().numpy(), el), "labels differ"


@pytest.mark.parametrize("block", [64, 128, 256, 512])
@pytest.mark.parametrize("k", [1, 16, 32, 64, 100, 128, 256, 512, 1024, 2048])
def test_uniform_rows_all_k_and_blocks(bk, dev, oracle, block, k):
    m = oracle.uniform_matrix(2000 + k + block, 5, 30000)
    _check(bk, dev, oracle, m, k, block)


@pytest.mark.parametrize("cols", [1, 2, 63, 64, 65, 127, 129, 511, 512, 513, 1000, 4095, 4097, 12289])
def test_ragged_row_lengths(bk, dev, oracle, cols):
    m = oracle.uniform_matrix(cols + 5, 3, cols)
    for k, block in ((1, 64), (16, 512), (32, 128), (300, 256), (2048, 64)):
        _check(bk, dev, oracle, m, k, block)


@pytest.mark.parametrize("kind", ["ascending", "descending", "256-values", "constant"])
def test_hard_inputs(bk, dev, oracle, kind):
    base = oracle.uniform_matrix(98, 4, 65536)
    if kind == "ascending":
        m = np.sort(base, axis=1)
    elif kind == "descending":
        m = np.ascontiguousarray(np.sort(base, axis=1)[:, ::-1])
    elif kind == "256-values":
        m = (np.floor(base * 256) / 256).astype(np.float32)
    else:
        m = np.full_like(base, 0.25)
    for k, block in ((32, 128), (256, 256), (2048, 512), (2048, 64)):
        _check(bk, dev, oracle, m, k, block)


def test_infinities_negative_values_and_short_rows(bk, dev, oracle):
    m = oracle.uniform_matrix(3, 4, 20000, -5.0, 5.0)
    m[0, 17] = -np.inf
    m[1, 5] = np.inf
    m[2, :] = np.inf
    m[2, 100] = 1.0
    _check(bk, dev, oracle, m, 64, 256)
    _check(bk, dev, oracle, m, 1024, 128)
    _check(bk, dev, oracle, oracle.uniform_matrix(8, 3, 20), 32, 128)   # k > cols: padded tail


def test_strided_views_and_errors(bk, dev, oracle):
    import torch
    big = oracle.uniform_matrix(6, 7, 30011)
    t = torch.from_numpy(big).to(dev)
    od = torch.full((7, 100), -1.0, device=dev)
    ol = torch.full((7, 100), -1, dtype=torch.int32, device=dev)
    bk.topk_partial_bitonic(t[:, 3:20000], 40, 256, out_dist=od, out_label=ol)
    torch.cuda.synchronize()
    ed, el = oracle.topk(big[:, 3:20000], 40)
    assert np.array_equal(od[:, :40].cpu().numpy(), ed) and np.array_equal(ol[:, :40].cpu().numpy(), el)
    assert (od[:, 40:] == -1).all() and (ol[:, 40:] == -1).all()
    with pytest.raises(bk.BitsKnnError, match="Unsupported block size: 1024"):
        bk.topk_partial_bitonic(t, 16, 1024)
    with pytest.raises(bk.BitsKnnError, match="Unsupported k value: 4096"):
        bk.topk_partial_bitonic(t, 4096, 256)


def test_same_result_as_bits_at_full_row_length(bk, dev):
    """2^20-column rows: the unfiltered kernel and the bits kernel agree bit for bit."""
    import torch
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    m = torch.rand((64, 1 << 20), device=dev, generator=gen)
    for k, block in ((32, 256), (512, 512)):
        pd, pl = bk.topk_partial_bitonic(m, k, block)
        bd, bl = bk.topk_bits(m, k, 256, 8)
        torch.cuda.synchronize()
        assert torch.equal(pd, bd) and torch.equal(pl, bl)
