"""Product range builders (C ABI, host side) and the Python ranges API on CPU tensors:
bit-exact against the C oracle and the golden vectors; API behaviour of
kernel_matmul/ranges.py:39-156 of the reference."""
import os

import numpy as np
import pytest
import torch

from kernel_matmul_amd import ranges
from oracle import ranges as oracle_ranges

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "ranges_golden.npz")


def test_golden_vectors_host():
    data = np.load(GOLDEN)
    keys = sorted({k.rsplit("_", 1)[0] for k in data.files if k.endswith("_meta")})
    for key in keys:
        meta = data[key + "_meta"]
        if key.startswith("asym"):
            cutoff, bs, align = float(meta[0]), int(meta[1]), bool(meta[2])
            x1, x2 = torch.from_numpy(data[key + "_x1"]), torch.from_numpy(data[key + "_x2"])
            s, e = ranges.make_ranges(cutoff, x1, x2, block_size=bs, align=align)
            assert s.dtype == torch.int32 and e.dtype == torch.int32
            np.testing.assert_array_equal(s.numpy(), data[key + "_start"], err_msg=key)
            np.testing.assert_array_equal(e.numpy(), data[key + "_end"], err_msg=key)
            if align:
                st, et = ranges.transpose_ranges(s, e, x1.shape[1], x2.shape[1], block_size=bs)
                np.testing.assert_array_equal(st.numpy(), data[key + "_start_t"], err_msg=key)
                np.testing.assert_array_equal(et.numpy(), data[key + "_end_t"], err_msg=key)
        else:
            cutoff, bs = float(meta[0]), int(meta[1])
            s, e = ranges.make_ranges(cutoff, torch.from_numpy(data[key + "_x"]), block_size=bs)
            np.testing.assert_array_equal(s.numpy(), data[key + "_start"], err_msg=key)
            np.testing.assert_array_equal(e.numpy(), data[key + "_end"], err_msg=key)


@pytest.mark.parametrize("batch", [(), (3,), (2, 3)])
@pytest.mark.parametrize("block_size", [1, 3, 128])
def test_random_against_oracle(batch, block_size):
    rng = np.random.default_rng(hash((batch, block_size)) % 2**32)
    for _ in range(30):
        n1, n2 = int(rng.integers(1, 900)), int(rng.integers(1, 900))
        x1 = np.sort((rng.random((*batch, n1)) * 30).astype(np.float32), axis=-1)
        x2 = np.sort((rng.random((*batch, n2)) * 30).astype(np.float32), axis=-1)
        cutoff = float(rng.choice([0.0, 0.2, 2.0, 50.0]))
        for align in (False, True):
            s, e = ranges.make_ranges(cutoff, torch.from_numpy(x1), torch.from_numpy(x2),
                                      block_size=block_size, align=align)
            so, eo = oracle_ranges.make_ranges(cutoff, x1, x2, block_size=block_size, align=align)
            assert s.shape == (*batch, -(-n1 // block_size))
            np.testing.assert_array_equal(s.numpy(), so)
            np.testing.assert_array_equal(e.numpy(), eo)
        st, et = ranges.transpose_ranges(s, e, n1, n2, block_size=block_size)
        sto, eto = oracle_ranges.transpose_ranges(so, eo, n1, n2, block_size=block_size)
        np.testing.assert_array_equal(st.numpy(), sto)
        np.testing.assert_array_equal(et.numpy(), eto)
        s, e = ranges.make_ranges(cutoff, torch.from_numpy(x1), block_size=block_size)
        so, eo = oracle_ranges.make_ranges(cutoff, x1, block_size=block_size)
        np.testing.assert_array_equal(s.numpy(), so)
        np.testing.assert_array_equal(e.numpy(), eo)


def test_transpose_noalign_raises():
    # the reference's own known-answer case, tests/test_ranges.py:193-199
    x1 = torch.tensor([[0.0, 0.0, 2.0]])
    x2 = torch.tensor([[0.0, 2.0, 2.0]])
    start, end = ranges.make_ranges(1.0, x1, x2, block_size=2, align=False)
    assert start.tolist() == [[0, 1]] and end.tolist() == [[1, 3]]
    with pytest.raises(ValueError, match="Ranges must be block-aligned"):
        ranges.transpose_ranges(start, end, 3, 3, block_size=2)


def test_dense_pattern_and_shapes():
    x1 = torch.sort(torch.rand(2, 3, 50))[0]
    x2 = torch.sort(torch.rand(2, 3, 55))[0]
    for bs in (1, 3):
        start, end = ranges.make_ranges(None, x1, x2, block_size=bs)
        assert torch.all(start == 0) and torch.all(end == 55)
        assert start.shape == (2, 3, -(-50 // bs)) and start.dtype == torch.int32
        start, end = ranges.make_ranges(None, x1, block_size=bs)
        assert torch.all(start == 0) and torch.all(end == 50)
    start, end = ranges.make_ranges(1.0, x1[0, 0], block_size=3)
    assert start.shape == (17,)


def test_ranges_cache():
    x = torch.sort(torch.rand(300) * 10)[0]
    cache = ranges.RangesCache(x, align=True)
    assert cache.x is x and cache.align is True
    first = cache[1.0]
    assert cache[1.0] is first
    other = cache[2.0]
    assert other is not first
    expected = ranges.make_ranges(1.0, x, align=True)
    assert torch.equal(first[0], expected[0]) and torch.equal(first[1], expected[1])
    dense = cache[None]
    assert torch.all(dense[0] == 0) and torch.all(dense[1] == 300)


def test_empty_and_tiny_inputs():
    start, end = ranges.make_ranges(1.0, torch.zeros(0, 10), torch.zeros(0, 12), block_size=4)
    assert start.shape == (0, 3) and end.shape == (0, 3)
    x = torch.tensor([1.0, 2.0, 3.0])
    start, end = ranges.make_ranges(0.5, x, block_size=128)
    so, eo = oracle_ranges.make_ranges(0.5, x.numpy(), block_size=128)
    np.testing.assert_array_equal(start.numpy(), so)
    np.testing.assert_array_equal(end.numpy(), eo)
    assert end.tolist() == [128]  # reference quirk: fewer points than one block


def test_non_float_input_rejected():
    with pytest.raises(RuntimeError, match="Float"):
        ranges.make_ranges(1.0, torch.zeros(10, dtype=torch.float64))
