"""Pins the C range oracle (oracle/ranges_oracle.c): the reference's literal known answer,
golden vectors written by the reference's own ranges.cpp, a direct comparison with that build
where it exists, and the property suite of the reference's tests/test_ranges.py:77-190."""
import math
import os
import sys

import numpy as np
import pytest
import torch

from oracle import ranges as oracle_ranges

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "ranges_golden.npz")
REF_DIR = os.path.join(os.path.dirname(os.path.dirname(__file__)), "oracle", "_ref")


def _golden_cases():
    data = np.load(GOLDEN)
    keys = sorted({k.rsplit("_", 1)[0] for k in data.files if k.endswith("_meta")})
    return data, keys


def test_known_answer_from_reference_test():
    # tests/test_ranges.py:193-199 of the reference: x1=[0,0,2], x2=[0,2,2], cutoff 1, bs 2.
    x1 = np.array([[0.0, 0.0, 2.0]], dtype=np.float32)
    x2 = np.array([[0.0, 2.0, 2.0]], dtype=np.float32)
    start, end = oracle_ranges.make_ranges(1.0, x1, x2, block_size=2, align=False)
    assert start.tolist() == [[0, 1]] and end.tolist() == [[1, 3]]
    with pytest.raises(ValueError, match="Ranges must be block-aligned"):
        oracle_ranges.transpose_ranges(start, end, 3, 3, block_size=2)


def test_golden_vectors():
    data, keys = _golden_cases()
    assert len(keys) > 200
    for key in keys:
        meta = data[key + "_meta"]
        if key.startswith("asym"):
            cutoff, bs, align = float(meta[0]), int(meta[1]), bool(meta[2])
            x1, x2 = data[key + "_x1"], data[key + "_x2"]
            s, e = oracle_ranges.make_ranges(cutoff, x1, x2, block_size=bs, align=align)
            np.testing.assert_array_equal(s, data[key + "_start"], err_msg=key)
            np.testing.assert_array_equal(e, data[key + "_end"], err_msg=key)
            if align:
                st, et = oracle_ranges.transpose_ranges(s, e, x1.shape[1], x2.shape[1], block_size=bs)
                np.testing.assert_array_equal(st, data[key + "_start_t"], err_msg=key)
                np.testing.assert_array_equal(et, data[key + "_end_t"], err_msg=key)
        else:
            cutoff, bs = float(meta[0]), int(meta[1])
            s, e = oracle_ranges.make_ranges(cutoff, data[key + "_x"], block_size=bs)
            np.testing.assert_array_equal(s, data[key + "_start"], err_msg=key)
            np.testing.assert_array_equal(e, data[key + "_end"], err_msg=key)


@pytest.mark.skipif(not os.path.exists(os.path.join(REF_DIR, "km_ranges_ref.so")),
                    reason="reference range builder not built (oracle/build_ref.sh)")
def test_against_reference_build():
    sys.path.insert(0, REF_DIR)
    import km_ranges_ref as ref

    rng = np.random.default_rng(5)
    for _ in range(150):
        bs = int(rng.choice([1, 2, 3, 7, 128]))
        n1, n2 = int(rng.integers(1, 700)), int(rng.integers(1, 700))
        batch = int(rng.integers(1, 4))
        scale = float(rng.choice([1.0, 10.0, 1000.0]))
        x1 = np.sort((rng.random((batch, n1)) * scale).astype(np.float32), axis=1)
        x2 = np.sort((rng.random((batch, n2)) * scale).astype(np.float32), axis=1)
        cutoff = float(rng.choice([0.0, 0.05, 0.5, 3.0, 2000.0]))
        for align in (False, True):
            s, e = oracle_ranges.make_ranges(cutoff, x1, x2, block_size=bs, align=align)
            rs, re_ = ref.make_ranges(torch.from_numpy(x1), torch.from_numpy(x2), cutoff, bs, align)
            np.testing.assert_array_equal(s, rs.numpy())
            np.testing.assert_array_equal(e, re_.numpy())
        st, et = oracle_ranges.transpose_ranges(s, e, n1, n2, block_size=bs)
        rst, ret = ref.transpose_ranges(rs, re_, n1, n2, bs)
        np.testing.assert_array_equal(st, rst.numpy())
        np.testing.assert_array_equal(et, ret.numpy())
        s, e = oracle_ranges.make_ranges(cutoff, x1, block_size=bs)
        rs, re_ = ref.make_ranges_symmetric(torch.from_numpy(x1), cutoff, bs)
        np.testing.assert_array_equal(s, rs.numpy())
        np.testing.assert_array_equal(e, re_.numpy())


def _x_pair(rng, offset, gap1, gap2, batch):
    x1 = np.sort(rng.random((*batch, 50)).astype(np.float32) * 10, axis=-1)
    x2 = np.sort(rng.random((*batch, 55)).astype(np.float32) * 10, axis=-1) + np.float32(offset)
    if gap1 is not None:
        x1[..., gap1:] += 20
    if gap2 is not None:
        x2[..., gap2:] += 20
    return x1, x2


@pytest.mark.parametrize("cutoff", [0.1, 1.0, 11.0])
@pytest.mark.parametrize("align", [True, False])
@pytest.mark.parametrize("block_size", [1, 3])
def test_asymmetric_properties(cutoff, align, block_size):
    # Bounds, alignment and exact membership at the stepped positions
    # (tests/test_ranges.py:77-114 of the reference).
    rng = np.random.default_rng(11)
    for offset in (-1.0, 0.0, 1.5):
        for gap1 in (None, 0, 10):
            for gap2, batch in ((None, ()), (0, (3,)), (10, (2, 3))):
                x1, x2 = _x_pair(rng, offset, gap1, gap2, batch)
                start, end = oracle_ranges.make_ranges(cutoff, x1, x2, block_size=block_size, align=align)
                step = block_size if align else 1
                assert np.all(start >= 0) and np.all(start <= end) and np.all(end <= x2.shape[-1])
                assert start.shape == end.shape and start.shape[:-1] == x1.shape[:-1]
                if align:
                    assert np.all((start % block_size == 0) | (start == x2.shape[-1]))
                    assert np.all((end % block_size == 0) | (end == x2.shape[-1]))
                x1_, x2_ = x1.reshape(-1, 50), x2.reshape(-1, 55)
                s_, e_ = start.reshape(-1, start.shape[-1]), end.reshape(-1, end.shape[-1])
                c = np.float32(cutoff)
                for b in range(x1_.shape[0]):
                    for i in range(int(math.ceil(50 / block_size))):
                        lo = x1_[b, i * block_size]
                        hi = x1_[b, min(i * block_size + block_size, 50) - 1]
                        for j in range(0, 55, step):
                            inside = (lo - c <= x2_[b, j]) and (x2_[b, j] <= hi + c)
                            if inside:
                                assert s_[b, i] <= j < e_[b, i]
                            else:
                                assert j < s_[b, i] or e_[b, i] <= j


@pytest.mark.parametrize("cutoff", [0.1, 1.0, 11.0])
@pytest.mark.parametrize("block_size", [1, 3])
def test_symmetric_properties(cutoff, block_size):
    # Symmetric mask and block membership (tests/test_ranges.py:139-160 of the reference).
    rng = np.random.default_rng(12)
    for gap in (None, 0, 10):
        for batch in ((), (3,), (2, 3)):
            x = np.sort(rng.random((*batch, 50)).astype(np.float32) * 10, axis=-1)
            if gap is not None:
                x[..., gap:] += 20
            start, end = oracle_ranges.make_ranges(cutoff, x, block_size=block_size)
            assert np.all(start >= 0) and np.all(start <= end) and np.all(end <= 50)
            x_ = x.reshape(-1, 50)
            s_, e_ = start.reshape(-1, start.shape[-1]), end.reshape(-1, end.shape[-1])
            for b in range(x_.shape[0]):
                mask = np.zeros((50, 50), dtype=bool)
                for i in range(s_.shape[1]):
                    mask[i * block_size:(i + 1) * block_size, s_[b, i]:e_[b, i]] = True
                assert np.array_equal(mask, mask.T)
                for i in range(0, 50, block_size):
                    row_last = min(i + block_size, 50) - 1
                    for j in range(i, 50, block_size):
                        in_range = x_[b, j] <= x_[b, row_last] + np.float32(cutoff)
                        assert np.all(mask[i:i + block_size, j:j + block_size] == in_range)


@pytest.mark.parametrize("cutoff", [0.1, 1.0, 11.0])
@pytest.mark.parametrize("block_size", [1, 3])
def test_transpose_mask_equality(cutoff, block_size):
    # mask == mask_t^T (tests/test_ranges.py:163-190 of the reference).
    rng = np.random.default_rng(13)
    for offset in (-1.0, 0.0, 1.5):
        for gap1, gap2 in ((None, None), (0, 10), (10, 0)):
            x1, x2 = _x_pair(rng, offset, gap1, gap2, (2,))
            start, end = oracle_ranges.make_ranges(cutoff, x1, x2, block_size=block_size, align=True)
            start_t, end_t = oracle_ranges.transpose_ranges(start, end, 50, 55, block_size=block_size)
            assert np.all(start_t >= 0) and np.all(start_t <= end_t) and np.all(end_t <= 50)
            for b in range(2):
                mask = np.zeros((50, 55), dtype=bool)
                mask_t = np.zeros((55, 50), dtype=bool)
                for i in range(start.shape[1]):
                    mask[i * block_size:(i + 1) * block_size, start[b, i]:end[b, i]] = True
                for i in range(start_t.shape[1]):
                    mask_t[i * block_size:(i + 1) * block_size, start_t[b, i]:end_t[b, i]] = True
                assert np.array_equal(mask, mask_t.T)


def test_dense_pattern_and_quirks():
    x1 = np.sort(np.random.default_rng(1).random((2, 50)).astype(np.float32))
    x2 = np.sort(np.random.default_rng(2).random((2, 55)).astype(np.float32))
    for bs in (1, 3):
        start, end = oracle_ranges.make_ranges(None, x1, x2, block_size=bs)
        assert np.all(start == 0) and np.all(end == 55)
        assert start.shape == (2, math.ceil(50 / bs))
        start, end = oracle_ranges.make_ranges(None, x1, block_size=bs)
        assert np.all(start == 0) and np.all(end == 50)
    # fewer points than one block: the symmetric scan never starts and end[0] = block size
    start, end = oracle_ranges.make_ranges(1.0, x1[:, :7], block_size=128)
    assert start.tolist() == [[0], [0]] and end.tolist() == [[128], [128]]
