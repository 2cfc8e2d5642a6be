"""Device range builders: bit-exact against the C oracle on sorted inputs."""
import numpy as np
import pytest
import torch

from kernel_matmul_amd.ranges import make_ranges
from oracle import ranges as oracle_ranges

pytestmark = pytest.mark.gpu


def _sorted(*shape, scale=10.0, gap_at=None):
    x = torch.sort(torch.rand(*shape) * scale, dim=-1)[0]
    if gap_at is not None:
        x[..., gap_at:] += 20
    return x


@pytest.mark.parametrize("batch", [(), (3,), (2, 3)])
@pytest.mark.parametrize("cutoff", [0.0, 0.1, 1.0, 11.0])
@pytest.mark.parametrize("block_size", [1, 3, 128])
@pytest.mark.parametrize("align", [True, False])
def test_asymmetric_device_matches_oracle(batch, cutoff, block_size, align):
    for n1, n2, offset, gap1, gap2 in [(50, 55, 0.0, None, None), (50, 55, -1.0, 10, None),
                                       (300, 257, 1.5, None, 0), (1000, 1200, 0.0, 400, 700),
                                       (5, 300, 0.0, None, None)]:
        x1 = _sorted(*batch, n1, gap_at=gap1)
        x2 = _sorted(*batch, n2, gap_at=gap2) + offset
        start, end = make_ranges(cutoff, x1.cuda(), x2.cuda(), block_size=block_size, align=align)
        s_ref, e_ref = oracle_ranges.make_ranges(cutoff, x1.numpy(), x2.numpy(), block_size=block_size, align=align)
        assert start.dtype == torch.int32 and start.is_cuda
        np.testing.assert_array_equal(start.cpu().numpy(), s_ref)
        np.testing.assert_array_equal(end.cpu().numpy(), e_ref)


@pytest.mark.parametrize("batch", [(), (3,), (2, 3)])
@pytest.mark.parametrize("cutoff", [0.0, 0.1, 1.0, 11.0])
@pytest.mark.parametrize("block_size", [1, 3, 128])
def test_symmetric_device_matches_oracle(batch, cutoff, block_size):
    for n, gap in [(50, None), (50, 10), (100, 0), (1000, 400), (4096, None), (7, None), (128, None), (129, None)]:
        x = _sorted(*batch, n, gap_at=gap)
        start, end = make_ranges(cutoff, x.cuda(), block_size=block_size)
        s_ref, e_ref = oracle_ranges.make_ranges(cutoff, x.numpy(), block_size=block_size)
        np.testing.assert_array_equal(start.cpu().numpy(), s_ref)
        np.testing.assert_array_equal(end.cpu().numpy(), e_ref)


def test_duplicates_and_large_device():
    x = torch.sort(torch.randint(0, 2000, (2, 200_000)).float() / 7.0, dim=-1)[0]
    for cutoff in [0.0, 0.5, 3.0]:
        start, end = make_ranges(cutoff, x.cuda())
        s_ref, e_ref = oracle_ranges.make_ranges(cutoff, x.numpy())
        np.testing.assert_array_equal(start.cpu().numpy(), s_ref)
        np.testing.assert_array_equal(end.cpu().numpy(), e_ref)
        x2 = x[:, ::3].contiguous() + 0.01
        for align in (False, True):
            start, end = make_ranges(cutoff, x.cuda(), x2.cuda(), align=align)
            s_ref, e_ref = oracle_ranges.make_ranges(cutoff, x.numpy(), x2.numpy(), align=align)
            np.testing.assert_array_equal(start.cpu().numpy(), s_ref)
            np.testing.assert_array_equal(end.cpu().numpy(), e_ref)


@pytest.mark.parametrize("symmetric", [True, False])
def test_unsorted_device_input_with_check(symmetric):
    """Contract of the device builders: sorted input.  With ``check_sorted=True`` (the default) unsorted GPU
    input takes the host scan and so gives the pattern the oracle (the reference's sequential
    scan) gives for the same data; sorted input keeps the device path and the same answer."""
    g = torch.Generator().manual_seed(5)
    x1 = torch.rand(2, 700, generator=g) * 10.0
    x1[0] = torch.sort(x1[0])[0]          # one batch item sorted, one not
    x2 = None if symmetric else torch.rand(2, 650, generator=g) * 10.0
    for cutoff in (0.3, 2.0):
        args = (x1.numpy(),) if symmetric else (x1.numpy(), x2.numpy())
        s_ref, e_ref = oracle_ranges.make_ranges(cutoff, *args)
        dev = (x1.cuda(),) if symmetric else (x1.cuda(), x2.cuda())
        start, end = make_ranges(cutoff, *dev)
        assert start.is_cuda and start.dtype == torch.int32
        np.testing.assert_array_equal(start.cpu().numpy(), s_ref)
        np.testing.assert_array_equal(end.cpu().numpy(), e_ref)
    xs = torch.sort(x1, dim=-1)[0]
    a = make_ranges(1.0, xs.cuda())
    b = make_ranges(1.0, xs.cuda(), check_sorted=False)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
