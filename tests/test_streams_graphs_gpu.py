"""The device entry points only enqueue work on the caller's stream: they can run on a side
stream and be captured into a HIP graph and replayed."""
import numpy as np
import pytest
import torch

from kernel_matmul_amd.compile import load_native
from kernel_matmul_amd.configurations import BilinearDerivativeConfiguration, MatmulSingleConfiguration
from kernel_matmul_amd.ranges import make_ranges
from oracle import kernels as oracle

pytestmark = pytest.mark.gpu


def _problem(n=3000, k=16, batch=3):
    g = torch.Generator().manual_seed(21)
    x = torch.sort(torch.rand(n, generator=g) * 100)[0]
    params = torch.stack([0.5 + torch.rand(batch, generator=g), 0.1 + 0.3 * torch.rand(batch, generator=g),
                          0.5 + torch.rand(batch, generator=g)], dim=-1)
    rhs = torch.randn(batch, n, k, generator=g)
    start, end = make_ranges(4.0, x)
    return x, params, rhs, start, end


def test_side_stream():
    x, params, rhs, start, end = _problem()
    dev = torch.device("cuda:0")
    side = torch.cuda.Stream()
    xd, pd, rd = x.to(dev).expand(3, -1), params.to(dev), rhs.to(dev)
    sd, ed = start.to(dev).expand(3, -1), end.to(dev).expand(3, -1)
    args = (xd, xd, rd, pd, sd, ed)
    op = load_native("matmul", MatmulSingleConfiguration("spectral").make_config(args))
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        out = op.call(*args)
    side.synchronize()
    bc = lambda v: np.broadcast_to(v, (3, *v.shape))
    expected = oracle.matmul("spectral", bc(x.numpy()), bc(x.numpy()), rhs.numpy(), params.numpy(),
                             bc(start.numpy()), bc(end.numpy()))
    np.testing.assert_allclose(out.cpu().numpy(), expected, rtol=1e-4, atol=1e-5)


def test_graph_capture_and_replay():
    x, params, rhs, start, end = _problem()
    dev = torch.device("cuda:0")
    xd, pd = x.to(dev).expand(3, -1), params.to(dev)
    sd, ed = start.to(dev).expand(3, -1), end.to(dev).expand(3, -1)
    rhs_static = rhs.to(dev).clone()
    left_static = torch.randn(3, x.shape[0], 4, device=dev)
    args = (xd, xd, rhs_static, pd, sd, ed)
    op = load_native("matmul", MatmulSingleConfiguration("spectral").make_config(args))
    gargs = (xd, xd, left_static, rhs_static[..., :4], pd, sd, ed)
    gop = load_native("bilinear_derivative", BilinearDerivativeConfiguration("spectral").make_config(gargs))

    # warm-up on a side stream as torch asks before capture
    warm = torch.cuda.Stream()
    warm.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(warm):
        op.call(*args)
        gop.call(*gargs)
    torch.cuda.current_stream().wait_stream(warm)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = op.call(*args)
        grad_static = gop.call(*gargs)

    for step in range(4):
        new_rhs = torch.randn_like(rhs_static) * (step + 1)
        rhs_static.copy_(new_rhs)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager_out = op.call(*args)
        eager_grad = gop.call(*gargs)
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager_out), f"replay {step} differs from the eager result"
        assert torch.equal(grad_static, eager_grad), f"replay {step}: gradient differs"
