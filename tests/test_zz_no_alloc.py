"""The allocation-free entry point km_param_grad_static (static per-GPU device scratch) against
km_param_grad (caller's workspace), both called straight through the C ABI: same kernels, fixed
reduction order, so the results must be bit-identical.  Two calls in a row, the second on a
smaller problem (the shared scratch keeps the first call's contents)."""
import ctypes

import numpy as np
import pytest
import torch

from kernel_matmul_amd import _native
from oracle import kernels as oracle

pytestmark = pytest.mark.gpu


def _i64(values):
    return (ctypes.c_int64 * max(len(values), 1))(*values)


def _problem(kernel_type, n, batch, c, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.sort(torch.rand(n, generator=g) * (n / 10.0))[0]
    cols = {"rbf": 2, "spectral": 3, "locally_periodic": 4}[kernel_type]
    params = 0.5 + torch.rand(batch, cols, generator=g)
    left = torch.randn(batch, n, c, generator=g)
    right = torch.randn(n, c, generator=g)
    rows = -(-n // 128)
    width = 300
    start = torch.clamp(torch.arange(rows, dtype=torch.int32) * 128 - width, min=0)
    end = torch.clamp(torch.arange(rows, dtype=torch.int32) * 128 + 128 + width, max=n)
    dev = torch.device("cuda:0")
    t = dict(x=x.to(dev).expand(batch, n), left=left.to(dev), right=right.to(dev).expand(batch, n, c),
             params=params.to(dev), start=start.to(dev).expand(batch, rows), end=end.to(dev).expand(batch, rows))
    return t


def _call(lib, kernel_type, t, static):
    kid = _native.KERNEL_TYPES[kernel_type]
    batch, n = t["x"].shape
    c = t["left"].shape[-1]
    sizes = _i64([batch])
    grad = torch.full((batch, t["params"].shape[-1]), float("nan"), device=t["x"].device)
    tensor_args = []
    for name in ("x", "x", "left", "right", "params", "start", "end"):
        tensor_args += [ctypes.c_void_p(t[name].data_ptr()), _i64(t[name].stride())]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if static:
        status = lib.km_param_grad_static(kid, 1, sizes, n, n, c, *tensor_args,
                                          ctypes.c_void_p(grad.data_ptr()), stream)
    else:
        need = lib.km_param_grad_workspace_size(kid, 1, sizes, n, n, c)
        assert 0 < need <= 4 << 20
        workspace = torch.empty(need, dtype=torch.uint8, device=t["x"].device)
        status = lib.km_param_grad(kid, 1, sizes, n, n, c, *tensor_args, ctypes.c_void_p(grad.data_ptr()),
                                   ctypes.c_void_p(workspace.data_ptr()), need, stream)
    assert status == 0, lib.km_last_error()
    torch.cuda.synchronize()
    return grad


@pytest.mark.parametrize("kernel_type", ["spectral", "rbf", "locally_periodic"])
def test_static_scratch_matches_workspace_entry_point(kernel_type):
    lib = _native.load_library()
    big = _problem(kernel_type, 20_000, 4, 8, seed=41)
    small = _problem(kernel_type, 3_000, 2, 3, seed=42)
    for t in (big, small):  # two calls in a row, the second smaller
        expected = _call(lib, kernel_type, t, static=False)
        got = _call(lib, kernel_type, t, static=True)
        assert torch.isfinite(got).all()
        assert torch.equal(got, expected), (got, expected)
    # and the small problem against the float64 oracle
    f = lambda v: v.cpu().numpy()
    ref = oracle.param_grad(kernel_type, f(small["x"]), f(small["x"]), f(small["left"]), f(small["right"]),
                            f(small["params"]), f(small["start"]), f(small["end"]))
    err = np.abs(got.cpu().double().numpy() - ref)
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(ref).max(axis=-1, keepdims=True))


def test_static_scratch_rejects_problems_beyond_its_capacity():
    lib = _native.load_library()
    t = _problem("rbf", 2_000, 1, 2, seed=43)
    kid = _native.KERNEL_TYPES["rbf"]
    # 10^6 points x 64 batch items need 8 MiB of partial sums: more than the 4 MiB array
    sizes = _i64([64])
    assert lib.km_param_grad_workspace_size(kid, 1, sizes, 1_000_000, 1_000_000, 2) > 4 << 20
    tensor_args = []
    for name in ("x", "x", "left", "right", "params", "start", "end"):
        tensor_args += [ctypes.c_void_p(t[name].data_ptr()), _i64([0] + list(t[name].stride()[1:]))]
    grad = torch.zeros(64, 2, device=t["x"].device)
    status = lib.km_param_grad_static(kid, 1, sizes, 1_000_000, 1_000_000, 2, *tensor_args,
                                      ctypes.c_void_p(grad.data_ptr()), None)
    assert status == -4 and b"static buffer" in lib.km_last_error()


def test_python_binding_without_allocation():
    """_native.param_grad(out=..., static_scratch=True) writes into the caller's tensor."""
    t = _problem("spectral", 5_000, 3, 4, seed=44)
    expected = _native.param_grad("spectral", t["x"], t["x"], t["left"], t["right"], t["params"], t["start"], t["end"])
    out = torch.empty_like(expected)
    got = _native.param_grad("spectral", t["x"], t["x"], t["left"], t["right"], t["params"], t["start"], t["end"],
                             out=out, static_scratch=True)
    assert got is out and torch.equal(out, expected)


def test_python_binding_orders_static_scratch_calls_across_streams():
    """Two streams in turn: the binding orders each call behind the last one on the GPU's one
    scratch array, so both results equal the workspace entry point's."""
    device = torch.device("cuda:0")
    a = _problem("spectral", 20_000, 3, 4, seed=45)
    b = _problem("rbf", 6_000, 2, 3, seed=46)
    expected = [_native.param_grad(kt, t["x"], t["x"], t["left"], t["right"], t["params"], t["start"], t["end"])
                for kt, t in (("spectral", a), ("rbf", b))]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=device), torch.cuda.Stream(device=device)]
    outs = [torch.empty_like(e) for e in expected]
    for _ in range(3):
        for (kt, t), stream, out in zip((("spectral", a), ("rbf", b)), streams, outs):
            with torch.cuda.stream(stream):
                _native.param_grad(kt, t["x"], t["x"], t["left"], t["right"], t["params"], t["start"], t["end"],
                                   out=out, static_scratch=True)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], expected[0]) and torch.equal(outs[1], expected[1])
