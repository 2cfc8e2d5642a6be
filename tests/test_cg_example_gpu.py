"""The forward operator used the way its callers use it: repeated K @ v inside conjugate
gradients on K + noise I (kernel_matmul_amd/examples/cg_solve.py; the reference's
examples/fit_sine.py:17-67 runs the same loop through GPyTorch).  The iterates are checked
against the same iteration in float64 on the dense masked matrix at a size that affords it;
at n = 100 000 the graph-captured iteration is checked, replay by replay, against the eager one."""
import numpy as np
import pytest
import torch

from kernel_matmul_amd.examples.cg_solve import ConjugateGradients
from oracle import kernels as oracle
from oracle import ranges as oracle_ranges

pytestmark = pytest.mark.gpu


def _setup(n, batch, k, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.sort(torch.rand(n, generator=g) * (n / 10.0))[0]
    u = lambda lo, hi: lo + (hi - lo) * torch.rand(batch, generator=g)
    params = torch.stack([u(0.5, 2.0), u(0.05, 0.5), u(0.5, 2.0)], dim=-1)
    b = torch.randn(batch, n, k, generator=g)
    cutoff = 6.0 * float(params[:, 0].max())
    return x, params, b, cutoff


def _cg_float64(a, b, iterations):
    """Textbook CG per column in float64: a [batch, n, n], b [batch, n, k]."""
    x = np.zeros_like(b)
    r = b.copy()
    p = b.copy()
    rs = np.sum(r * r, axis=-2, keepdims=True)
    for _ in range(iterations):
        ap = a @ p
        alpha = rs / np.sum(p * ap, axis=-2, keepdims=True)
        x += alpha * p
        r -= alpha * ap
        rs_new = np.sum(r * r, axis=-2, keepdims=True)
        p = r + (rs_new / rs) * p
        rs = rs_new
    return x, np.sqrt(rs[:, 0, :])


@pytest.mark.parametrize("use_graph", [False, True])
def test_cg_iterates_match_float64(use_graph):
    n, batch, k, iterations, noise = 3000, 2, 5, 25, 0.5
    x, params, b, cutoff = _setup(n, batch, k, seed=71)
    device = torch.device("cuda:0")
    cg = ConjugateGradients("spectral", x.to(device), params.to(device), cutoff, noise, k)
    sol, res = cg.solve(b.to(device), iterations, use_graph)
    start, end = oracle_ranges.make_ranges(cutoff, x.numpy())
    xb = np.broadcast_to(x.numpy(), (batch, n))
    dense = oracle.dense("spectral", xb, xb, params.numpy(), np.broadcast_to(start, (batch, len(start))),
                         np.broadcast_to(end, (batch, len(end))))
    a = dense + noise * np.eye(n)
    sol_ref, res_ref = _cg_float64(a, b.double().numpy(), iterations)
    b_norm = np.linalg.norm(b.double().numpy(), axis=-2)
    assert np.all(res_ref / b_norm < 1e-2)  # the iteration has converged by three decades or so
    # fp32 CG follows the float64 iterates up to rounding amplified by the conditioning
    err = np.abs(sol.cpu().double().numpy() - sol_ref)
    assert err.max() <= 2e-3 * np.abs(sol_ref).max(), err.max()
    np.testing.assert_allclose(res.cpu().double().numpy() / b_norm, res_ref / b_norm, rtol=0.05, atol=1e-4)
    # and the true residual of the returned iterate
    true_res = np.linalg.norm(b.double().numpy() - a @ sol.cpu().double().numpy(), axis=-2)
    assert np.all(true_res / b_norm < 2e-2)


def test_cg_graph_replays_match_eager_at_full_size():
    n, batch, k, noise = 100_000, 4, 16, 0.5
    x, params, b, cutoff = _setup(n, batch, k, seed=72)
    device = torch.device("cuda:0")
    eager = ConjugateGradients("spectral", x.to(device), params.to(device), cutoff, noise, k)
    graphed = ConjugateGradients("spectral", x.to(device), params.to(device), cutoff, noise, k)
    bd = b.to(device)
    eager.start(bd)
    graphed.start(bd)
    graphed.capture()
    graphed.start(bd)
    first = None
    for step in range(6):
        eager.iteration()
        torch.cuda.synchronize()
        graphed.graph.replay()
        torch.cuda.synchronize()
        # eager work and synchronisations lie between the replays; every replay is compared
        for name in ("x", "r", "p", "rs"):
            assert torch.equal(getattr(graphed, name), getattr(eager, name)), (step, name)
        rel = float((graphed.rs.sqrt().squeeze(-2) / bd.norm(dim=-2)).max())
        first = rel if first is None else first
    assert rel < 0.5 * first  # the residual goes down


def test_update_keeps_a_captured_iteration_valid():
    """New hyper-parameters, cutoff and noise are written into the buffers the captured iteration
    reads: replays after `update` equal a solver built from scratch with the new values."""
    n, batch, k = 4000, 2, 5
    x, params, b, cutoff = _setup(n, batch, k, seed=73)
    device = torch.device("cuda:0")
    xd, bd = x.to(device), b.to(device)
    graphed = ConjugateGradients("spectral", xd, params.to(device), cutoff, 0.5, k)
    before = graphed.solve(bd, 8, use_graph=True)[0].clone()   # captures
    new_params = params * torch.tensor([0.7, 1.3, 1.1])
    new_cutoff = 6.0 * float(new_params[:, 0].max())
    graphed.update(new_params.to(device), new_cutoff, torch.tensor(0.3, device=device))
    fresh = ConjugateGradients("spectral", xd, new_params.to(device), new_cutoff, 0.3, k)
    sol_g, res_g = graphed.solve(bd, 8, use_graph=True)
    sol_f, res_f = fresh.solve(bd, 8, use_graph=False)
    assert torch.equal(sol_g, sol_f) and torch.equal(res_g, res_f)
    assert not torch.allclose(sol_g, before, rtol=1e-2)
