"""The end-to-end fit (kernel_matmul_amd/examples/fit_sine.py: the workload of the reference's
examples/fit_sine.py:17-67 without GPyTorch).  Checked here: the parameter constraints and the
cutoff rule against hand-computed values; the marginal-likelihood gradient (CG solves + one
bilinear-derivative call) against the same probe-vector estimator evaluated in float64 on the
dense masked matrix; the fitted hyper-parameters against the data's truth; the predictions
against an exact float64 GP on the dense masked matrix at the fitted hyper-parameters."""
import math

import numpy as np
import pytest
import torch

from kernel_matmul_amd.examples import fit_sine
from oracle import kernels as oracle
from oracle import ranges as oracle_ranges


def test_constraints_and_cutoff_rule():
    theta = fit_sine.constrained(fit_sine.initial_raw(0.1, "cpu"))
    softplus0 = math.log(2.0)
    np.testing.assert_allclose(theta.numpy(), [0.505, 0.1, 1e-6 + softplus0, 1e-4 + softplus0], rtol=1e-6)
    far = fit_sine.constrained(torch.tensor([-40.0, -40.0, 40.0, -40.0]))
    np.testing.assert_allclose(far.numpy(), [0.01, 1e-6, 40.0, 1e-4], rtol=1e-5)
    # two-sided tail mass 1e-4 of a unit Gaussian lies beyond 3.8906 standard deviations
    assert abs(fit_sine.cutoff_for(1.0, 1e-4) - 3.8906) < 1e-3
    assert abs(fit_sine.cutoff_for(0.25, 1e-4) - 0.25 * 3.8906) < 1e-3


def _dense_system(x, theta, epsilon):
    """float64 masked K(x, x) + noise I and the pattern it was cut with."""
    cutoff = fit_sine.cutoff_for(float(theta[0]), epsilon)
    start, end = oracle_ranges.make_ranges(cutoff, x)
    k = oracle.dense("spectral", x, x, np.asarray(theta[:3], dtype=np.float64), start, end)
    return k + float(theta[3]) * np.eye(len(x)), start, end


@pytest.mark.gpu
def test_objective_gradient_against_float64_estimator():
    n, t, epsilon = 1500, 3, 1e-4
    device = torch.device("cuda:0")
    train_x, train_y, _, _ = fit_sine.make_data(1700, "cpu", seed=3)
    train_x, train_y = train_x[:n], train_y[:n]
    theta = torch.tensor([0.5, 0.3, 0.8, 0.3])
    probes = torch.randn(n, t, generator=torch.Generator().manual_seed(4))
    grad, data_fit = fit_sine.objective_gradient(train_x.to(device), train_y.to(device), theta.to(device),
                                                 probes.to(device), epsilon, cg_iterations=300)

    x = train_x.numpy()
    a, start, end = _dense_system(x, theta.numpy(), epsilon)
    rhs = np.concatenate([train_y.double().numpy()[:, None], probes.double().numpy()], axis=1)
    solves = np.linalg.solve(a, rhs)
    alpha = solves[:, :1]
    left = np.concatenate([-0.5 * alpha, (0.5 / t) * solves[:, 1:]], axis=1)
    right = np.concatenate([alpha, probes.double().numpy()], axis=1)
    expected = np.concatenate([
        oracle.param_grad("spectral", x, x, left, right, theta[:3].double().numpy(), start, end),
        [np.sum(left * right)],
    ]) / n
    np.testing.assert_allclose(data_fit.item(), (train_y.double().numpy() @ alpha[:, 0]) / n, rtol=1e-4)
    np.testing.assert_allclose(grad.cpu().numpy(), expected, rtol=2e-3, atol=2e-3 * np.abs(expected).max())


@pytest.mark.gpu
def test_fit_recovers_the_sine_and_predictions_match_an_exact_gp():
    device = torch.device("cuda:0")
    train_x, train_y, test_x, test_y = fit_sine.make_data(8000, device, seed=0)
    result = fit_sine.fit(train_x, train_y, iterations=100, seed=0)
    lengthscale, frequency, outputscale, noise = result.theta.tolist()
    print(f"fitted: lengthscale {lengthscale:.3f} frequency {frequency:.4f} outputscale {outputscale:.3f} "
          f"noise sd {math.sqrt(noise):.3f} in {result.seconds:.2f} s")
    # the trace estimate makes the gradient noisy: the frequency ends within one spectral
    # bandwidth of the sine's, where the likelihood is nearly flat; the noise level is sharp
    assert abs(frequency - 0.5) < 1.0 / (2 * math.pi * lengthscale)
    assert lengthscale > 0.8
    assert 0.47 < math.sqrt(noise) < 0.53
    # stationarity in the overall scale of A = K + noise I means y^T A^-1 y = n
    assert abs(result.history[-1] - 1.0) < 0.05

    mean, variance = fit_sine.predict(train_x, train_y, test_x, result.theta)
    rmse = (mean - test_y).square().mean().sqrt().item()
    assert rmse < 0.1

    # exact GP in float64 on the same masked matrices
    theta = result.theta.cpu().double().numpy()
    x, xs = train_x.cpu().numpy(), test_x.cpu().numpy()
    a, _, _ = _dense_system(x, theta, 1e-4)
    cutoff = fit_sine.cutoff_for(float(theta[0]), 1e-4)
    start, end = oracle_ranges.make_ranges(cutoff, xs, x, align=True)
    cross = oracle.dense("spectral", xs, x, theta[:3], start, end)
    solved = np.linalg.solve(a, np.concatenate([train_y.cpu().double().numpy()[:, None], cross.T], axis=1))
    mean_ref = cross @ solved[:, 0]
    variance_ref = theta[2] - np.sum(cross.T * solved[:, 1:], axis=0)
    np.testing.assert_allclose(mean.cpu().numpy(), mean_ref, atol=2e-3)
    np.testing.assert_allclose(variance.cpu().numpy(), variance_ref, atol=2e-3)
