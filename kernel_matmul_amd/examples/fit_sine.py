"""Fit of a Gaussian process with a spectral kernel to a noisy sine, start to end on the
on-the-fly kernel matrix.

The workload of the reference's examples/fit_sine.py:17-67 (8000 sorted points on [0, 10],
y = sin(2 pi 0.5 x) + 0.5 N(0, 1), the middle tenth held out; zero mean, one spectral component
with cutoff from epsilon = 1e-4 and lengthscale in (0.01, 1), Gaussian noise, frequency started
at 0.1, Adam with lr 0.1 for 100 iterations), written out without GPyTorch.  What GPyTorch does
behind ``ExactMarginalLogLikelihood`` for matrices of this size is spelled out here with the
operator's own calls:

* solves with A = K + noise I by conjugate gradients, i.e. repeated ``K @ v``
  (the forward operator) against the targets and a few random probe vectors at once;
* the gradient of the negative log marginal likelihood
      -1/2 alpha^T dK alpha + 1/2 tr(A^-1 dK),   alpha = A^-1 y,
  with the trace replaced by its probe-vector estimate (1/t) sum_i (A^-1 z_i)^T dK z_i:
  both terms are ONE call of ``K._bilinear_derivative(left, right)`` with 1 + t columns;
* predictions through the rectangular operator K(test, train) and, for the variances, solves
  against its dense columns (``to_dense()``).

The trace estimate makes the gradient noisy (10 probe vectors, GPyTorch's default count): noise
level, lengthscale and output scale settle within the 100 iterations, the frequency drifts from
0.1 to within one spectral bandwidth 1 / (2 pi lengthscale) of the sine's 0.5, where the
likelihood is nearly flat (measured on an MI355X: about 1 s for the 100 iterations).

    python -m kernel_matmul_amd.examples.fit_sine [--n 8000] [--iterations 100] [--periodogram-init]
"""
from __future__ import annotations

import argparse
import math
import time
from dataclasses import dataclass

import torch
from torch import Tensor
from torch.nn.functional import softplus

from kernel_matmul_amd.linear_operator import KernelMatmulLinearOperator
from kernel_matmul_amd.ranges import make_ranges

LENGTHSCALE_BOUNDS = (1e-2, 1.0)  # Interval constraint of the reference's example
MIN_NOISE = 1e-4                  # GaussianLikelihood's default lower bound
MIN_POSITIVE = 1e-6               # default constraint of the kernel modules


def constrained(raw: Tensor) -> Tensor:
    """(lengthscale, frequency, outputscale, noise variance) from the four unconstrained
    values: sigmoid into the lengthscale interval, softplus above the lower bounds."""
    lo, hi = LENGTHSCALE_BOUNDS
    return torch.stack([
        lo + (hi - lo) * torch.sigmoid(raw[0]),
        MIN_POSITIVE + softplus(raw[1]),
        MIN_POSITIVE + softplus(raw[2]),
        MIN_NOISE + softplus(raw[3]),
    ])


def initial_raw(frequency: float, device) -> Tensor:
    """All raw values zero except the frequency, which starts at ``frequency``."""
    raw = torch.zeros(4, device=device)
    raw[1] = math.log(math.expm1(frequency - MIN_POSITIVE))
    return raw


def cutoff_for(lengthscale: float, epsilon: float) -> float:
    """Distance beyond which a Gaussian profile of this lengthscale holds a tail mass below
    epsilon (the rule of the kernel modules, kernel_matmul/gpytorch/base.py:59-64 of the reference)."""
    return math.sqrt(2.0) * torch.special.erfinv(torch.tensor(1.0 - epsilon)).item() * lengthscale


def kernel_operator(x1: Tensor, x2: Tensor | None, theta: Tensor, epsilon: float) -> KernelMatmulLinearOperator:
    """Spectral K(x1, x2) (K(x1, x1) if x2 is None) under the epsilon cutoff."""
    cutoff = cutoff_for(theta[0].item(), epsilon)
    if x2 is None:
        start, end = make_ranges(cutoff, x1)
        x2 = x1
        symmetric = True
    else:
        start, end = make_ranges(cutoff, x1, x2, align=True)
        symmetric = False
    return KernelMatmulLinearOperator(x1.unsqueeze(-1), x2.unsqueeze(-1), theta[:3].contiguous(), start, end,
                                      kernel_type="spectral", symmetric=symmetric)


def conjugate_gradients(k: KernelMatmulLinearOperator, noise: Tensor, b: Tensor, iterations: int,
                        tolerance: float = 1e-5) -> Tensor:
    """Solves (K + noise I) X = B column by column (independent step sizes), all columns in one
    ``K @ P`` per iteration.  Columns whose residual has dropped below ``tolerance`` times the
    norm of their right-hand side stop moving (their step is set to zero), so iterations past
    convergence do no harm; no host synchronisation inside the loop."""
    x = torch.zeros_like(b)
    r = b.clone()
    p = b.clone()
    rs = (r * r).sum(dim=-2, keepdim=True)
    floor = rs * tolerance**2
    for _ in range(iterations):
        ap = k @ p + noise * p
        live = rs > floor
        alpha = torch.where(live, rs / (p * ap).sum(dim=-2, keepdim=True), torch.zeros_like(rs))
        x = x + alpha * p
        r = r - alpha * ap
        rs_new = (r * r).sum(dim=-2, keepdim=True)
        p = r + torch.where(live, rs_new / rs, torch.zeros_like(rs)) * p
        rs = torch.where(live, rs_new, rs)
    return x


def objective_gradient(x: Tensor, y: Tensor, theta: Tensor, probes: Tensor, epsilon: float,
                       cg_iterations: int) -> tuple[Tensor, Tensor]:
    """Gradient of -log p(y) / n with respect to (lengthscale, frequency, outputscale, noise
    variance), the trace term estimated with the given probe vectors [n, t]; also returns the
    data-fit term y^T A^-1 y / n."""
    n, t = probes.shape
    k = kernel_operator(x, None, theta, epsilon)
    solves = conjugate_gradients(k, theta[3], torch.cat([y.unsqueeze(-1), probes], dim=-1), cg_iterations)
    alpha = solves[:, :1]
    left = torch.cat([-0.5 * alpha, (0.5 / t) * solves[:, 1:]], dim=-1)
    right = torch.cat([alpha, probes], dim=-1)
    grad_kernel = k._bilinear_derivative(left, right)[2]
    # dA / d(noise) = I: the same bilinear form with the identity in place of dK
    grad_noise = (left * right).sum()
    grad = torch.cat([grad_kernel.reshape(3), grad_noise.reshape(1)]) / n
    return grad, (y * alpha.squeeze(-1)).sum() / n


@dataclass
class Fit:
    theta: Tensor            # lengthscale, frequency, outputscale, noise variance
    history: list            # data-fit term per iteration
    seconds: float


def fit(x: Tensor, y: Tensor, iterations: int = 100, lr: float = 0.1, epsilon: float = 1e-4,
        num_probes: int = 10, cg_iterations: int = 60, initial_frequency: float = 0.1,
        seed: int = 0, progress: bool = False) -> Fit:
    raw = initial_raw(initial_frequency, x.device).requires_grad_(True)
    optimizer = torch.optim.Adam([raw], lr=lr)
    g = torch.Generator(device=x.device).manual_seed(seed)
    history = []
    torch.cuda.synchronize(x.device)
    begin = time.perf_counter()
    for it in range(iterations):
        optimizer.zero_grad()
        theta = constrained(raw)
        probes = torch.randn(x.shape[0], num_probes, device=x.device, generator=g)
        grad, data_fit = objective_gradient(x, y, theta.detach(), probes, epsilon, cg_iterations)
        theta.backward(grad)  # chain rule through the constraints
        optimizer.step()
        history.append(data_fit)
        if progress and (it % 10 == 9 or it == iterations - 1):
            ls, f, os_, nz = constrained(raw.detach()).tolist()
            print(f"iteration {it + 1:4d}: data fit {data_fit.item():.4f}  lengthscale {ls:.3f} "
                  f"frequency {f:.4f} outputscale {os_:.3f} noise {math.sqrt(nz):.3f}", flush=True)
    torch.cuda.synchronize(x.device)
    seconds = time.perf_counter() - begin
    return Fit(constrained(raw.detach()), [h.item() for h in history], seconds)


def predict(train_x: Tensor, train_y: Tensor, test_x: Tensor, theta: Tensor, epsilon: float = 1e-4,
            cg_iterations: int = 100) -> tuple[Tensor, Tensor]:
    """Posterior mean and variance of the latent function at ``test_x``."""
    k = kernel_operator(train_x, None, theta, epsilon)
    cross = kernel_operator(test_x, train_x, theta, epsilon)       # K(test, train)
    alpha = conjugate_gradients(k, theta[3], train_y.unsqueeze(-1), cg_iterations)
    mean = (cross @ alpha).squeeze(-1)
    columns = cross._transpose_nonbatch().to_dense()                 # K(train, test), dense columns
    solved = conjugate_gradients(k, theta[3], columns, cg_iterations)
    variance = theta[2] - (columns * solved).sum(dim=-2)
    return mean, variance


def make_data(n: int, device, seed: int = 0, noise: float = 0.5):
    """The reference example's data: sorted uniform x on [0, 10], a 0.5 Hz sine, Gaussian noise,
    the points from 45 % to 55 % of the index range held out."""
    g = torch.Generator().manual_seed(seed)
    full_x = torch.sort(torch.rand(n, generator=g) * 10)[0]
    full_y = torch.sin((2 * math.pi * 0.5) * full_x)
    noisy = full_y + torch.randn(n, generator=g) * noise
    mask = torch.ones(n, dtype=torch.bool)
    mask[int(0.45 * n):int(0.55 * n)] = False
    to = lambda t: t.to(device)
    return to(full_x[mask]), to(noisy[mask]), to(full_x[~mask]), to(full_y[~mask])


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--n", type=int, default=8000)
    ap.add_argument("--iterations", type=int, default=100)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--periodogram-init", action="store_true",
                    help="start the frequency at the highest Lomb-Scargle peak instead of the reference's 0.1")
    args = ap.parse_args()
    device = torch.device("cuda:0")
    train_x, train_y, test_x, test_y = make_data(args.n, device, args.seed)
    initial_frequency = 0.1
    if args.periodogram_init:
        from kernel_matmul_amd.util import find_periodogram_peaks

        peaks, _ = find_periodogram_peaks(train_x, train_y, 1, max_frequency=5.0)
        initial_frequency = peaks[0].item()
        print(f"Periodogram peak: {initial_frequency:.4f}")
    result = fit(train_x, train_y, iterations=args.iterations, seed=args.seed, progress=True,
                 initial_frequency=initial_frequency)
    ls, f, os_, nz = result.theta.tolist()
    print(f"{args.iterations} iterations in {result.seconds:.2f} s")
    print("Fitted parameters:")
    print(f"Frequency: {f}")
    print(f"Lengthscale: {ls}")
    print(f"Outputscale: {os_}")
    print(f"Noise: {math.sqrt(nz)}")
    mean, variance = predict(train_x, train_y, test_x, result.theta)
    sd = variance.clamp_min(0).sqrt()
    inside = ((test_y > mean - 2 * sd) & (test_y < mean + 2 * sd)).float().mean().item()
    rmse = (mean - test_y).square().mean().sqrt().item()
    print(f"Held-out points: rmse against the noise-free sine {rmse:.4f}, "
          f"{100 * inside:.1f} % inside the two-sigma band (mean width {4 * sd.mean().item():.3f})")


if __name__ == "__main__":
    main()
