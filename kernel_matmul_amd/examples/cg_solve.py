"""Conjugate gradients on (K + noise * I) X = B with the on-the-fly kernel matrix.

This is the inner loop of a GP fit as the reference runs it (examples/fit_sine.py:17-67 there:
GPyTorch's marginal log likelihood solves with the KernelMatmulLinearOperator by CG, i.e. by
repeated ``K @ rhs``), written out without GPyTorch: a fixed number of iterations, every
right-hand-side column and every batch item (hyper-parameter set) iterated independently, no
host synchronisation inside the loop.  The iteration body allocates nothing (the operator
writes into a preallocated buffer), so it can be captured once into a HIP graph and replayed.

    python -m kernel_matmul_amd.examples.cg_solve [--n 100000] [--k 16] [--batch 8] [--iterations 30]
"""
from __future__ import annotations

import argparse
import time

import torch
from torch import Tensor

from kernel_matmul_amd import _native
from kernel_matmul_amd.ranges import make_ranges


class ConjugateGradients:
    """Fixed-iteration CG for A = K(x, x) + noise * I, A symmetric positive definite.

    Args:
        kernel_type: "rbf", "spectral" or "locally_periodic".
        x: sorted inputs ``(n,)`` on the GPU.
        params: hyper-parameters ``(batch, P)``.
        cutoff: sparsity cutoff of the symmetric pattern (``make_ranges(cutoff, x)``).
        noise: the diagonal shift (observation noise variance), scalar.
        k: number of right-hand-side columns.
    """

    def __init__(self, kernel_type: str, x: Tensor, params: Tensor, cutoff: float | None, noise: float, k: int):
        self.kernel_type = kernel_type
        batch, n = params.shape[0], x.shape[0]
        # Hyper-parameters, pattern and noise live in buffers of their own, so that a captured
        # iteration keeps reading the current ones after `update`.
        self.points = x
        self.params = params.clone()
        self.range_start, self.range_end = (t.clone() for t in make_ranges(cutoff, x))
        self.noise = torch.full((1,), float(noise), dtype=torch.float32, device=x.device)
        self._op_args = (x.expand(batch, n), x.expand(batch, n), self.params,
                         self.range_start.expand(batch, -1), self.range_end.expand(batch, -1))
        new = lambda *shape: torch.zeros(*shape, dtype=torch.float32, device=x.device)
        self.x = new(batch, n, k)    # iterate
        self.r = new(batch, n, k)    # residual
        self.p = new(batch, n, k)    # search direction
        self.ap = new(batch, n, k)   # A @ p
        self.tmp = new(batch, n, k)
        self.rs = new(batch, 1, k)   # <r, r> per column
        self.rs_new = new(batch, 1, k)
        self.pap = new(batch, 1, k)
        self.alpha = new(batch, 1, k)
        self.beta = new(batch, 1, k)
        self.ones = torch.ones(batch, 1, n, dtype=torch.float32, device=x.device)
        self.graph: torch.cuda.CUDAGraph | None = None

    def _matvec(self, v: Tensor, out: Tensor) -> None:
        x1, x2, params, start, end = self._op_args
        _native.matmul(self.kernel_type, x1, x2, v, params, start, end, out=out)
        out.addcmul_(v, self.noise)

    def _column_dots(self, a: Tensor, b: Tensor, out: Tensor) -> None:
        # per-column inner products as a batched (1 x n) @ (n x k) product
        torch.mul(a, b, out=self.tmp)
        torch.bmm(self.ones, self.tmp, out=out)

    def update(self, params: Tensor, cutoff: float | None, noise) -> None:
        """New hyper-parameters ``(batch, P)``, sparsity cutoff and noise (float or 0-d tensor) for
        the same points: written into the buffers the iterations read, so a captured graph stays
        valid."""
        start, end = make_ranges(cutoff, self.points)
        self.range_start.copy_(start)
        self.range_end.copy_(end)
        self.params.copy_(params)
        if isinstance(noise, Tensor):
            self.noise.copy_(noise.reshape(1))
        else:
            self.noise.fill_(float(noise))

    def start(self, b: Tensor) -> None:
        """x = 0, r = p = b."""
        self.x.zero_()
        self.r.copy_(b)
        self.p.copy_(b)
        self._column_dots(self.r, self.r, self.rs)

    def iteration(self) -> None:
        self._matvec(self.p, self.ap)
        self._column_dots(self.p, self.ap, self.pap)
        torch.div(self.rs, self.pap, out=self.alpha)
        self.alpha.nan_to_num_(nan=0.0, posinf=0.0, neginf=0.0)  # a column that has converged to 0 / 0
        self.x.addcmul_(self.p, self.alpha)
        self.r.addcmul_(self.ap, self.alpha, value=-1.0)
        self._column_dots(self.r, self.r, self.rs_new)
        torch.div(self.rs_new, self.rs, out=self.beta)
        self.beta.nan_to_num_(nan=0.0, posinf=0.0, neginf=0.0)
        self.p.mul_(self.beta).add_(self.r)
        self.rs.copy_(self.rs_new)

    def capture(self) -> None:
        """Capture one iteration into a HIP graph (after a warm-up on a side stream)."""
        saved = [t.clone() for t in (self.x, self.r, self.p, self.rs)]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.iteration()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.iteration()
        self.graph = graph
        for t, s in zip((self.x, self.r, self.p, self.rs), saved):
            t.copy_(s)
        torch.cuda.synchronize()

    def solve(self, b: Tensor, iterations: int, use_graph: bool = False) -> tuple[Tensor, Tensor]:
        """Returns (solution, residual norms per column after the last iteration)."""
        self.start(b)
        if use_graph and self.graph is None:
            self.capture()
            self.start(b)
        for _ in range(iterations):
            if use_graph:
                self.graph.replay()
            else:
                self.iteration()
        return self.x, self.rs.sqrt().squeeze(-2)


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--n", type=int, default=100_000)
    ap.add_argument("--k", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--iterations", type=int, default=30)
    ap.add_argument("--noise", type=float, default=0.5)
    args = ap.parse_args()

    device = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    x = torch.sort(torch.rand(args.n, generator=g) * (args.n / 10.0))[0].to(device)
    u = lambda lo, hi: lo + (hi - lo) * torch.rand(args.batch, generator=g)
    params = torch.stack([u(0.5, 2.0), u(0.05, 0.5), u(0.5, 2.0)], dim=-1).to(device)
    b = torch.randn(args.batch, args.n, args.k, generator=g).to(device)
    cg = ConjugateGradients("spectral", x, params, 6.0 * float(params[:, 0].max()), args.noise, args.k)
    for use_graph in (False, True):
        cg.solve(b, 2, use_graph)  # warm-up (and capture)
        torch.cuda.synchronize()
        begin = time.perf_counter()
        _, res = cg.solve(b, args.iterations, use_graph)
        torch.cuda.synchronize()
        seconds = time.perf_counter() - begin
        rel = (res / b.norm(dim=-2)).max().item()
        print(f"{'graph replay' if use_graph else 'eager':>12}: {args.iterations} iterations in "
              f"{seconds * 1e3:.2f} ms ({seconds * 1e6 / args.iterations:.0f} us per iteration), "
              f"largest relative residual {rel:.2e}")


if __name__ == "__main__":
    main()
