"""Random sweep of matmul and bilinear_derivative against the float64 oracle.

Shapes, batch shapes, coordinate units and offsets (the regimes that decide between the separable
and the direct evaluation), lengthscales, frequencies, signs of the outputscale, cutoffs, sorted
and unsorted coordinates with arbitrary ranges, rhs magnitudes, contraction variants, launch
shapes and memory layouts (a quarter of the tensors are handed over as strided views: transposed,
cut out of a wider tensor, or every second element) are drawn at random; every case is compared
element by element.

Tolerance of the forward result, per element: 1e-5 max|rhs| + 1e-4 |expected| + 2e-6 |K| @ |rhs|
(fp32 evaluation and accumulation), plus, for the oscillating kernels, the fp32 rounding of the
phase f * d: one ulp of the largest phase times the envelope (Gaussian factor alone) @ |rhs| — the
error a product formed in fp32 has, in the reference's kernels as much as here.  Gradients: 1e-4
of the largest component + 8e-6 of sum |coefficient| |dK/dtheta| (twice what the feature form of
the gradient kernels measures against float64) plus, for the oscillating kernels, the same one ulp
of every pair's phase: sum |coefficient| |change of dK/dtheta| when the frequency (the period)
moves by a relative 2^-23, taken from the float64 oracle by a finite difference.
"""
import random

import numpy as np
import pytest
import torch

from kernel_matmul_amd.compile import load_native
from kernel_matmul_amd.configurations import BilinearDerivativeConfiguration, MatmulSingleConfiguration
from kernel_matmul_amd.ranges import make_ranges
from oracle import kernels as oracle
from tests.test_strided_inputs_gpu import column_major, interleaved, padded

pytestmark = pytest.mark.gpu

CASES_PER_SEED = 100


def _draw(rng):
    kt = rng.choice(["rbf", "spectral", "spectral", "locally_periodic"])
    m = rng.choice([1, 17, 127, 128, 129, 300, 640, 1100, 1500])
    square = rng.random() < 0.5
    n = m if square else rng.choice([1, 33, 128, 257, 700, 1300])
    k = rng.choice([1, 2, 4, 5, 8, 11, 16, 17, 32, 33, 64, 70])
    batch = rng.choice([(), (), (2,), (3,), (2, 2)])
    scale = rng.choice([1.0, 1.0, 0.01, 100.0])  # coordinate unit
    shift = rng.choice([0.0, 0.0, 5.0, 100.0, 1e4, -50.0, -3.0]) * scale
    extent = rng.choice([3.0, 10.0, 10.0, 40.0]) * scale
    lfac = rng.choice([1.0, 1.0, 0.3, 3.0, 0.02])
    cutoff = rng.choice([None, 1.0, 2.0, 4.0, 8.0])
    is_sorted = rng.random() < 0.9
    x1 = torch.rand(*batch, m) * extent + shift
    x2 = x1.clone() if square else torch.rand(*batch, n) * extent + shift
    if is_sorted:
        x1 = torch.sort(x1, dim=-1)[0]
        x2 = x1.clone() if square else torch.sort(x2, dim=-1)[0]
    r = lambda: torch.rand(batch)
    if kt == "rbf":
        cols = [(1 + r()) * lfac * scale, (1 + r()) * rng.choice([1, 1, -1])]
    elif kt == "spectral":
        cols = [(1 + r()) * lfac * scale, (0.2 + r() * rng.choice([0.5, 5.0, 50.0])) / scale,
                (1 + r()) * rng.choice([1, 1, -1])]
    else:
        cols = [(1 + r()) * lfac * scale, (1 + r()) * lfac, (1 + r()) * scale, 1 + r()]
    params = torch.stack(cols, dim=-1).float()
    cut = None if cutoff is None else cutoff * lfac * scale * 2
    if is_sorted:
        start, end = make_ranges(cut, x1) if square else make_ranges(cut, x1, x2)
    else:
        rows = (m + 127) // 128
        start = torch.randint(0, max(n // 2, 1), (*batch, rows), dtype=torch.int32)
        width = torch.randint(0, n + 1, (*batch, rows), dtype=torch.int32)
        end = torch.minimum(start + width, torch.tensor(n, dtype=torch.int32))
    rhs = torch.randn(*batch, n, k) * rng.choice([1.0, 1e-3, 1e3])
    variant = rng.choice([None, None, None, "mfma_f16", "mfma_f16_direct", "block", "mfma_f32", "mfma_f32_direct", "valu"])
    rows_per_wave = rng.choice([None, None, 16, 32, 64, 128])
    splits = rng.choice([None, None, 1, 2, 3, 4, 5, 8])
    c = rng.choice([1, 3, 4, 5, 8, 10, 16])
    left, right = torch.randn(*batch, m, c), torch.randn(*batch, n, c)
    return dict(kt=kt, x1=x1, x2=x2, rhs=rhs, params=params, start=start, end=end, variant=variant,
                rows_per_wave=rows_per_wave, splits=splits, left=left, right=right)


def _on_device(d, keys, device, layouts):
    """The tensors of a case on the GPU, some of them as strided views of the same values (drawn
    from a generator of its own, so that the cases themselves do not depend on it)."""
    out = []
    for key in keys:
        t = d[key].to(device)
        if t.numel() > 0 and layouts.random() < 0.25:
            matrix = key in ("rhs", "left", "right")
            t = layouts.choice([column_major, padded, interleaved] if matrix else [padded, interleaved])(t)
        out.append(t)
    return tuple(out)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_cases_against_oracle(seed):
    rng = random.Random(seed)
    torch.manual_seed(seed)
    device = torch.device("cuda:0")
    for case in range(CASES_PER_SEED):
        d = _draw(rng)
        kt = d["kt"]
        what = (seed, case, kt, tuple(d["x1"].shape), tuple(d["rhs"].shape), d["variant"], d["rows_per_wave"],
                d["splits"])
        layouts = random.Random(7919 * seed + case)
        args = _on_device(d, ("x1", "x2", "rhs", "params", "start", "end"), device, layouts)
        defines = MatmulSingleConfiguration(kt).make_config(args)
        if d["variant"]:
            defines["MATMUL_VARIANT"] = d["variant"]
        if d["variant"] != "block":
            if d["rows_per_wave"]:
                defines["MATMUL_ROWS_PER_WAVE"] = d["rows_per_wave"]
            if d["splits"]:
                defines["MATMUL_COL_BLOCKS"] = d["splits"]
        out = load_native("matmul", defines).call(*args).cpu().double().numpy()

        x1, x2, rhs, params, start, end = (d[key].numpy() for key in ("x1", "x2", "rhs", "params", "start", "end"))
        dense = oracle.dense(kt, x1, x2, params, start, end)
        rhs64 = rhs.astype(np.float64)
        expected = dense @ rhs64
        tol = 1e-5 * np.abs(rhs).max() + 1e-4 * np.abs(expected) + 2e-6 * (np.abs(dense) @ np.abs(rhs64))
        if kt != "rbf":
            fmax = float(np.abs(params[..., 1]).max() if kt == "spectral" else (1.0 / np.abs(params[..., 2])).max())
            dmax = float(max(x1.max(), x2.max()) - min(x1.min(), x2.min()))
            envelope_params = np.stack([params[..., 0], params[..., -1]], axis=-1)
            envelope = np.abs(oracle.dense("rbf", x1, x2, envelope_params, start, end)) @ np.abs(rhs64)
            tol = tol + envelope * (2 * np.pi * fmax * dmax * 2.0 ** -23 + 1e-6)
        assert np.all(np.isfinite(out)), what
        assert np.all(np.abs(out - expected) <= tol), (what, float(np.max(np.abs(out - expected) / tol)))

        gargs = _on_device(d, ("x1", "x2", "left", "right", "params", "start", "end"), device, layouts)
        got = load_native("bilinear_derivative", BilinearDerivativeConfiguration(kt).make_config(gargs)).call(*gargs)
        got = got.cpu().double().numpy()
        left, right = d["left"].numpy(), d["right"].numpy()
        expected_g = oracle.param_grad(kt, x1, x2, left, right, params, start, end)
        terms = np.abs(oracle.kernel_matrix_grad(kt, x1, x2, params))
        mask = oracle.range_mask(start, end, x1.shape[-1], x2.shape[-1])
        coeff = np.abs(left.astype(np.float64) @ np.swapaxes(right.astype(np.float64), -1, -2))
        size = np.sum(np.where(mask, coeff, 0.0)[..., None, :, :] * terms, axis=(-2, -1))
        tol_g = 1e-4 * np.abs(expected_g).max(axis=-1, keepdims=True) + 8e-6 * size + 1e-6
        if kt != "rbf":
            eta = 2.0 ** -20
            moved = params.astype(np.float64).copy()
            moved[..., 1 if kt == "spectral" else 2] *= 1.0 + eta
            change = np.abs(oracle.kernel_matrix_grad(kt, x1, x2, moved) - oracle.kernel_matrix_grad(kt, x1, x2, params))
            tol_g = tol_g + np.sum(np.where(mask, coeff, 0.0)[..., None, :, :] * change, axis=(-2, -1)) * (2.0 ** -23 / eta)
        assert np.all(np.isfinite(got)), what
        assert np.all(np.abs(got - expected_g) <= tol_g), (what, float(np.max(np.abs(got - expected_g) / tol_g)))
