"""Small helpers shared by the configuration tables and the tests."""
from __future__ import annotations

import itertools
from typing import Any, TypeVar

K = TypeVar("K")
V = TypeVar("V")


def format_dict(d: dict[str, Any]) -> str:
    """``dict(a=1, b=2)`` style rendering (reference: kernel_matmul/util.py:11-13)."""
    return "dict(" + ", ".join(f"{key}={value}" for key, value in d.items()) + ")"


def dict_product(*factors: list[dict[K, V]]) -> list[dict[K, V]]:
    """Cartesian product of lists of dicts, merging one dict per factor.

    Empty factors are skipped; all dicts of one factor must share their keys
    (reference: kernel_matmul/util.py:20-40).
    """
    used = [factor for factor in factors if factor]
    for factor in used:
        keys = set(factor[0])
        for entry in factor[1:]:
            if set(entry) != keys:
                raise ValueError("All dicts in a factor must have the same keys")
    merged = []
    for combination in itertools.product(*used):
        out: dict[K, V] = {}
        for entry in combination:
            out.update(entry)
        merged.append(out)
    return merged


def _lomb_scargle_power(t, y, f_min: float, df: float, num_freqs: int, work_elements: int = 1 << 22):
    """Floating-mean Lomb-Scargle periodogram of (t, y) on the grid f_min + k df, k < num_freqs.

    power(f) = 1 - chi^2(f) / chi^2_0 for the least-squares fit of a cos + b sin + c at frequency
    f, chi^2_0 the residual of the mean alone: what gatspy's ``LombScargleFast().fit(t, y)
    .score_frequency_grid(f_min, df, num_freqs)`` returns (the reference's call,
    kernel_matmul/util.py:106-108), here from the exact trigonometric sums in float64 instead of
    gatspy's FFT extirpolation.  Runs on the tensors' device, a block of frequencies at a time.

    Cost: O(n * num_freqs) float64 sine / cosine pairs (about 1e11 at the caller's own limits of
    1e6 frequencies and n ~ 1e5 points) where gatspy's approximation is O(n log n); agreement with
    gatspy's numbers is not checked anywhere (the package is not available to the tests): the
    contract is the least-squares definition above, which the tests check directly.
    """
    import torch

    t = t.to(torch.float64)
    y = y.to(torch.float64)
    y = y - y.mean()
    yy = (y * y).mean()
    n = t.numel()
    per_block = max(1, work_elements // max(n, 1))
    power = torch.empty(num_freqs, dtype=torch.float64, device=t.device)
    for first in range(0, num_freqs, per_block):
        last = min(first + per_block, num_freqs)
        f = f_min + df * torch.arange(first, last, dtype=torch.float64, device=t.device)
        arg = (2.0 * torch.pi) * f[:, None] * t[None, :]
        s, c = torch.sin(arg), torch.cos(arg)
        s_mean, c_mean = s.mean(dim=1), c.mean(dim=1)
        ys, yc = (s * y).mean(dim=1), (c * y).mean(dim=1)  # the data's own mean is zero
        cc = (c * c).mean(dim=1) - c_mean * c_mean
        ss = (s * s).mean(dim=1) - s_mean * s_mean
        cs = (c * s).mean(dim=1) - c_mean * s_mean
        det = cc * ss - cs * cs
        power[first:last] = (ss * yc * yc + cc * ys * ys - 2.0 * cs * yc * ys) / (yy * det)
    return power


def find_periodogram_peaks(
    x,
    y,
    num_components: int,
    max_frequency: float,
    peak_distance: int = 5,
    peak_oversample: int = 1,
    sum_tasks: bool = True,
    min_num_freqs: int = 10000,
    max_num_freqs: int = 1000000,
):
    """Find peaks in the Lomb-Scargle periodogram of a time series: initial frequencies and
    weights for spectral components (reference: kernel_matmul/util.py:43-142, same arguments,
    frequency grid, peak selection and return shapes).

    Args:
        x: time points ``(n,)``, ascending.
        y: observations ``(n,)`` or ``(n, tasks)``.
        num_components: number of peaks to return.
        max_frequency: upper end of the frequency grid (the lower end is 1 / time span).
        peak_distance: minimum distance between peaks, in grid points.
        peak_oversample: every found peak is returned this many times (slightly jittered).
        sum_tasks: add the tasks' periodograms before looking for peaks.
        min_num_freqs, max_num_freqs: bounds on the grid size ``5 * time span * max_frequency``.

    Returns:
        ``(frequencies, magnitudes)``, float32 on the CPU, each ``(num_components,)`` or, with
        ``sum_tasks=False`` and several tasks, ``(tasks, num_components)``; magnitudes sum to one.

    The periodogram is evaluated from the exact sums on ``x``'s device (the reference goes
    through the ``gatspy`` package's FFT approximation on the CPU, which agrees with the exact
    sums to about 1e-3 of the peak height); peak picking is SciPy's ``find_peaks`` as there.
    """
    import math

    import scipy.signal
    import torch

    single = y.dim() == x.dim()
    if single:
        y = y.unsqueeze(-1)
        sum_tasks = True
    num_tasks = y.shape[-1]

    # frequency grid (kernel_matmul/util.py:84-102 of the reference, in its float32 arithmetic)
    f_max = torch.tensor(float(max_frequency))
    timespan = (x[-1] - x[0]).detach().cpu().to(torch.float32)
    f_min = 1 / timespan
    num_freqs = int(
        torch.ceil(
            torch.clamp(5 * timespan * f_max, min=torch.tensor(min_num_freqs), max=torch.tensor(float(max_num_freqs)))
        ).to(torch.long)
    )
    df = (f_max - f_min) / num_freqs
    freqs = torch.arange(num_freqs) * df + f_min

    pgrams = [
        _lomb_scargle_power(x.detach(), y[..., i].detach(), f_min.item(), df.item(), num_freqs).cpu().numpy()
        for i in range(num_tasks)
    ]
    if sum_tasks:
        pgrams = [sum(pgrams)]

    peak_freqs, peak_mags = [], []
    for pgram in pgrams:
        peaks, _ = scipy.signal.find_peaks(pgram, distance=peak_distance)
        pgram = torch.from_numpy(pgram)
        peaks = torch.from_numpy(peaks)
        # the highest peaks, each repeated peak_oversample times
        num_peaks = int(math.ceil(num_components / peak_oversample))
        best = torch.argsort(-pgram[peaks])[:num_peaks]
        peak_idx = peaks[best].repeat(peak_oversample)[:num_components]
        peak_mag = pgram[peak_idx]
        peak_freq = freqs[peak_idx]
        if peak_oversample > 1:
            # repeated peaks must not start with identical gradients
            peak_freq = peak_freq + torch.rand_like(peak_freq) * df / 10
        peak_mag = peak_mag / torch.sum(peak_mag)
        peak_freqs.append(peak_freq.to(torch.float32))
        peak_mags.append(peak_mag.to(torch.float32))

    if sum_tasks:
        return peak_freqs[0], peak_mags[0]
    return torch.stack(peak_freqs, dim=0), torch.stack(peak_mags, dim=0)
