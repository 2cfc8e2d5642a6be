"""find_periodogram_peaks (reference: kernel_matmul/util.py:43-142).  The reference evaluates the
periodogram through the gatspy package, which is not installed here, so its numbers cannot be
compared directly; pinned instead by the reference's own test case
(tests/test_find_periodogram_peaks.py:5-18 there), by explicit least-squares fits (the
definition of the floating-mean periodogram) and by the documented shapes."""
import numpy as np
import torch

from kernel_matmul_amd.util import _lomb_scargle_power, find_periodogram_peaks


def test_two_sinusoids_as_in_the_reference_test():
    x = torch.linspace(0, 1, 1000)
    freq1, freq2 = 2.5, 9
    y = torch.sin(2 * torch.pi * freq1 * x + 0.1) * 5 + torch.sin(2 * torch.pi * freq2 * x + 0.1)
    freqs, mags = find_periodogram_peaks(x, y, 2, 10)
    assert torch.allclose(freqs, torch.tensor([freq1, freq2]), atol=0.1)
    assert freqs.dtype == torch.float32 and mags.dtype == torch.float32
    assert abs(mags.sum().item() - 1.0) < 1e-6 and mags[0] > mags[1]


def test_power_is_the_explained_variance_of_a_least_squares_sinusoid():
    rng = np.random.default_rng(3)
    t = np.sort(rng.uniform(0.0, 7.0, 300))                   # uneven sampling
    y = 1.5 + np.sin(2 * np.pi * 0.8 * t + 0.3) + 0.5 * rng.standard_normal(300)
    f_min, df, count = 0.05, 0.013, 400
    power = _lomb_scargle_power(torch.from_numpy(t), torch.from_numpy(y), f_min, df, count, work_elements=7000).numpy()
    chi0 = np.sum((y - y.mean()) ** 2)
    for k in (0, 1, 57, 58, 199, 399):
        f = f_min + k * df
        design = np.stack([np.cos(2 * np.pi * f * t), np.sin(2 * np.pi * f * t), np.ones_like(t)], axis=1)
        coeff, *_ = np.linalg.lstsq(design, y, rcond=None)
        chi = np.sum((y - design @ coeff) ** 2)
        np.testing.assert_allclose(power[k], 1.0 - chi / chi0, rtol=1e-9, atol=1e-12)
    assert abs((f_min + np.argmax(power) * df) - 0.8) < 2 * df
    assert np.all(power >= -1e-12) and np.all(power <= 1 + 1e-12)


def test_tasks_oversampling_and_grid_size():
    g = torch.Generator().manual_seed(0)
    x = torch.sort(torch.rand(400, generator=g) * 20)[0]
    y = torch.stack([torch.sin(2 * torch.pi * 0.7 * x), torch.sin(2 * torch.pi * 1.9 * x)], dim=-1)
    y = y + 0.1 * torch.randn(400, 2, generator=g)
    freqs, mags = find_periodogram_peaks(x, y, 2, 3.0, min_num_freqs=2000)
    assert freqs.shape == (2,) and sorted(np.round(freqs.numpy(), 1)) == [0.7, 1.9]   # summed periodograms
    per_task_f, per_task_m = find_periodogram_peaks(x, y, 3, 3.0, sum_tasks=False, min_num_freqs=2000)
    assert per_task_f.shape == (2, 3) and per_task_m.shape == (2, 3)
    assert abs(per_task_f[0, 0].item() - 0.7) < 0.02 and abs(per_task_f[1, 0].item() - 1.9) < 0.02
    np.testing.assert_allclose(per_task_m.sum(dim=-1).numpy(), [1.0, 1.0], rtol=1e-6)
    # 4 components from 2 peaks: each returned twice, a fraction of a grid step apart
    over_f, over_m = find_periodogram_peaks(x, y[:, 0], 4, 3.0, peak_oversample=2, min_num_freqs=2000)
    assert over_f.shape == (4,)
    step = (3.0 - 1.0 / (x[-1] - x[0]).item()) / 2000
    assert abs(over_f[0] - over_f[2]) < step and abs(over_f[1] - over_f[3]) < step and over_f[0] != over_f[2]
