"""Parity at the full sizes of the benchmark configurations through properties that do not need a dense oracle:
oracle on sampled row blocks, linearity in rhs, symmetry of the bilinear form, agreement of the
three contraction variants, d/d(outputscale) identity, index lookups against per-entry closed
forms, and bit-exact device ranges at n = 10^6."""
import zlib

import numpy as np
import pytest
import torch

from kernel_matmul_amd.compile import load_native
from kernel_matmul_amd.configurations import (
    BilinearDerivativeConfiguration,
    IndexConfiguration,
    MatmulBwdConfiguration,
    MatmulSingleConfiguration,
)
from kernel_matmul_amd.ranges import make_ranges
from oracle import kernels as oracle
from oracle import ranges as oracle_ranges

pytestmark = pytest.mark.gpu

CONFIGS = {
    # name: kernel, n, extent (None = cumulative Exp(1) gaps), batch, k, cutoff factor
    "c2": ("spectral", 20_000, 2000.0, 4, 16, 6.0),
    "c3": ("spectral", 50_000, None, 2, 8, 6.0),
    "c3_rbf": ("rbf", 50_000, None, 2, 8, 6.0),
    "c4": ("spectral", 100_000, 10_000.0, 16, 4, 6.0),
    "headline": ("spectral", 100_000, 10_000.0, 8, 16, 6.0),
    "c5": ("spectral", 1_000_000, 100_000.0, 8, 32, 5.0),
}


def _build(name):
    kernel, n, extent, batch, k, cf = CONFIGS[name]
    g = torch.Generator().manual_seed(zlib.crc32(name.encode()) % 1000 + 2000)
    if extent is None:
        x = torch.cumsum(-torch.log1p(-torch.rand(n, generator=g)), dim=0)
    else:
        x = torch.sort(torch.rand(n, generator=g) * extent)[0]
    u = lambda lo, hi: lo + (hi - lo) * torch.rand(batch, generator=g)
    if kernel == "spectral":
        params = torch.stack([u(0.5, 2.0), u(0.05, 0.5), u(0.5, 2.0)], dim=-1)
    else:
        params = torch.stack([u(0.5, 2.0), u(0.5, 2.0)], dim=-1)
    rhs = torch.randn(n, k, generator=g)
    cutoff = cf * float(params[:, 0].max())
    device = torch.device("cuda:0")
    xd = x.to(device)
    start, end = make_ranges(cutoff, xd)
    rows = start.shape[-1]
    args = dict(
        x=xd.expand(batch, n), rhs=rhs.to(device).expand(batch, n, k), params=params.to(device),
        start=start.expand(batch, rows), end=end.expand(batch, rows),
    )
    host = dict(x=x.numpy(), rhs=rhs.numpy(), params=params.numpy(), start=start.cpu().numpy(),
                end=end.cpu().numpy(), cutoff=cutoff)
    return kernel, n, batch, k, args, host


def _banded_matmul_oracle(kernel, h, rhs, batch_items=None):
    """float64 K @ rhs over the whole pattern, one row block at a time (K never larger than
    128 x window); rhs is [n, k] shared by the batch or [batch, n, k].  Returns [batch, n, k]."""
    params = h["params"] if batch_items is None else h["params"][batch_items]
    nb = params.shape[0]
    x = h["x"]
    n = x.shape[0]
    rhs = np.asarray(rhs, dtype=np.float64)
    if rhs.ndim == 3 and batch_items is not None:
        rhs = rhs[batch_items]
    out = np.zeros((nb, n, rhs.shape[-1]))
    for blk in range(len(h["start"])):
        r0, r1 = blk * 128, min(blk * 128 + 128, n)
        s, e = int(h["start"][blk]), min(int(h["end"][blk]), n)
        if s >= e:
            continue
        kb = oracle.kernel_matrix(kernel, np.broadcast_to(x[r0:r1], (nb, r1 - r0)),
                                  np.broadcast_to(x[s:e], (nb, e - s)), params)
        seg = rhs[s:e] if rhs.ndim == 2 else rhs[:, s:e]
        out[:, r0:r1] = kb @ seg
    return out


_FORWARD_ORACLE_CACHE = {}


def _forward_oracle(name, kernel, h):
    """Banded oracle of the configuration's own rhs, computed once per test session (_build is
    deterministic per name)."""
    if name not in _FORWARD_ORACLE_CACHE:
        _FORWARD_ORACLE_CACHE[name] = _banded_matmul_oracle(kernel, h, h["rhs"])
    return _FORWARD_ORACLE_CACHE[name]


def _banded_param_grad_oracle(kernel, h, left, right, batch_items):
    """float64 gradient of sum((left @ right^T) * masked K) w.r.t. the parameters for the chosen
    batch items, one row block at a time.  left is [batch, n, c], right [n, c] (shared)."""
    params = h["params"][batch_items]
    nb = params.shape[0]
    x = h["x"]
    n = x.shape[0]
    right = np.asarray(right, dtype=np.float64)
    left = np.asarray(left[batch_items], dtype=np.float64)
    grad = np.zeros((nb, params.shape[-1]))
    for blk in range(len(h["start"])):
        r0, r1 = blk * 128, min(blk * 128 + 128, n)
        s, e = int(h["start"][blk]), min(int(h["end"][blk]), n)
        if s >= e:
            continue
        g = oracle.kernel_matrix_grad(kernel, np.broadcast_to(x[r0:r1], (nb, r1 - r0)),
                                      np.broadcast_to(x[s:e], (nb, e - s)), params)
        coeff = left[:, r0:r1] @ right[s:e].T
        grad += np.einsum("bij,bpij->bp", coeff, g)
    return grad


def _matmul(kernel, a, rhs=None, variant=None):
    rhs = a["rhs"] if rhs is None else rhs
    op_args = (a["x"], a["x"], rhs, a["params"], a["start"], a["end"])
    defines = MatmulSingleConfiguration(kernel).make_config(op_args)
    if variant:
        defines["MATMUL_VARIANT"] = variant
    return load_native("matmul", defines).call(*op_args)


@pytest.mark.parametrize("name,variant", [("c3_rbf", None), ("c5", None), ("c3_rbf", "block"), ("c5", "block")])
def test_forward_sampled_blocks_against_oracle(name, variant):
    kernel, n, batch, k, a, h = _build(name)
    out = _matmul(kernel, a, variant=variant)
    assert out.shape == (batch, n, k)
    # first / last blocks, the last 16 row blocks (where the launch cuts items into 16-row
    # pieces) and a random sample
    nblk = len(h["start"])
    blocks = np.unique(np.concatenate([[0, 1], np.arange(max(nblk - 16, 0), nblk),
                                       np.random.default_rng(1).integers(0, nblk, 48)]))
    for blk in blocks:
        r0, r1 = blk * 128, min(blk * 128 + 128, n)
        s, e = int(h["start"][blk]), int(h["end"][blk])
        x1 = np.broadcast_to(h["x"][r0:r1], (batch, r1 - r0))
        x2 = np.broadcast_to(h["x"][s:e], (batch, e - s))
        rhs = np.broadcast_to(h["rhs"][s:e], (batch, e - s, k))
        full = np.zeros((batch, 1), dtype=np.int64)
        expected = oracle.matmul(kernel, x1, x2, rhs, h["params"], full, full + (e - s))
        got = out[:, r0:r1].cpu().double().numpy()
        err = np.abs(got - expected)
        assert np.all(err <= 1e-5 + 1e-4 * np.abs(expected)), (name, blk, err.max())


@pytest.mark.parametrize("name,variant", [("c2", None), ("c3", None), ("headline", None), ("headline", "block"),
                                          ("headline", "mfma_f32")])
def test_forward_every_row_block_against_oracle(name, variant):
    """Every output element of every batch item against the banded float64 oracle."""
    kernel, n, batch, k, a, h = _build(name)
    out = _matmul(kernel, a, variant=variant).cpu().double().numpy()
    expected = _forward_oracle(name, kernel, h)
    err = np.abs(out - expected)
    tol = 1e-5 + 1e-4 * np.abs(expected)
    worst = np.unravel_index(np.argmax(err - tol), err.shape)
    assert np.all(err <= tol), (name, variant, worst, err[worst], expected[worst])


@pytest.mark.parametrize("variant", [None, "mfma_f32"])
def test_c5_every_row_block_of_two_batch_items_against_oracle(variant):
    """Benchmark configuration 5 (n = 10^6, 32 rhs columns: the table kernels with two groups of
    rhs columns): every output element of two of the eight batch items against the banded
    float64 oracle."""
    kernel, n, batch, k, a, h = _build("c5")
    items = np.array([1, 6])
    out = _matmul(kernel, a, variant=variant)[items].cpu().double().numpy()
    key = ("c5", tuple(items))
    if key not in _FORWARD_ORACLE_CACHE:
        _FORWARD_ORACLE_CACHE[key] = _banded_matmul_oracle(kernel, h, h["rhs"], batch_items=items)
    expected = _FORWARD_ORACLE_CACHE[key]
    err = np.abs(out - expected)
    tol = 1e-5 + 1e-4 * np.abs(expected)
    worst = np.unravel_index(np.argmax(err - tol), err.shape)
    assert np.all(err <= tol), (variant, worst, err[worst], expected[worst])


@pytest.mark.parametrize("name,group_tail,halves,rows", [
    ("headline", 0, None, 128), ("headline", 97, None, 128), ("headline", 97, 0, 128), ("headline", 97, 97, 128),
    ("headline", 10_000, None, 128), ("headline", 10_000, 0, 128), ("c2", 5, None, 128), ("c2", 5, 5, 128),
    ("c3_rbf", 3, 2, 128),
    # 64-row items (mid-size launches): none, some, the usual remainder and all of them split
    ("c2", 0, None, 64), ("c2", 29, None, 64), ("c2", 10_000, None, 64), ("c3", 68, None, 64), ("c3_rbf", 7, None, 64)])
def test_forward_grouped_launch_against_oracle(name, group_tail, halves, rows):
    """Workgroups of four wavefronts: full items one per wavefront, the last `group_tail` items of
    every XCD split by columns between the four wavefronts of a workgroup (fixed-order sum), the
    last `halves` of them (default: a quarter) also into two workgroups of 64 rows each.  With 64
    rows per wavefront the items are 64-row chunks (no halves)."""
    kernel, n, batch, k, a, h = _build(name)
    op_args = (a["x"], a["x"], a["rhs"], a["params"], a["start"], a["end"])
    defines = MatmulSingleConfiguration(kernel).make_config(op_args)
    defines["MATMUL_VARIANT"] = "mfma_f16"
    defines["MATMUL_ROWS_PER_WAVE"] = rows
    defines["MATMUL_GROUP_TAIL"] = group_tail
    if halves is not None:
        defines["MATMUL_GROUP_TAIL_HALVES"] = halves
    op = load_native("matmul", defines)
    assert ("grouped64" if rows == 64 else "grouped<") in op.describe(*op_args)
    out = load_native("matmul", defines).call(*op_args)
    again = load_native("matmul", defines).call(*op_args)
    assert torch.equal(out, again)  # fixed reduction order: reproducible
    expected = _forward_oracle(name, kernel, h)
    err = np.abs(out.cpu().double().numpy() - expected)
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(expected)), (name, group_tail, halves, err.max())


@pytest.mark.parametrize("rows_per_wave", [None, 64])
def test_forward_grouped_launches_with_a_batch_shape_that_does_not_collapse(rows_per_wave):
    """The grouped launches (the launch table's choice at this size, and the 64-row one) with two
    batch dimensions whose strides do not merge (rhs is a slice of a larger tensor): the kernels'
    general batch addressing instead of the one-stride short cut, every element against the
    banded oracle."""
    kernel, n, batch, k, a, h = _build("c3")
    device = a["x"].device
    g = torch.Generator().manual_seed(9)
    big = torch.randn(2, 3, n, k, generator=g).to(device)
    rhs = big[:, :2]                                   # [2, 2, n, k], batch strides (3nk, nk)
    params = torch.stack([a["params"], a["params"].flip(0) * 1.1], dim=0)   # [2, 2, 3]
    rows = a["start"].shape[-1]
    expand = lambda t, *tail: t.expand(2, 2, *tail)
    op_args = (expand(a["x"][0], n), expand(a["x"][0], n), rhs, params,
               expand(a["start"][0], rows), expand(a["end"][0], rows))
    defines = MatmulSingleConfiguration(kernel).make_config(op_args)
    if rows_per_wave:
        defines["MATMUL_ROWS_PER_WAVE"] = rows_per_wave
        defines["MATMUL_GROUP_TAIL"] = 7
    op = load_native("matmul", defines)
    assert ("grouped64" if rows_per_wave else "grouped<") in op.describe(*op_args)
    out = op.call(*op_args).cpu().double().numpy().reshape(4, n, k)
    h4 = dict(h, params=params.cpu().numpy().reshape(4, 3))
    expected = _banded_matmul_oracle(kernel, h4, rhs.cpu().numpy().reshape(4, n, k))
    err = np.abs(out - expected)
    assert np.all(err <= 1e-5 + 1e-4 * np.abs(expected)), err.max()


def test_split_fp16_error_against_fp32_mfma_on_headline():
    """How much accuracy the split-fp16 contraction (the default) trades against the fp32 MFMA
    contraction, over the full headline output, each against the float64 oracle.  Both must
    meet rtol 1e-4 / atol 1e-5; the default may be at most 4x worse than the fp32 contraction
    in worst-case absolute error."""
    kernel, n, batch, k, a, h = _build("headline")
    expected = _forward_oracle("headline", kernel, h)
    errs = {}
    for variant in (None, "mfma_f32"):
        out = _matmul(kernel, a, variant=variant).cpu().double().numpy()
        err = np.abs(out - expected)
        assert np.all(err <= 1e-5 + 1e-4 * np.abs(expected)), variant
        errs[variant or "auto"] = (err.max(), (err / (np.abs(expected) + 1e-3)).max())
    print("max abs / max rel(|expected| + 1e-3) error vs float64:", errs)
    assert errs["auto"][0] <= 4 * errs["mfma_f32"][0] + 1e-6


def test_c3_rhs_and_param_gradients_through_the_operator():
    """Benchmark configuration 3 asks for the gradients w.r.t. the hyper-parameters and rhs given
    grad_out [50000, 8]: autograd through KernelMatmulLinearOperator, every element of the rhs
    gradient and the full parameter gradient against the banded float64 oracle."""
    from kernel_matmul_amd.linear_operator import KernelMatmulLinearOperator

    for name in ("c3", "c3_rbf"):
        kernel, n, batch, k, a, h = _build(name)
        device = a["x"].device
        params = a["params"].clone().requires_grad_(True)
        rhs = a["rhs"][0].clone().requires_grad_(True)  # one [n, k] leaf shared by the batch
        op = KernelMatmulLinearOperator(a["x"][0].unsqueeze(-1), a["x"][0].unsqueeze(-1), params,
                                        a["start"][0], a["end"][0], kernel_type=kernel, symmetric=True)
        g = torch.Generator().manual_seed(5)
        grad_out = torch.randn(batch, n, k, generator=g).to(device)
        out = op._matmul(rhs)
        assert out.shape == (batch, n, k)
        (out * grad_out).sum().backward()
        # d/d rhs = sum_b K_b^T G_b; the pattern and K are symmetric
        expected_rhs = _banded_matmul_oracle(kernel, h, grad_out.cpu().numpy()).sum(axis=0)
        bound = _banded_matmul_oracle(kernel, h, np.abs(grad_out.cpu().numpy())).sum(axis=0)
        err = np.abs(rhs.grad.cpu().double().numpy() - expected_rhs)
        assert np.all(err <= 1e-5 + 1e-4 * np.abs(expected_rhs) + 1e-6 * np.abs(bound)), (name, err.max())
        expected_params = _banded_param_grad_oracle(kernel, h, grad_out.cpu().numpy(), h["rhs"], np.arange(batch))
        tol = 1e-5 + 1e-4 * np.abs(expected_params).max(axis=-1, keepdims=True)
        perr = np.abs(params.grad.cpu().double().numpy() - expected_params)
        assert np.all(perr <= tol), (name, params.grad, expected_params)


def test_c4_bilinear_derivative_against_oracle():
    """Benchmark configuration 4: bilinear derivative, spectral, n = 100000, batch 16, 4 vector
    columns; the full sums of all sixteen batch items against the banded float64 oracle."""
    kernel, n, batch, k, a, h = _build("c4")
    g = torch.Generator().manual_seed(6)
    left = torch.randn(batch, n, k, generator=g).to(a["x"].device)
    args = (a["x"], a["x"], left, a["rhs"], a["params"], a["start"], a["end"])
    got = load_native("bilinear_derivative",
                      BilinearDerivativeConfiguration(kernel).make_config(args)).call(*args)
    assert got.shape == (batch, 3)
    items = np.arange(batch)
    expected = _banded_param_grad_oracle(kernel, h, left.cpu().numpy(), h["rhs"], items)
    tol = 1e-5 + 1e-4 * np.abs(expected).max(axis=-1, keepdims=True)
    err = np.abs(got.cpu().double().numpy()[items] - expected)
    assert np.all(err <= tol), (got.cpu().numpy()[items], expected)


@pytest.mark.parametrize("name", ["headline", "c5"])
def test_forward_linearity_symmetry_and_variants(name):
    kernel, n, batch, k, a, h = _build(name)
    out = _matmul(kernel, a)
    scale = out.abs().mean()

    # linear in rhs
    g = torch.Generator().manual_seed(3)
    other = torch.randn(n, k, generator=g).to(out.device).expand(batch, n, k)
    mixed = _matmul(kernel, a, rhs=1.5 * a["rhs"] - 0.25 * other)
    expected = 1.5 * out - 0.25 * _matmul(kernel, a, rhs=other)
    assert torch.allclose(mixed, expected, rtol=1e-4, atol=float(1e-4 * scale))

    # K is symmetric on the symmetric pattern: <u, K v> == <v, K u>
    lhs = (other * out).double().sum(dim=(-2, -1))
    rhs_side = (a["rhs"] * _matmul(kernel, a, rhs=other)).double().sum(dim=(-2, -1))
    denom = (other.double().norm() * out.double().norm() / batch**0.5)
    assert torch.all((lhs - rhs_side).abs() <= 1e-5 * denom)

    # the three contraction variants agree
    for variant in ("mfma_f32", "valu"):
        alt = _matmul(kernel, a, variant=variant)
        assert torch.allclose(alt, out, rtol=1e-4, atol=float(1e-4 * scale)), variant


@pytest.mark.parametrize("name", ["c3", "c3_rbf", "c4", "headline"])
def test_param_grad_identities(name):
    kernel, n, batch, k, a, h = _build(name)
    g = torch.Generator().manual_seed(4)
    grad_out = torch.randn(batch, n, k, generator=g).to(a["x"].device)
    bwd_args = (a["x"], a["x"], a["rhs"], a["params"], a["start"], a["end"], grad_out)
    bwd = load_native("matmul_bwd", MatmulBwdConfiguration(kernel).make_config(bwd_args)).call(*bwd_args)
    bil_args = (a["x"], a["x"], grad_out, a["rhs"], a["params"], a["start"], a["end"])
    bil = load_native("bilinear_derivative",
                      BilinearDerivativeConfiguration(kernel).make_config(bil_args)).call(*bil_args)
    assert torch.equal(bwd, bil)  # same sum, same kernel, fixed reduction order
    again = load_native("matmul_bwd", MatmulBwdConfiguration(kernel).make_config(bwd_args)).call(*bwd_args)
    assert torch.equal(bwd, again)  # run-to-run reproducible

    # d/d(outputscale) = <grad_out, K rhs> / outputscale
    out = _matmul(kernel, a)
    expected = (grad_out.double() * out.double()).sum(dim=(-2, -1)) / a["params"][:, -1].double()
    ref_scale = (grad_out.double().norm(dim=(-2, -1)) * out.double().norm(dim=(-2, -1))) / a["params"][:, -1].double()
    assert torch.all((bwd[:, -1].double() - expected).abs() <= 1e-5 * ref_scale + 1e-4 * expected.abs())

    # oracle on a sub-problem: the rows of a few row blocks only
    nblk = len(h["start"])
    for blk in (0, nblk // 2, nblk - 1):
        r0, r1 = blk * 128, min(blk * 128 + 128, n)
        s, e = int(h["start"][blk]), int(h["end"][blk])
        sub = dict(x1=a["x"][:, r0:r1], left=grad_out[:, r0:r1])
        zeros = torch.zeros(batch, 1, dtype=torch.int32, device=a["x"].device)
        sub_args = (sub["x1"], a["x"][:, s:e], sub["left"], a["rhs"][:, s:e], a["params"], zeros, zeros + (e - s))
        got = load_native("bilinear_derivative",
                          BilinearDerivativeConfiguration(kernel).make_config(sub_args)).call(*sub_args)
        expected = oracle.param_grad(
            kernel, np.broadcast_to(h["x"][r0:r1], (batch, r1 - r0)), np.broadcast_to(h["x"][s:e], (batch, e - s)),
            grad_out[:, r0:r1].cpu().numpy(), np.broadcast_to(h["rhs"][s:e], (batch, e - s, k)), h["params"],
            np.zeros((batch, 1), dtype=np.int64), np.full((batch, 1), e - s))
        tol = 1e-5 + 1e-4 * np.abs(expected).max(axis=-1, keepdims=True)
        assert np.all(np.abs(got.cpu().double().numpy() - expected) <= tol), (name, blk)


def test_index_rows_at_full_size():
    kernel, n, batch, k, a, h = _build("c5")
    rng = np.random.default_rng(9)
    rows = rng.integers(0, n, 4096)
    delta = rng.integers(-600, 600, 4096)
    cols = np.clip(rows + delta, 0, n - 1)
    bi = rng.integers(0, batch, 4096)
    device = a["x"].device
    t = lambda v: torch.from_numpy(v.astype(np.int32)).to(device)
    args = (a["x"], a["x"], a["params"], a["start"], a["end"], (t(bi),), t(rows), t(cols))
    got = load_native("index", IndexConfiguration(kernel).make_config(args)).call(*args)
    blk = rows // 128
    inside = (cols >= h["start"][blk]) & (cols < h["end"][blk])
    assert 0 < inside.sum() < 4096
    x = h["x"].astype(np.float64)
    p = h["params"].astype(np.float64)[bi]
    d = x[rows] - x[cols]
    expected = np.where(inside, p[:, 2] * np.exp(-d * d / (2 * p[:, 0] ** 2)) * np.cos(2 * np.pi * p[:, 1] * d), 0.0)
    np.testing.assert_allclose(got.cpu().double().numpy(), expected, rtol=1e-4, atol=1e-5)
    assert torch.all(got[torch.from_numpy(~inside).to(device)] == 0)


def test_ranges_at_full_size_bit_exact():
    _, n, _, _, a, h = _build("c5")
    s_ref, e_ref = oracle_ranges.make_ranges(h["cutoff"], h["x"])
    np.testing.assert_array_equal(h["start"], s_ref)
    np.testing.assert_array_equal(h["end"], e_ref)
    x_cpu = torch.from_numpy(h["x"])
    s_host, e_host = make_ranges(h["cutoff"], x_cpu)
    np.testing.assert_array_equal(s_host.numpy(), s_ref)
    x2 = x_cpu[::2].contiguous() + 0.003
    for align in (False, True):
        s_dev, e_dev = make_ranges(h["cutoff"], x_cpu.cuda(), x2.cuda(), align=align)
        s_o, e_o = oracle_ranges.make_ranges(h["cutoff"], h["x"], x2.numpy(), align=align)
        np.testing.assert_array_equal(s_dev.cpu().numpy(), s_o)
        np.testing.assert_array_equal(e_dev.cpu().numpy(), e_o)


def test_c1_dense_check():
    """Benchmark configuration 1 (the reference's CPU-runnable case): rbf, n = 4096, k = 1, l = sigma = 1,
    cutoff 8, checked against the full dense float64 product on the CPU."""
    n = 4096
    g = torch.Generator().manual_seed(1001)
    x = torch.sort(torch.rand(n, generator=g) * 100.0)[0]
    rhs = torch.randn(n, 1, generator=g)
    params = torch.tensor([1.0, 1.0])
    device = torch.device("cuda:0")
    xd = x.to(device)
    start, end = make_ranges(8.0, xd)
    args = (xd, xd, rhs.to(device), params.to(device), start, end)
    for variant in (None, "block", "mfma_f32", "valu"):
        defines = MatmulSingleConfiguration("rbf").make_config(args)
        if variant:
            defines["MATMUL_VARIANT"] = variant
        out = load_native("matmul", defines).call(*args)
        expected = oracle.matmul("rbf", x.numpy(), x.numpy(), rhs.numpy(), params.numpy(),
                                 start.cpu().numpy(), end.cpu().numpy())
        err = np.abs(out.cpu().double().numpy() - expected)
        assert np.all(err <= 1e-5 + 1e-4 * np.abs(expected)), (variant, err.max())
        # cutoff 8 l: what the band leaves out is below exp(-32) per entry
        dense = oracle.kernel_matrix("rbf", x.numpy(), x.numpy(), params.numpy()) @ rhs.double().numpy()
        assert np.abs(out.cpu().double().numpy() - dense).max() < 2e-5
