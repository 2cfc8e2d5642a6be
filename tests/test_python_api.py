"""Host-side logic of the Python surface (no GPU): configurations, NativeFunction selection and
caching, load_native's handling of define dicts, error texts, and the drop-in alias package."""
import pytest
import torch

import kernel_matmul_amd
from kernel_matmul_amd import _native, compile as km_compile, native_function
from kernel_matmul_amd.configurations import (
    BilinearDerivativeConfiguration,
    Configuration,
    DenseBwdConfiguration,
    DenseConfiguration,
    IndexBwdConfiguration,
    IndexConfiguration,
    MatmulAutotuneConfiguration,
    MatmulBwdConfiguration,
    MatmulSingleConfiguration,
)
from kernel_matmul_amd.util import dict_product, format_dict


def _args(batch=(3,), m=300, n=200, k=11, p=3):
    x1 = torch.zeros(*batch, m)
    x2 = torch.zeros(*batch, n)
    rhs = torch.zeros(*batch, n, k)
    params = torch.ones(*batch, p)
    rows = -(-m // 128)
    start = torch.zeros(*batch, rows, dtype=torch.int32)
    end = torch.zeros(*batch, rows, dtype=torch.int32)
    return x1, x2, rhs, params, start, end


def test_block_size_constant():
    assert kernel_matmul_amd._BLOCK_SIZE == 128


def test_dict_product():
    assert dict_product([dict(a=1), dict(a=2)], [dict(b=3)]) == [dict(a=1, b=3), dict(a=2, b=3)]
    assert dict_product([dict(a=1)], []) == [dict(a=1)]
    assert dict_product() == [{}]
    with pytest.raises(ValueError, match="same keys"):
        dict_product([dict(a=1), dict(b=2)])
    assert format_dict(dict(a=1, b=None)) == "dict(a=1, b=None)"


def test_matmul_configurations():
    args = _args()
    single = MatmulSingleConfiguration("spectral").make_config(args)
    assert single["BLOCK_SIZE"] == 128 and single["BATCH_DIM"] == 1
    assert single["MATMUL_K_BLOCK_SIZE"] == 11 and single["MATMUL_COL_BLOCKS"] == 1
    assert "KERNEL_SPECTRAL" in single and single["KERNEL_SPECTRAL"] is None
    assert MatmulSingleConfiguration("spectral").cache_key(args) == "1_11"
    assert MatmulSingleConfiguration("rbf").make_config(_args(k=65, p=2))["MATMUL_K_BLOCK_SIZE"] == 32

    auto = MatmulAutotuneConfiguration("rbf")
    candidates = auto.make_candidates(_args(batch=(), p=2))
    assert len(candidates) == 1  # gfx950 table instead of a search
    assert candidates[0]["BATCH_DIM"] == 0 and "KERNEL_RBF" in candidates[0]
    assert auto.cache_key(_args(batch=(2, 3), k=4, p=2)) == "2_4"
    assert isinstance(auto, Configuration)


def test_other_configurations():
    x1, x2, rhs, params, start, end = _args(p=4)
    out_grad = torch.zeros(3, 300, 11)
    bwd = MatmulBwdConfiguration("locally_periodic")
    cfg = bwd.make_config((x1, x2, rhs, params, start, end, out_grad))
    assert cfg["MATMUL_BWD_THREAD_DIM"] == 16 and cfg["MATMUL_BWD_PER_THREAD"] == 8
    assert "KERNEL_LOCALLY_PERIODIC" in cfg and bwd.cache_key((x1, x2, rhs, params, start, end, out_grad)) == "1"
    assert bwd.make_candidates((x1, x2, rhs, params, start, end, out_grad)) == [cfg]

    bil = BilinearDerivativeConfiguration("rbf").make_config((x1, x2, rhs, rhs, params[..., :2], start, end))
    assert bil["BILINEAR_DERIVATIVE_THREAD_DIM"] == 16 and "KERNEL_RBF" in bil

    idx = torch.zeros(5, 7, dtype=torch.int32)
    iargs = (x1, x2, params[..., :3], start, end, (idx,), idx, idx)
    icfg = IndexConfiguration("spectral").make_config(iargs)
    assert icfg["INDEX_THREAD_DIM"] == 64 and icfg["INDEX_BATCH_DIM"] == 1
    assert IndexConfiguration("spectral").cache_key(iargs) == "1_1"
    bcfg = IndexBwdConfiguration("spectral").make_config((*iargs, idx.float()))
    assert bcfg["INDEX_BWD_THREAD_DIM"] == 64 and bcfg["INDEX_BWD_BATCH_DIM"] == 1
    assert DenseConfiguration("rbf").make_config((x1, x2, params[..., :2], start, end))["DENSE_THREAD_DIM"] == 16
    assert DenseBwdConfiguration("rbf").make_config((x1, x2, params[..., :2], start, end, rhs))["DENSE_BWD_THREAD_DIM"] == 16


class _FakeModule:
    def __init__(self, name, defines):
        self.name, self.defines, self.calls = name, defines, 0

    def call(self, *args):
        self.calls += 1
        return (self.name, self.defines.get("TAG"))


class _TwoCandidates(Configuration):
    def make_candidates(self, args):
        return [dict(TAG="a"), dict(TAG="b")]

    def cache_key(self, args):
        return str(args[0])


def test_native_function_selection_and_cache(monkeypatch):
    loaded = []

    def fake_load(name, defines=None):
        module = _FakeModule(name, defines)
        loaded.append(module)
        return module

    found = []

    def fake_find_best(name, args, candidates, return_timings=False, num_measurements=1, compile_pool=None):
        found.append((name, num_measurements))
        return candidates[1], [2.0, 1.0]

    monkeypatch.setattr(native_function, "load_native", fake_load)
    monkeypatch.setattr(native_function, "find_best", fake_find_best)

    fn = native_function.NativeFunction("matmul", _TwoCandidates(), num_measurements=3, verbose=True)
    assert fn.defines is None
    assert fn(1) == ("matmul", "b")
    assert fn.defines == dict(TAG="b") and found == [("matmul", 3)]
    fn(1)
    assert len(loaded) == 1 and loaded[0].calls == 2  # same cache key: no reselection
    fn(2)
    assert len(loaded) == 2 and len(found) == 2  # key changed: selected again

    single = native_function.NativeFunction("matmul", MatmulSingleConfiguration("rbf"))
    single(*_args(p=2))
    assert len(found) == 2  # one candidate: nothing to time
    assert single.defines["KERNEL_RBF"] is None


def test_load_native_define_handling():
    rbf = {"KERNEL_RBF": None, "BLOCK_SIZE": 128, "BATCH_DIM": 1, "MATMUL_COL_BLOCKS": 4}
    module = km_compile.load_native("matmul", rbf)
    assert module.kernel_type == "rbf" and module._options.col_splits == 4
    assert module.name == "km___matmul___BATCH_DIM__1___BLOCK_SIZE__128___KERNEL_RBF___MATMUL_COL_BLOCKS__4"
    assert km_compile.load_native("matmul", {**rbf, "MATMUL_COL_BLOCKS": 16})._options.col_splits == 8
    assert hasattr(module, "call")
    with pytest.raises(ValueError, match="Unknown native module"):
        km_compile.load_native("nope", rbf)
    with pytest.raises(ValueError, match="No kernel function defined"):
        km_compile.load_native("matmul", {"BLOCK_SIZE": 128})
    with pytest.raises(ValueError, match="BLOCK_SIZE"):
        km_compile.load_native("matmul", {**rbf, "BLOCK_SIZE": 64})
    with pytest.raises(NotImplementedError):
        km_compile.load_native("matmul", {"KERNEL_COMPACT": None, "NUM_ORDERS": 2})


def test_debug_flag_changes_module_name(monkeypatch):
    monkeypatch.setenv("KERNEL_MATMUL_COMPILE_DEBUG", "true")
    module = km_compile.load_native("index", {"KERNEL_SPECTRAL": None})
    assert module.debug and module.name.endswith("___debug")


def test_entry_point_checks_on_cpu_tensors():
    x1, x2, rhs, params, start, end = _args(p=2)
    module = km_compile.load_native("matmul", MatmulSingleConfiguration("rbf").make_config((x1, x2, rhs, params, start, end)))
    with pytest.raises(RuntimeError, match="x must be a CUDA tensor"):
        module.call(x1, x2, rhs, params, start, end)
    with pytest.raises(RuntimeError, match="x must be int32"):
        _native.check_int32(start.long())
    with pytest.raises(RuntimeError, match="expected scalar type Float but found Double"):
        _native.check_float(x1.double())
    wrong_rank = km_compile.load_native("matmul", {"KERNEL_RBF": None, "BATCH_DIM": 0})
    with pytest.raises(RuntimeError, match="batch dimension"):
        wrong_rank.call(x1, x2, rhs, params, start, end)


def test_compile_pool_is_exclusive():
    with km_compile.compile_pool(1):
        with pytest.raises(RuntimeError, match="compile_pool is already active"):
            with km_compile.compile_pool(1):
                pass
    with km_compile.compile_pool(1):
        pass  # can be opened again after closing


def test_alias_package_is_the_same_modules():
    import kernel_matmul
    import kernel_matmul.compile
    import kernel_matmul.native_function
    import kernel_matmul.ranges
    from kernel_matmul.configurations import MatmulAutotuneConfiguration as Aliased

    assert kernel_matmul._BLOCK_SIZE == 128
    assert kernel_matmul.compile is km_compile
    assert kernel_matmul.native_function.NativeFunction is native_function.NativeFunction
    assert Aliased is MatmulAutotuneConfiguration
    with pytest.raises(ModuleNotFoundError):
        import kernel_matmul.does_not_exist  # noqa: F401
