"""Variant search, host side: enumeration order, seeded random search, ranking, failed trials,
and the search spaces the functions of the path publish (reference tuning/my_autograd_func_tuner.py:14-68,
layers_and_funcs/utils.py:61-118)."""
import pytest
import torch

from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.sputnik import MySpMM, SPMM_KERNELS, spmm_kernel_choices
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.torch import GEMM_TILES, MyLinear
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.utils import MyAutogradFunc, TunableItemCfg
from intrasm_engine_amd.pytorch.horizontal_rewriter import make_kernel_pair_or_triple_autograd_function
from intrasm_engine_amd.pytorch import ops
from intrasm_engine_amd.tuning.my_autograd_func_tuner import (
    GridSearchTuner,
    RandomSearchTuner,
    tune_my_autograd_function,
)

SPACE = {"a": TunableItemCfg("choice", [1, 2, 3]), "b": TunableItemCfg("choice", ["x", "y"])}


def _cost(_, p):
    return {"x": 10.0, "y": 5.0}[p["b"]] + abs(p["a"] - 2)


def test_grid_search_visits_every_point_in_row_major_order():
    seen = []
    tuner = GridSearchTuner(SPACE, lambda i, p: (seen.append((i, dict(p))), _cost(i, p))[1], max_trials=100)
    assert tuner.size() == 6
    assert tuner.tune() == {"a": 2, "b": "y"} and tuner.best_latency == 5.0
    assert [p for _, p in seen] == [{"a": a, "b": b} for a in (1, 2, 3) for b in ("x", "y")]
    assert [i for i, _ in seen] == list(range(6))
    # max_trials cuts the walk short
    short = GridSearchTuner(SPACE, _cost, max_trials=2)
    assert short.tune() == {"a": 1, "b": "y"} and len(short.trials) == 2


def test_random_search_is_seeded_and_never_repeats_a_point():
    def visited(seed, trials):
        t = RandomSearchTuner(SPACE, _cost, max_trials=trials, seed=seed)
        t.tune()
        return [tuple(p.items()) for p, _ in t.trials]
    assert visited(1, 6) == visited(1, 6)
    assert len(set(visited(1, 6))) == 6                       # a full pass visits every point once
    assert visited(1, 4) == visited(1, 6)[:4]
    assert any(visited(s, 6) != visited(1, 6) for s in range(2, 6))
    big = {f"p{i}": TunableItemCfg("choice", list(range(8))) for i in range(6)}     # 262144 points
    t = RandomSearchTuner(big, lambda i, p: float(sum(p.values())), max_trials=50, seed=3)
    t.tune()
    assert len({tuple(p.values()) for p, _ in t.trials}) == 50


def test_failed_trials_are_skipped():
    def flaky(_, p):
        if p["b"] == "y":
            raise RuntimeError("variant cannot run these operands")
        return _cost(_, p)
    t = GridSearchTuner(SPACE, flaky, max_trials=6)
    assert t.tune() == {"a": 2, "b": "x"}
    assert sum(lat is None for _, lat in t.trials) == 3
    never = GridSearchTuner(SPACE, lambda i, p: 1 / 0, max_trials=6)
    assert never.tune() is None and never.best_config is None


def test_tunable_item_validation():
    with pytest.raises(ValueError, match="at least one choice"):
        TunableItemCfg("choice", [])
    with pytest.raises(ValueError, match="unsupported tunable item type"):
        TunableItemCfg("range", [1, 2])


class _Fake(MyAutogradFunc):
    calls = []

    @classmethod
    def param_names(cls):
        return ("a", "b")

    @classmethod
    def get_search_space(cls, sample_inputs, sample_grads=None):
        return SPACE

    @classmethod
    def build_and_test(cls, sample_inputs, sample_grads, params, repeats=5):
        cls.check_params_sanity(params)
        cls.calls.append(dict(params))
        return _cost(0, params)


def test_tune_my_autograd_function_front_end():
    _Fake.calls.clear()
    assert tune_my_autograd_function(_Fake, "fake", [], None, algo="grid", max_trials=40) == {"a": 2, "b": "y"}
    assert len(_Fake.calls) == 6                              # max_trials is clipped to the size of the space
    tuner = tune_my_autograd_function(_Fake, "fake", [], None, algo="random", max_trials=3, seed=7, return_tuner=True)
    assert len(tuner.trials) == 3 and tuner.best_config in [p for p, _ in tuner.trials]
    with pytest.raises(ValueError, match="unsupported tuner algorithm"):
        tune_my_autograd_function(_Fake, "fake", [], None, algo="anneal")
    with pytest.raises(ValueError, match="unknown parameters"):
        _Fake.check_params_sanity({"c": 1})
    with pytest.raises(AssertionError, match="group prefix"):
        _Fake.check_params_sanity({"space_1.a": 1})


def test_search_spaces_of_the_path():
    half = spmm_kernel_choices(torch.float16, 128, 64, 256)
    assert half[0] == "auto" and "mfma8_windows4" in half and "mfma4_lanes16" in half and "dense_form_gemm" in half
    assert "dense_form_gemm" not in spmm_kernel_choices(torch.float16, 128)          # shape of the sparse operand unknown
    assert "dense_form_gemm" not in spmm_kernel_choices(torch.float16, 128, 64, 100)  # m % 8 != 0 (k of the backward product)
    assert not any(k.startswith("mfma32") for k in half)
    assert not any(k.startswith("mfma") for k in spmm_kernel_choices(torch.float16, 100))    # n % 8 != 0
    single = spmm_kernel_choices(torch.float32, 64)
    assert "mfma32_windows4" in single and "rows_by_length" in single and not any(k.startswith(("mfma4", "mfma8")) for k in single)
    assert "rows_by_length" in half and "rows_by_length" not in spmm_kernel_choices(torch.float32, 66)
    assert "few_columns" in spmm_kernel_choices(torch.float32, 256, 64, 128) and "few_columns" not in single
    assert set(half) | set(single) | {"few_columns"} == set(SPMM_KERNELS)
    for flags in SPMM_KERNELS.values():                       # every name maps to legal tuning keys
        with ops.kernel_params(spmm=flags):
            pass
    with pytest.raises(TypeError, match="unknown spmm kernel parameters"):
        with ops.kernel_params(spmm={"tile": 1}):
            pass

    b, values = torch.empty(64, 128, dtype=torch.float16), torch.empty(10, dtype=torch.float16)
    space = MySpMM.get_search_space([b, None, values, None, None, 32, None])
    assert list(space) == ["spmm_kernel", "grad_dense_kernel", "grad_values_wpr"]
    assert space["spmm_kernel"]._value == half and space["grad_values_wpr"]._value == [0, 1, 4]
    MySpMM.check_params_sanity({"spmm_kernel": "row", "grad_values_wpr": 4})
    with pytest.raises(ValueError, match="unknown kernel"):
        MySpMM.check_params_sanity({"spmm_kernel": "fastest"})
    with pytest.raises(ValueError, match="grad_values_wpr"):
        MySpMM.check_params_sanity({"grad_values_wpr": 2})
    assert MyLinear.get_search_space([None, None])["gemm_tile"]._value == list(GEMM_TILES)
    with pytest.raises(ValueError, match="unknown tile"):
        MyLinear.check_params_sanity({"gemm_tile": "64x64"})

    pair = make_kernel_pair_or_triple_autograd_function(MySpMM, MyLinear)
    joint = pair.get_search_space([b, None, values, None, None, 32, None, None, None])
    assert list(joint) == ["space_1.spmm_kernel", "space_1.grad_dense_kernel", "space_1.grad_values_wpr",
                           "space_2.gemm_tile", "space_2.grad_input_tile", "space_2.grad_weight_tile"]
    kw = pair.get_test_fwd_kwargs({"space_1.spmm_kernel": "row", "space_2.gemm_tile": "128x256"})
    assert kw["fwd_kwargs_1"]["params"] == {"spmm_kernel": "row"} and kw["fwd_kwargs_1"]["stream_beg"] == 0
    assert kw["fwd_kwargs_2"]["params"] == {"gemm_tile": "128x256"} and kw["fwd_kwargs_2"]["stream_beg"] == 1
    with pytest.raises(ValueError, match="unknown tile"):
        pair.check_params_sanity({"space_2.gemm_tile": "row"})
    with pytest.raises(ValueError, match="third operator"):
        pair.check_params_sanity({"space_3.gemm_tile": "auto"})


def test_nested_kernel_params_keep_the_other_categories():
    """A block for one category leaves what an enclosing block set for the others; an "auto" choice inside
    the autograd functions does not erase a caller's choice."""
    from intrasm_engine_amd.pytorch import ops as pyops
    seen = lambda: tuple(getattr(pyops._TUNING, k, None) for k in ("spmm", "sddmm", "gemm"))
    with pyops.kernel_params(spmm={"force_variant": 1}, gemm={"tile": 6}):
        with pyops.kernel_params(sddmm={"force_wpr": 4}):
            assert seen() == ({"force_variant": 1}, {"force_wpr": 4}, {"tile": 6})
            with pyops.kernel_params(spmm=None, gemm={"tile": 5}):
                assert seen() == ({"force_variant": 1}, {"force_wpr": 4}, {"tile": 5})
            with pyops.kernel_params(spmm={}):               # an empty dict hands the category back to the library
                assert seen() == (None, {"force_wpr": 4}, {"tile": 6})
        assert seen() == ({"force_variant": 1}, None, {"tile": 6})
    assert seen() == (None, None, None)
