"""Variant search on the device: every named kernel choice reaches the kernels and keeps parity
with the CPU oracle, ``build_and_test`` returns a positive time, and the tuner's winner is a point
of the space that still gives the oracle's result."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from intrasm_engine_amd.pytorch import utils as U
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.sputnik import MySpMM, spmm, spmm_kernel_choices
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.torch import GEMM_TILES, MyLinear, linear
from intrasm_engine_amd.pytorch.horizontal_rewriter import make_kernel_pair_or_triple_autograd_function
from intrasm_engine_amd.tuning.my_autograd_func_tuner import tune_my_autograd_function
from _util import RTOL, assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu


def _spmm_case(dev, dtype, n=128, sparsity=0.8):
    rng = np.random.default_rng(3)
    a = W.config2_matrix(sparsity, m=512, k=384, seed=4)
    b_np = rng.standard_normal((a.k, n)).astype(np.float32)
    g_np = rng.standard_normal((a.m, n)).astype(np.float32)
    ri, v, ro, ci = to_dev(a, dev, dtype)
    info = U.transpose_info(a.m, a.k, ro, ci)
    t = lambda x: torch.from_numpy(x).to(dev).to(dtype)
    return a, b_np, g_np, [t(b_np), ri, v, ro, ci, a.m, info], [t(g_np)]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_every_kernel_choice_keeps_parity(oracle, dev, dtype):
    a, b_np, g_np, inputs, grads = _spmm_case(dev, dtype)
    vals, br, gr = rounded(a.values, dtype), rounded(b_np, dtype), rounded(g_np, dtype)
    want = oracle.spmm(br[None], a.row_indices, vals, a.row_offsets, a.column_indices, a.m)[0]
    scale = oracle.spmm_abs_scale(br[None], a.row_indices, vals, a.row_offsets, a.column_indices, a.m)[0]
    ro_t, ci_t, perm = oracle.csr_transpose(a.m, a.k, a.row_offsets, a.column_indices)
    ri_t = W.swizzle_from_offsets(ro_t)
    want_db = oracle.spmm(gr[None], ri_t, vals[perm], ro_t, ci_t, a.k)[0]
    scale_db = oracle.spmm_abs_scale(gr[None], ri_t, vals[perm], ro_t, ci_t, a.k)[0]
    want_dv = oracle.sddmm(gr[None], br[None], a.row_indices, a.row_offsets, a.column_indices)
    scale_dv = oracle.sddmm_abs_scale(gr[None], br[None], a.row_indices, a.row_offsets, a.column_indices)
    outputs = {}
    choices = spmm_kernel_choices(dtype, b_np.shape[1], a.k, a.m)
    assert ("dense_form_gemm" in choices) == (dtype == torch.float16)
    for i, kernel in enumerate(choices):
        b = inputs[0].detach().clone().requires_grad_(True)
        v = inputs[2].detach().clone().requires_grad_(True)
        params = {"spmm_kernel": kernel, "grad_dense_kernel": kernel, "grad_values_wpr": (0, 1, 4)[i % 3]}
        out = spmm(b, inputs[1], v, *inputs[3:], params=params)
        out.backward(grads[0])
        assert_close(out.detach().float().cpu().numpy(), want, scale, RTOL[dtype], f"forward, {kernel}")
        assert_close(b.grad.float().cpu().numpy(), want_db, scale_db, RTOL[dtype], f"d(dense), {kernel}")
        assert_close(v.grad.float().cpu().numpy(), want_dv, scale_dv, RTOL[dtype], f"d(values), {kernel}")
        outputs[kernel] = out.detach()
    # the choice reaches the kernels: the matrix-core families sum in another order than the row kernel
    mfma = "mfma8_windows4" if dtype == torch.float16 else "mfma32_windows4"
    assert not torch.equal(outputs[mfma], outputs["row"])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_every_gemm_tile_keeps_parity(oracle, dev, dtype):
    rng = np.random.default_rng(5)
    x_np, w_np = rng.standard_normal((320, 256)).astype(np.float32), rng.standard_normal((264, 256)).astype(np.float32)
    g_np = rng.standard_normal((320, 264)).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev).to(dtype)
    xr, wr, gr = rounded(x_np, dtype), rounded(w_np, dtype), rounded(g_np, dtype)
    for tile in GEMM_TILES:
        x, w = t(x_np).requires_grad_(True), t(w_np).requires_grad_(True)
        y = linear(x, w, params={"gemm_tile": tile, "grad_input_tile": tile, "grad_weight_tile": tile})
        y.backward(t(g_np))
        assert_close(y.detach().float().cpu().numpy(), oracle.gemm(xr, wr, trans_b=True),
                     oracle.gemm(np.abs(xr), np.abs(wr), trans_b=True), 1e-2, f"y, {tile}")
        assert_close(x.grad.float().cpu().numpy(), oracle.gemm(gr, wr), oracle.gemm(np.abs(gr), np.abs(wr)), 1e-2,
                     f"dx, {tile}")
        assert_close(w.grad.float().cpu().numpy(), oracle.gemm(np.ascontiguousarray(gr.T), xr),
                     oracle.gemm(np.abs(np.ascontiguousarray(gr.T)), np.abs(xr)), 1e-2, f"dw, {tile}")


def test_tune_spmm_and_pair(oracle, dev):
    a, b_np, g_np, inputs, grads = _spmm_case(dev, torch.float16, n=256, sparsity=0.7)
    assert MySpMM.build_and_test(inputs, grads, {"spmm_kernel": "row"}) > 0.0
    tuner = tune_my_autograd_function(MySpMM, "spmm", inputs, grads, algo="random", max_trials=8, seed=1,
                                      return_tuner=True)
    space = MySpMM.get_search_space(inputs, grads)
    best = tuner.best_config
    assert best is not None and all(best[k] in space[k]._value for k in space)
    assert all(lat is not None and lat > 0 for _, lat in tuner.trials) and len(tuner.trials) == 8
    assert tuner.best_latency == min(lat for _, lat in tuner.trials)
    out = spmm(*inputs, params=best)
    vals, br = rounded(a.values, torch.float16), rounded(b_np, torch.float16)
    assert_close(out.float().cpu().numpy(),
                 oracle.spmm(br[None], a.row_indices, vals, a.row_offsets, a.column_indices, a.m)[0],
                 oracle.spmm_abs_scale(br[None], a.row_indices, vals, a.row_offsets, a.column_indices, a.m)[0],
                 RTOL[torch.float16], "tuned forward")

    pair = make_kernel_pair_or_triple_autograd_function(MySpMM, MyLinear)
    x = torch.randn(512, 256, device=dev, dtype=torch.float16)
    w = torch.randn(384, 256, device=dev, dtype=torch.float16)
    best = tune_my_autograd_function(pair, "pair", [*inputs, x, w], None, algo="random", max_trials=5, seed=2)
    assert best is not None and set(best) == set(pair.get_search_space([*inputs, x, w]))
    y1, y2 = pair.apply(pair.get_test_fwd_kwargs(best), *inputs, x, w)
    assert_close(y1.float().cpu().numpy(),
                 oracle.spmm(br[None], a.row_indices, vals, a.row_offsets, a.column_indices, a.m)[0],
                 oracle.spmm_abs_scale(br[None], a.row_indices, vals, a.row_offsets, a.column_indices, a.m)[0],
                 RTOL[torch.float16], "tuned pair, sparse part")
    xr, wr = x.float().cpu().numpy(), w.float().cpu().numpy()
    assert_close(y2.float().cpu().numpy(), oracle.gemm(xr, wr, trans_b=True),
                 oracle.gemm(np.abs(xr), np.abs(wr), trans_b=True), 1e-2, "tuned pair, dense part")
