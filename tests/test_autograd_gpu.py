"""MySpMM / MyLinear: forward and both gradients against the CPU oracle, eager and
recorded into forward / backward graph constructors."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from intrasm_engine_amd.pytorch import utils as U
from intrasm_engine_amd.pytorch.cpp_extensions.cuda_graph_constructor import TorchCUDAGraphConstructor
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.sputnik import MySpMM, spmm
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.torch import MyLinear, linear
from _util import RTOL, assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu


def _oracle_grads(oracle, a, vals, b_np, g_np):
    want = oracle.spmm(b_np[None], a.row_indices, vals, a.row_offsets, a.column_indices, a.m)[0]
    d_vals = oracle.sddmm(g_np[None], b_np[None], a.row_indices, a.row_offsets, a.column_indices)
    ro_t, ci_t, perm = oracle.csr_transpose(a.m, a.k, a.row_offsets, a.column_indices)
    d_b = oracle.spmm(g_np[None], W.swizzle_from_offsets(ro_t), vals[perm], ro_t, ci_t, a.k)[0]
    s_out = oracle.spmm_abs_scale(b_np[None], a.row_indices, vals, a.row_offsets, a.column_indices, a.m)[0]
    s_vals = oracle.sddmm_abs_scale(g_np[None], b_np[None], a.row_indices, a.row_offsets, a.column_indices)
    s_b = oracle.spmm_abs_scale(g_np[None], W.swizzle_from_offsets(ro_t), vals[perm], ro_t, ci_t, a.k)[0]
    return (want, s_out), (d_vals, s_vals), (d_b, s_b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_myspmm_forward_backward(oracle, dev, dtype):
    rng = np.random.default_rng(0)
    a = W.config2_matrix(0.90, m=384, k=256)
    n = 128
    b_np = rng.standard_normal((a.k, n)).astype(np.float32)
    g_np = rng.standard_normal((a.m, n)).astype(np.float32)
    ri, v, ro, ci = to_dev(a, dev, dtype)
    v.requires_grad_(True)
    b = torch.from_numpy(b_np).to(dev).to(dtype).requires_grad_(True)
    info = U.transpose_info(a.m, a.k, ro, ci)
    out = spmm(b, ri, v, ro, ci, a.m, info)
    assert out.shape == (a.m, n)
    out.backward(torch.from_numpy(g_np).to(dev).to(dtype))
    (want, s_out), (d_vals, s_vals), (d_b, s_b) = _oracle_grads(
        oracle, a, rounded(a.values, dtype), rounded(b_np, dtype), rounded(g_np, dtype))
    assert_close(out.detach().float().cpu().numpy(), want, s_out, RTOL[dtype], "forward")
    assert_close(v.grad.float().cpu().numpy(), d_vals, s_vals, RTOL[dtype], "d(values)")
    assert_close(b.grad.float().cpu().numpy(), d_b, s_b, RTOL[dtype], "d(dense)")
    # transposition info computed on the fly gives the same gradients
    v2 = v.detach().clone().requires_grad_(True)
    b2 = b.detach().clone().requires_grad_(True)
    MySpMM.apply({}, b2, ri, v2, ro, ci, a.m, None).backward(torch.from_numpy(g_np).to(dev).to(dtype))
    assert torch.equal(v2.grad, v.grad) and torch.equal(b2.grad, b.grad)


def test_myspmm_recorded_into_forward_and_backward_graphs(dev):
    """constructor_enabled: the forward launch is recorded into one constructor, both
    backward launches into another; replaying them reproduces the eager tensors."""
    a = W.config2_matrix(0.95, m=256, k=256)
    ri, v, ro, ci = to_dev(a, dev)
    v.requires_grad_(True)
    b = torch.randn(a.k, 64, device=dev, requires_grad=True)
    g = torch.randn(a.m, 64, device=dev)
    info = U.transpose_info(a.m, a.k, ro, ci)
    eager = spmm(b, ri, v, ro, ci, a.m, info)
    eager.backward(g)
    gv, gb = v.grad.clone(), b.grad.clone()
    v.grad = b.grad = None

    fwd, bwd = TorchCUDAGraphConstructor(), TorchCUDAGraphConstructor()
    out = spmm(b, ri, v, ro, ci, a.m, info, constructor=fwd, backward_constructor=bwd, constructor_enabled=True)
    fwd.instantiate_graph_exec()
    fwd.execute_graph()
    fwd.synchronize()
    assert torch.equal(out.detach(), eager.detach())
    out.backward(g)
    bwd.instantiate_graph_exec()
    bwd.execute_graph()
    bwd.synchronize()
    assert torch.equal(v.grad, gv) and torch.equal(b.grad, gb)
    assert bwd.constructor.node_types().count(0) == 2        # SDDMM + SpMM(A^T) kernels
    fwd.destroy_graph_exec()
    bwd.destroy_graph_exec()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mylinear_forward_backward(oracle, dev, dtype):
    rng = np.random.default_rng(1)
    x_np = rng.standard_normal((96, 64)).astype(np.float32)
    w_np = rng.standard_normal((40, 64)).astype(np.float32)
    g_np = rng.standard_normal((96, 40)).astype(np.float32)
    x = torch.from_numpy(x_np).to(dev).to(dtype).requires_grad_(True)
    w = torch.from_numpy(w_np).to(dev).to(dtype).requires_grad_(True)
    y = linear(x, w)
    y.backward(torch.from_numpy(g_np).to(dev).to(dtype))
    xr, wr, gr = rounded(x_np, dtype), rounded(w_np, dtype), rounded(g_np, dtype)
    assert_close(y.detach().float().cpu().numpy(), oracle.gemm(xr, wr, trans_b=True),
                 oracle.gemm(np.abs(xr), np.abs(wr), trans_b=True), 1e-2, "y")
    assert_close(x.grad.float().cpu().numpy(), oracle.gemm(gr, wr), oracle.gemm(np.abs(gr), np.abs(wr)), 1e-2, "dx")
    assert_close(w.grad.float().cpu().numpy(), oracle.gemm(np.ascontiguousarray(gr.T), xr),
                 oracle.gemm(np.abs(np.ascontiguousarray(gr.T)), np.abs(xr)), 1e-2, "dw")
    assert MyLinear.num_inputs() == 2
