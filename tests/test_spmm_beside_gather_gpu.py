"""IEX_SPMM_BESIDE_GATHER_KERNEL: a launch that is told it shares the chip with a gather-bound launch takes the fp32
matrix-core kernel where that kernel and the row kernel are close (density from 19.5 %, n from 128), and nothing else
changes: same results against the oracle, no effect on sparser or narrower products, on other element types, on
patterns whose columns may come in any order, or on a forced family."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import _lib, workloads as W
from intrasm_engine_amd.pytorch import ops as pyops
from _util import assert_close, to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops
HINT = {"beside_gather_kernel": True}


@pytest.mark.parametrize("sparsity,n,takes_matrix_cores", [(0.8, 256, True), (0.7, 128, True), (0.8, 128, True), (0.9, 256, False),
                                                            (0.8, 64, False), (0.7, 256, True)])
def test_kernel_choice_and_parity_on_the_sweeps_cells(oracle, dev, sparsity, n, takes_matrix_cores):
    c = W.config2_matrix(sparsity)
    ri, v, ro, ci = to_dev(c, dev)
    b_np = W.config2_dense(n)
    b = torch.from_numpy(b_np).to(dev)
    alone = ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, c.m)
    alone_kernel = _lib.last_kernels()
    with pyops.kernel_params(spmm=HINT):
        beside = ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, c.m)
    beside_kernel = _lib.last_kernels()
    assert ("spmm_mfma_f32_kernel" in beside_kernel) == takes_matrix_cores, beside_kernel
    if sparsity > 0.75 or n < 256:
        assert "mfma" not in alone_kernel, alone_kernel       # (alone only the densest n = 256 cell takes the matrix cores)
    if not takes_matrix_cores:
        assert beside_kernel == alone_kernel and torch.equal(beside, alone)
    want = oracle.spmm(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
    scale = oracle.spmm_abs_scale(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
    assert_close(beside.cpu().numpy(), want, scale, 1e-5, f"beside a gather kernel, s={sparsity} n={n}")


def test_the_hint_changes_nothing_else(dev):
    c = W.config2_matrix(0.8)
    ri, v, ro, ci = to_dev(c, dev)
    b = torch.from_numpy(W.config2_dense(256)).to(dev)
    # a forced family stays forced
    with pyops.kernel_params(spmm={"force_variant": 1, **HINT}):
        ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, c.m)
        assert "mfma" not in _lib.last_kernels()
    # columns in any order (here: every row reversed): the families that take such input, hint or not
    lens = np.diff(c.row_offsets)
    rev = np.concatenate([c.column_indices[s:e][::-1] for s, e in zip(c.row_offsets[:-1], c.row_offsets[1:])]).astype(np.int32)
    vals_rev = np.concatenate([c.values[s:e][::-1] for s, e in zip(c.row_offsets[:-1], c.row_offsets[1:])]).astype(np.float32)
    ci_rev, v_rev = torch.from_numpy(rev).to(dev), torch.from_numpy(vals_rev).to(dev)
    with pyops.kernel_params(spmm=HINT):
        got = ops.spmm_sputnik_reuse_weight(b, ri, v_rev, ro, ci_rev, c.m)
        assert "mfma" not in _lib.last_kernels()
    assert torch.allclose(got, ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, c.m), rtol=1e-4, atol=1e-5)
    # fp16: no fp32 matrix-core kernel to take; the choice is that of a call without the hint
    rih, vh, roh, cih = to_dev(c, dev, torch.float16, torch.int16)
    bh = b.half()
    ops.spmm_sputnik_reuse_weight_half(bh, rih, vh, roh, cih, c.m)
    without = _lib.last_kernels()
    with pyops.kernel_params(spmm=HINT):
        ops.spmm_sputnik_reuse_weight_half(bh, rih, vh, roh, cih, c.m)
    assert _lib.last_kernels() == without


def test_through_the_c_interface(dev):
    c = W.config2_matrix(0.8)
    ri, v, ro, ci = to_dev(c, dev)
    b = torch.from_numpy(W.config2_dense(256)).to(dev)
    lib = _lib.load()
    outs = {}
    for flags in (0, _lib.SPMM_BESIDE_GATHER_KERNEL, _lib.SPMM_BESIDE_GATHER_KERNEL | _lib.SPMM_ANY_COLUMN_ORDER):
        out = torch.empty(1, c.m, 256, device=dev)
        _lib.check(lib.iex_spmm_ex(_lib.F32, _lib.I32, flags, c.m, c.k, 256, c.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                                   b.data_ptr(), None, out.data_ptr(), torch.cuda.current_stream(dev).cuda_stream, 1), "spmm_ex")
        outs[flags] = (out, _lib.last_kernels())
    torch.cuda.synchronize()
    assert "mfma" not in outs[0][1] and "spmm_mfma_f32_kernel" in outs[_lib.SPMM_BESIDE_GATHER_KERNEL][1]
    assert "mfma" not in outs[_lib.SPMM_BESIDE_GATHER_KERNEL | _lib.SPMM_ANY_COLUMN_ORDER][1]
    assert torch.allclose(outs[0][0], outs[_lib.SPMM_BESIDE_GATHER_KERNEL][0], rtol=1e-4, atol=1e-5)
