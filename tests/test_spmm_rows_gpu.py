"""The row kernel with wavefronts per row that follow each row's own length (``iex_spmm_sched``, family 11): forced on
every tile width and chunk budget, where the library picks it by itself, with a wrong histogram and with rows in another
order (both may cost time, never correctness), and the histogram kernel against numpy."""
import ctypes

import numpy as np
import pytest
import torch

from intrasm_engine_amd import _lib, workloads as W
from intrasm_engine_amd.pytorch import ops as pyops
from _util import FP16_SUBNORMAL_HALF_STEP, assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops


def _histogram(row_offsets):
    lens = np.diff(row_offsets.astype(np.int64))
    return [int((lens > (64 << j)).sum()) for j in range(16)]


def test_histogram_kernel_counts_like_numpy(dev):
    for sparsity, m in ((0.7, 4096), (0.98, 4096), (0.9, 777)):
        c = W.config2_matrix(sparsity, m=m, k=4096, seed=5)
        ro = torch.from_numpy(c.row_offsets).to(dev)
        assert list(pyops._row_histogram_host(ro)) == _histogram(c.row_offsets)


def _call(c, dev, b_np, dtype, itype, flags, hist, batch=1, row_indices=None):
    ri, v, ro, ci = to_dev(c, dev, dtype, itype)
    if row_indices is not None:
        ri = torch.from_numpy(row_indices).to(dev)
    bt = torch.from_numpy(b_np).to(dev).to(dtype)
    out = torch.full((batch, c.m, b_np.shape[2]), float("nan"), device=dev, dtype=dtype)
    rc = _lib.load().iex_spmm_sched({torch.float32: _lib.F32, torch.float16: _lib.F16}[dtype], _lib.I16 if itype == torch.int16 else _lib.I32,
                                    flags, c.m, c.k, b_np.shape[2], c.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                                    bt.data_ptr(), None, out.data_ptr(), torch.cuda.current_stream().cuda_stream, batch, None, 0,
                                    (ctypes.c_int * 16)(*hist) if hist is not None else None)
    assert rc == 0, _lib.last_error()
    return out


@pytest.mark.parametrize("n", [32, 64, 128, 256, 520])
@pytest.mark.parametrize("rounds_code", [0, 1, 3, 5])
def test_forced_on_every_tile_width_fp32(oracle, dev, n, rounds_code):
    c = W.config2_matrix(0.9, m=700, k=1024, seed=11)     # rows from 1 to several hundred nonzeros, a ragged last workgroup
    rng = np.random.default_rng(n)
    b_np = rng.standard_normal((2, c.k, n)).astype(np.float32)
    out = _call(c, dev, b_np, torch.float32, torch.int32, (11 << 16) | (rounds_code << 20), _histogram(c.row_offsets), batch=2)
    assert "spmm_rows_kernel" in _lib.last_kernels()
    want = oracle.spmm(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
    scale = oracle.spmm_abs_scale(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
    assert_close(out.cpu().numpy(), want, scale, 1e-5, f"rows kernel n={n}")


@pytest.mark.parametrize("itype", [torch.int32, torch.int16])
def test_forced_fp16(oracle, dev, itype):
    c = W.config2_matrix(0.8, m=513, k=2048, seed=12)
    rng = np.random.default_rng(3)
    b_np = rng.standard_normal((1, c.k, 192)).astype(np.float32)
    out = _call(c, dev, b_np, torch.float16, itype, 11 << 16, _histogram(c.row_offsets))
    assert "spmm_rows_kernel" in _lib.last_kernels()
    v, b_r = rounded(c.values, torch.float16), rounded(b_np, torch.float16)
    want = oracle.spmm(b_r, c.row_indices, v, c.row_offsets, c.column_indices, c.m)
    scale = oracle.spmm_abs_scale(b_r, c.row_indices, v, c.row_offsets, c.column_indices, c.m)
    assert_close(out.float().cpu().numpy(), want, scale, 1e-2, "rows kernel fp16", atol=FP16_SUBNORMAL_HALF_STEP)


def test_a_wrong_histogram_or_another_row_order_costs_time_only(oracle, dev):
    c = W.config2_matrix(0.95, m=1024, k=4096, seed=13)
    rng = np.random.default_rng(4)
    b_np = rng.standard_normal((1, c.k, 64)).astype(np.float32)
    want = oracle.spmm(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
    scale = oracle.spmm_abs_scale(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
    for hist in ([0] * 16, [c.m] * 16, [c.m, c.m // 2, 3] + [0] * 13, [-5, 10 ** 9] + [0] * 14):
        out = _call(c, dev, b_np, torch.float32, torch.int32, 11 << 16, hist)
        assert_close(out.cpu().numpy(), want, scale, 1e-5, f"histogram {hist[:3]}")
    identity = np.arange(c.m, dtype=np.int32)
    out = _call(c, dev, b_np, torch.float32, torch.int32, 11 << 16, _histogram(c.row_offsets), row_indices=identity)
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "rows in natural order")
    out = _call(c, dev, b_np, torch.float32, torch.int32, 11 << 16, _histogram(c.row_offsets), row_indices=c.row_indices[::-1].copy())
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "shortest rows first")


def test_repeated_calls_give_the_same_bits(dev):
    c = W.config2_matrix(0.98)
    b_np = W.config2_dense(128)
    a = _call(c, dev, b_np, torch.float32, torch.int32, 11 << 16, _histogram(c.row_offsets))
    b = _call(c, dev, b_np, torch.float32, torch.int32, 11 << 16, _histogram(c.row_offsets))
    assert torch.equal(a, b)


def test_picked_by_the_operator_on_the_sparsest_cells_of_the_sweep(oracle, dev):
    c = W.config2_matrix(0.98)
    ri, v, ro, ci = to_dev(c, dev)
    for n, expect in ((64, True), (128, True), (256, False)):
        b_np = W.config2_dense(n)
        out = ops.spmm_sputnik_reuse_weight(torch.from_numpy(b_np).to(dev), ri, v, ro, ci, c.m)
        assert ("spmm_rows_kernel" in _lib.last_kernels()) == expect, _lib.last_kernels()
        want = oracle.spmm(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
        scale = oracle.spmm_abs_scale(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
        assert_close(out.cpu().numpy(), want, scale, 1e-5, f"sweep cell 98 % n={n}")


@pytest.mark.parametrize("sparsity,n", [(0.98, 64), (0.9, 128), (0.7, 64)])
def test_order_of_rows_and_histogram_change_no_bit(dev, sparsity, n):
    """The operators promise that the order of row_indices is scheduling only.  Here it settles how many wavefronts a
    row has, but the row's sum is cut by the row's own length: a random order, the reverse order (the longest rows
    where one wavefront serves a row, the shortest where 16 do) and wrong histograms (every row long, no row long)
    give the bits of the sorted order with the true histogram."""
    c = W.config2_matrix(sparsity, m=2048, k=4096, seed=9)
    # a few very long rows, so that every class is there
    lens = np.diff(c.row_offsets).copy()
    lens[[5, 77, 1000]] = [4096, 2500, 1100]
    rng = np.random.default_rng(2)
    ro, ci = W.csr_from_row_lengths(rng, c.m, c.k, lens)
    c = W.CSR(c.m, c.k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((1, c.k, n)).astype(np.float32)
    true_hist = _histogram(c.row_offsets)
    base = _call(c, dev, b_np, torch.float32, torch.int32, 11 << 16, true_hist)
    assert "spmm_rows_kernel" in _lib.last_kernels()
    perm = rng.permutation(c.m).astype(np.int32)
    for order in (perm, c.row_indices[::-1].copy()):
        for hist in (true_hist, [c.m] * 16, [0] * 16, [c.m, c.m // 2, 7] + [0] * 13):
            got = _call(c, dev, b_np, torch.float32, torch.int32, 11 << 16, hist, row_indices=order)
            assert torch.equal(got, base), (order[:4], hist[:4])
    for hist in ([c.m] * 16, [0] * 16):
        assert torch.equal(_call(c, dev, b_np, torch.float32, torch.int32, 11 << 16, hist), base)


def test_forcing_it_without_a_histogram_is_refused(dev):
    c = W.config2_matrix(0.9, m=64, k=256, seed=1)
    ri, v, ro, ci = to_dev(c, dev)
    b = torch.randn(1, c.k, 64, device=dev)
    out = torch.empty(1, c.m, 64, device=dev)
    rc = _lib.load().iex_spmm_ex(_lib.F32, _lib.I32, 11 << 16, c.m, c.k, 64, c.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                                 b.data_ptr(), None, out.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert rc == _lib.load().iex_spmm_ex.restype(-1) or rc == -1
    assert "histogram" in _lib.last_error()
