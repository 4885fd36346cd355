"""Host-side logic that runs without a GPU: CSR helpers against the oracle, operator
argument validation (same texts as the reference's TORCH_CHECKs), the work model used for
the roofline, and the benchmark's refusal of multi-GPU runs."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import intrasm_engine_amd  # noqa: F401
from intrasm_engine_amd import workloads as W
from intrasm_engine_amd.pytorch import utils as U

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ops = torch.ops.iex_ops


def test_dense_to_sparse_matches_oracle_bit_exact(oracle):
    rng = np.random.default_rng(0)
    dense = np.where(rng.random((57, 43)) < 0.2, rng.standard_normal((57, 43)), 0).astype(np.float32)
    dense[7] = 0
    values, ri, ro, ci = U.dense_to_sparse(torch.from_numpy(dense))
    v_o, ri_o, ro_o, ci_o = oracle.dense_to_csr(dense)
    assert values.dtype == torch.float32 and ri.dtype == ro.dtype == ci.dtype == torch.int32
    assert np.array_equal(values.numpy(), v_o)
    assert np.array_equal(ri.numpy(), ri_o)          # including the (stable) tie order
    assert np.array_equal(ro.numpy(), ro_o)
    assert np.array_equal(ci.numpy(), ci_o)
    assert torch.equal(U.sparse_to_dense(57, 43, values, ro, ci), torch.from_numpy(dense))
    vh, _, _, _ = U.dense_to_sparse(torch.from_numpy(dense).half())
    assert vh.dtype == torch.float16


def test_transpose_info_matches_oracle(oracle):
    a = W.config2_matrix(0.90, m=96, k=160)
    ri_t, ro_t, ci_t, perm = U.transpose_info(a.m, a.k, torch.from_numpy(a.row_offsets), torch.from_numpy(a.column_indices))
    ro_o, ci_o, perm_o = oracle.csr_transpose(a.m, a.k, a.row_offsets, a.column_indices)
    assert np.array_equal(ro_t.numpy(), ro_o) and np.array_equal(ci_t.numpy(), ci_o)
    assert np.array_equal(perm.numpy(), perm_o)
    assert np.array_equal(ri_t.numpy(), W.swizzle_from_offsets(ro_o))
    _, v_t, _, _ = U._transpose_with_info(torch.from_numpy(a.values), (ri_t, ro_t, ci_t, perm))
    assert np.array_equal(v_t.numpy(), a.values[perm_o])
    vb = torch.from_numpy(np.stack([a.values, 2 * a.values]))
    assert U._transpose_with_info(vb, (ri_t, ro_t, ci_t, perm))[1].shape == (2, a.nnz)


def test_operators_are_registered_under_the_reference_names():
    for name in ("spmm_sputnik_atomic", "spmm_sputnik_reuse_weight", "sddmm_sputnik_atomic_upd_weight",
                 "spmm_sputnik_reuse_weight_half", "sddmm_sputnik_half", "gemm_mfma", "fused_spmm_gemm"):
        assert hasattr(ops, name)


def test_cpu_tensors_are_rejected_with_the_reference_messages():
    """No CPU fallback: host tensors raise exactly what the reference's TORCH_CHECKs raise."""
    a = W.config2_matrix(0.90, m=16, k=16)
    ri, v, ro, ci = (torch.from_numpy(x) for x in (a.row_indices, a.values, a.row_offsets, a.column_indices))
    b = torch.zeros(1, 16, 8)
    with pytest.raises(RuntimeError, match="b must be a CUDA tensor"):
        ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, 16)
    with pytest.raises(RuntimeError, match="a must be a CUDA tensor"):
        ops.sddmm_sputnik_atomic_upd_weight(b, b, ri, ro, ci)
    with pytest.raises(RuntimeError):
        ops.spmm_sputnik_reuse_weight(b[0], ri, v, ro, ci, 16)
    with pytest.raises(RuntimeError, match="CUDA tensors"):
        ops.gemm_mfma(torch.zeros(8, 8).half(), torch.zeros(8, 8).half(), False)


def test_work_model_matches_the_published_formulas():
    # SpMM: nnz*(sv+si) + (m+1)*4 + m*4 + batch*(k*n + m*n)*sv ; flops 2*nnz*n*batch
    assert W.spmm_bytes(1024, 1024, 256, 104448) == 104448 * 8 + 1025 * 4 + 1024 * 4 + (1024 * 256 + 1024 * 256) * 4
    assert W.spmm_bytes(4, 4, 4, 8, batch=2, sv=2, si=2, per_batch_values=True) == 2 * 8 * 2 + 8 * 2 + 20 + 16 + 2 * 32 * 2
    assert W.spmm_flops(104448, 256) == 2 * 104448 * 256
    # SDDMM: nnz*4 + (m+1)*4 + m*4 + batch*(m*k + n*k)*sv + out_elems*sv
    assert W.sddmm_bytes(1024, 64, 1024, 104448) == 104448 * 4 + 1025 * 4 + 4096 + 2 * 1024 * 64 * 4 + 104448 * 4
    assert W.sddmm_bytes(8, 4, 8, 10, batch=3, sv=2, sum_over_batch=False) == 40 + 36 + 32 + 3 * 64 * 2 + 30 * 2
    assert W.gemm_bytes(4096, 2048, 4096) == (4096 * 4096 + 4096 * 2048 + 4096 * 2048) * 2
    assert W.gemm_flops(4096, 2048, 4096) == 2 * 4096 * 2048 * 4096


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode != 0 and "one GPU" in proc.stderr


def test_forward_options_are_validated():
    from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.utils import normalise_kwargs
    assert normalise_kwargs(None)["num_streams"] == 1
    with pytest.raises(TypeError):
        normalise_kwargs({"bogus": 1})
    with pytest.raises(ValueError):
        normalise_kwargs({"constructor_enabled": True})


@pytest.mark.gpu
def test_dense_to_sparse_on_a_device_tensor(oracle, dev):
    """The CSR build run on the GPU (torch kernels on a device tensor, as the reference calls it,
    pytorch/utils.py:143-153): values, offsets, column indices and the swizzle bit-equal to the oracle's, for a
    ragged matrix with empty rows and ties in row length."""
    import torch
    from intrasm_engine_amd.pytorch.utils import dense_to_sparse, sparse_to_dense
    rng = np.random.default_rng(5)
    dense = rng.standard_normal((197, 301)).astype(np.float32)
    dense[rng.random(dense.shape) < 0.83] = 0.0
    dense[[0, 50, 196]] = 0.0
    dense[7] = dense[9]                                   # equal lengths: the swizzle must keep row order
    values, row_indices, row_offsets, column_indices = dense_to_sparse(torch.from_numpy(dense), device=dev)
    assert all(t.is_cuda for t in (values, row_indices, row_offsets, column_indices))
    want = oracle.dense_to_csr(dense)
    for got, ref in zip((values, row_indices, row_offsets, column_indices), want):
        assert np.array_equal(got.cpu().numpy(), ref)
    assert torch.equal(sparse_to_dense(197, 301, values, row_offsets, column_indices).cpu(), torch.from_numpy(dense))
