"""SDDMM -> CSR softmax -> SpMM as one block, against the CPU oracle step by step and against
dense masked attention in float64 (a witness that shares no code with the oracle's CSR loops)."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from intrasm_engine_amd.pytorch.sparse_attention import sparse_attention
from _util import rounded, to_dev

pytestmark = pytest.mark.gpu


def _dense_attention(pattern, q, k, v, scale):
    mask = np.zeros((pattern.m, pattern.k), dtype=bool)
    rows = np.repeat(np.arange(pattern.m), np.diff(pattern.row_offsets))
    mask[rows, pattern.column_indices] = True
    s = np.einsum("htd,hsd->hts", q.astype(np.float64), k.astype(np.float64)) * scale
    s = np.where(mask[None], s, -np.inf)
    live = mask.any(axis=1)
    s[:, ~live, :] = 0.0
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    p = np.where(mask[None], p, 0.0)
    denom = p.sum(axis=-1, keepdims=True)
    p = np.divide(p, denom, out=np.zeros_like(p), where=denom > 0)
    return p @ v.astype(np.float64)


@pytest.mark.parametrize("dtype, tol", [(torch.float32, 2e-5), (torch.float16, 1e-2), (torch.bfloat16, 4e-2)])
def test_sparse_attention_block(oracle, dev, dtype, tol):
    pattern, q, k, v = W.config3(seed=12, tokens=384, heads=3, head_dim=64, band=48, extra=6)
    ri, _, ro, ci = to_dev(pattern, dev)
    qr, kr, vr = (rounded(x, dtype) for x in (q, k, v))
    t = lambda a: torch.from_numpy(a).to(dev).to(dtype)
    scale = 1.0 / 8.0
    out, probs = sparse_attention(t(q), t(k), t(v), ri, ro, ci, return_probs=True)
    assert out.shape == (3, 384, 64) and probs.shape == (3, pattern.nnz)

    # oracle, step by step, float64 throughout (the device rounds scores and probabilities to dtype)
    scores = oracle.sddmm(qr, kr, pattern.row_indices, pattern.row_offsets, pattern.column_indices,
                          sum_over_batch=False)
    want_probs = oracle.csr_softmax(scores * scale, pattern.row_offsets)
    want = oracle.spmm(vr, pattern.row_indices, want_probs, pattern.row_offsets, pattern.column_indices, pattern.m)
    got = out.float().cpu().numpy()
    # probabilities are in [0, 1] and rows of v are O(1): absolute tolerance on a convex combination
    assert np.abs(probs.float().cpu().numpy() - want_probs).max() <= tol
    assert np.abs(got - want).max() <= tol * np.abs(vr).max()
    dense = _dense_attention(pattern, qr, kr, vr, scale)
    assert np.abs(want - dense).max() <= 1e-6                  # the oracle agrees with dense masked attention
    assert np.abs(got - dense).max() <= tol * np.abs(vr).max()
    sums = np.add.reduceat(probs.float().cpu().numpy(), pattern.row_offsets[:-1], axis=1)
    assert np.allclose(sums, 1.0, atol=5 * tol)


def test_rows_without_entries_and_default_scale(oracle, dev):
    rng = np.random.default_rng(2)
    tokens, d = 96, 32
    mask = rng.random((tokens, tokens)) < 0.1
    mask[[0, 17, 95]] = False
    ro, ci, _ = W.csr_from_mask(mask)
    ri = W.swizzle_from_offsets(ro)
    q, k, v = (rng.standard_normal((2, tokens, d)).astype(np.float32) for _ in range(3))
    t = lambda a: torch.from_numpy(a).to(dev)
    out = sparse_attention(t(q), t(k), t(v), t(ri), t(ro), t(ci)).cpu().numpy()
    assert not out[:, [0, 17, 95]].any()
    pattern = W.CSR(tokens, tokens, np.ones(ci.shape[0], np.float32), ri, ro, ci)
    dense = _dense_attention(pattern, q, k, v, 1.0 / np.sqrt(d))
    assert np.abs(out - dense).max() <= 2e-5 * np.abs(v).max()
    with pytest.raises(RuntimeError, match="tokens x tokens"):
        sparse_attention(t(q), t(k), t(v), t(ri[:-1]), t(ro[:-1]), t(ci))


def test_block_with_a_plan_runs_both_structured_kernels_and_keeps_their_tables(oracle, dev):
    """A caller that keeps a plan for its mask: both sparse products take their kernels for masks with structure, the
    second call launches nothing but the three kernels of the block, and the result is that of the block without a
    plan (whose products, at this size, the library gives to the gather and row kernels) up to fp16 rounding, and
    the oracle's."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    pattern, q, k, v = W.config3(seed=21, tokens=640, heads=2, head_dim=64, band=160, extra=4)
    ri, _, ro, ci = to_dev(pattern, dev)
    t = lambda a: torch.from_numpy(a).to(dev).half()
    plan = pyops.SddmmPlan()
    assert plan.analyze(ro, ci, pattern.k) == 3
    first = sparse_attention(t(q), t(k), t(v), ri, ro, ci, plan=plan)
    assert "spmm_blocks_kernel" in _lib.last_kernels()
    again = sparse_attention(t(q), t(k), t(v), ri, ro, ci, plan=plan)
    assert _lib.last_kernels() == "spmm_blocks_kernel<false>" and torch.equal(again, first)
    plain = sparse_attention(t(q), t(k), t(v), ri, ro, ci)
    assert "spmm_blocks_kernel" not in _lib.last_kernels()
    assert torch.allclose(first.float(), plain.float(), rtol=1e-2, atol=5e-3)
    qr, kr, vr = (rounded(x, torch.float16) for x in (q, k, v))
    scores = oracle.sddmm(qr, kr, pattern.row_indices, pattern.row_offsets, pattern.column_indices, sum_over_batch=False)
    want = oracle.spmm(vr, pattern.row_indices, oracle.csr_softmax(scores * 0.125, pattern.row_offsets), pattern.row_offsets,
                       pattern.column_indices, pattern.m)
    assert np.abs(first.float().cpu().numpy() - want).max() <= 1e-2 * np.abs(vr).max()
