#!/usr/bin/env python3
"""Writes the committed golden vectors (``tests/golden/*.npz``).

The reference holds no golden vector for this path (its SpMM / SDDMM are never run by its
tests) and cannot be imported or built here, so the vectors are produced by this
repository's CPU oracle and accepted only if an independent implementation (scipy CSR for
SpMM, numpy float64 dense products for SDDMM / GEMM) reproduces them.  Run from the
repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import scipy.sparse as sp

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from intrasm_engine_amd import workloads as W  # noqa: E402


def small_csr(seed, m, k, mean_len, empty=()):
    rng = np.random.default_rng(seed)
    lens = np.clip(rng.geometric(1.0 / mean_len, m), 0, k)
    for r in empty:
        lens[r] = 0
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    vals = rng.standard_normal(ci.shape[0]).astype(np.float32)
    return W.CSR(m, k, vals, W.swizzle_from_offsets(ro), ro, ci), rng


def main():
    # 1. SpMM fp32: ragged rows, empty rows, batch 2, n not a multiple of 4
    a, rng = small_csr(101, 37, 29, 6, empty=(0, 11, 36))
    b = rng.standard_normal((2, 29, 10)).astype(np.float32)
    out = oracle.spmm(b, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m)
    ref = sp.csr_matrix((a.values.astype(np.float64), a.column_indices, a.row_offsets), shape=(a.m, a.k))
    for z in range(2):
        assert np.allclose(out[z], ref @ b[z].astype(np.float64), rtol=1e-13, atol=1e-13)
    np.savez(os.path.join(HERE, "spmm_fp32_ragged.npz"), m=a.m, k=a.k, row_indices=a.row_indices, values=a.values,
             row_offsets=a.row_offsets, column_indices=a.column_indices, b=b, expected=out)

    # 2. SpMM fp16-representable operands (values and b are exact in fp16), n = 64
    a, rng = small_csr(102, 48, 64, 12)
    a.values = a.values.astype(np.float16).astype(np.float32)
    b = rng.standard_normal((1, 64, 64)).astype(np.float16).astype(np.float32)
    out = oracle.spmm(b, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m)
    ref = sp.csr_matrix((a.values.astype(np.float64), a.column_indices, a.row_offsets), shape=(a.m, a.k))
    assert np.allclose(out[0], ref @ b[0].astype(np.float64), rtol=1e-13, atol=1e-13)
    np.savez(os.path.join(HERE, "spmm_fp16_inputs.npz"), m=a.m, k=a.k, row_indices=a.row_indices, values=a.values,
             row_offsets=a.row_offsets, column_indices=a.column_indices, b=b, expected=out)

    # 3. SDDMM: batch 3, k = 20, both output layouts
    a, rng = small_csr(103, 23, 31, 5, empty=(4,))
    lhs = rng.standard_normal((3, 23, 20)).astype(np.float32)
    rhs = rng.standard_normal((3, 31, 20)).astype(np.float32)
    per = oracle.sddmm(lhs, rhs, a.row_indices, a.row_offsets, a.column_indices, sum_over_batch=False)
    rows = np.repeat(np.arange(a.m), np.diff(a.row_offsets))
    full = np.einsum("zmk,znk->zmn", lhs.astype(np.float64), rhs.astype(np.float64))
    assert np.allclose(per, full[:, rows, a.column_indices], rtol=1e-13, atol=1e-13)
    np.savez(os.path.join(HERE, "sddmm_fp32.npz"), m=a.m, n=a.k, row_indices=a.row_indices, row_offsets=a.row_offsets,
             column_indices=a.column_indices, lhs=lhs, rhs=rhs, expected_per_batch=per, expected_summed=per.sum(0))

    # 4. GEMM with bf16-representable operands, both B layouts
    rng = np.random.default_rng(104)
    import torch
    ga = torch.from_numpy(rng.standard_normal((40, 24)).astype(np.float32)).bfloat16().float().numpy()
    gb = torch.from_numpy(rng.standard_normal((24, 40)).astype(np.float32)).bfloat16().float().numpy()
    c = oracle.gemm(ga, gb)
    assert np.allclose(c, ga.astype(np.float64) @ gb.astype(np.float64), rtol=1e-13, atol=1e-13)
    np.savez(os.path.join(HERE, "gemm_bf16_inputs.npz"), a=ga, b=gb, expected=c)

    # 5. the 3x4 example of the reference's tests/test_cuda_python_interop.py:79-86
    x = sp.csc_matrix((np.array([0, 1, 3, 2], float), np.array([0, 0, 2, 1]), np.array([0, 1, 2, 3, 4])), shape=(3, 4))
    y = np.array([[1, 2, 3, 4], [1, 2, 3, 4]], np.float32).T.copy()
    vals, ri, ro, ci = oracle.dense_to_csr(x.toarray())
    np.savez(os.path.join(HERE, "reference_3x4_example.npz"), m=3, k=4, row_indices=ri, values=vals, row_offsets=ro,
             column_indices=ci, b=y[None], expected=(x @ y.astype(np.float64))[None])

    # 6. checksums of the big seeded index arrays (generators must stay reproducible)
    import hashlib
    sums = {}
    for s in W.C2_SPARSITIES:
        c2 = W.config2_matrix(s)
        sums[f"c2_{s}"] = hashlib.sha256(c2.row_offsets.tobytes() + c2.column_indices.tobytes()).hexdigest()
    p3 = W.config3()[0]
    sums["c3"] = hashlib.sha256(p3.row_offsets.tobytes() + p3.column_indices.tobytes()).hexdigest()
    with open(os.path.join(HERE, "index_checksums.txt"), "w") as f:
        for k_, v in sums.items():
            f.write(f"{k_} {v}\n")
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
