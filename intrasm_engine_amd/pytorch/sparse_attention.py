"""Sparse attention over a fixed CSR mask: SDDMM -> softmax over the stored entries -> SpMM.

The reference's attention benchmark stops after the two sparse products it takes from Sputnik
(sddmm_sputnik_atomic_upd_weight and spmm_sputnik_*, sputnik_kernels.cpp:170-184) and has no
softmax between them; this block supplies the missing middle step so that the three launches
form the attention of one layer:

    scores[h, j] = <q[h, row(j)], k[h, col(j)]>            per head, at the nonzeros of the mask
    probs        = softmax over each CSR row of scores * scale        (in place)
    out[h]       = probs[h] (as CSR values) @ v[h]

All heads share the index arrays; values are per head.  Three launches on the current stream,
nothing leaves the device, no dense tokens x tokens matrix exists at any point.
"""
from __future__ import annotations

import math

import torch

ops = torch.ops.iex_ops


def sparse_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, row_indices: torch.Tensor,
                     row_offsets: torch.Tensor, column_indices: torch.Tensor, scale: float | None = None,
                     return_probs: bool = False, plan=None):
    """q, k: (heads, tokens, d); v: (heads, tokens, dv); mask pattern tokens x tokens as int32 CSR
    arrays (``row_indices`` = rows by decreasing length).  fp16, bf16 or fp32.  Returns
    (heads, tokens, dv), and the (heads, nnz) probabilities when ``return_probs``.
    Rows of the mask without entries give zero output rows.
    ``plan``: an ``ops.SddmmPlan`` that the caller keeps for this mask; with it the tables and lists that the two sparse
    products derive from the mask are written by the first call only (16-bit inputs; ignored where those kernels are not
    the ones that run)."""
    if q.dim() != 3 or k.shape != q.shape or v.dim() != 3 or v.shape[:2] != q.shape[:2]:
        raise RuntimeError("q, k must be (heads, tokens, d) and v (heads, tokens, dv)")
    tokens = q.shape[1]
    if row_indices.shape[0] != tokens:
        raise RuntimeError("the mask must be tokens x tokens")
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[2])
    from . import ops as _pyops
    if plan is None and q.dtype in (torch.float16, torch.bfloat16) and \
            _pyops.structured_tables(row_offsets, column_indices, tokens) is None:
        # for this call only: what the first product derives from the mask serves the second too.  (Not needed for a
        # pattern with structure that the operators have looked at before: its tables are kept with the pattern.)
        plan = _pyops.SddmmPlan()
    if plan is not None:
        scores = _pyops.sddmm_half_planned(q, k, row_indices, row_offsets, column_indices, plan)
    else:
        scores = ops.sddmm_sputnik_half(q, k, row_indices, row_offsets, column_indices)     # (heads, nnz)
    probs = ops.csr_softmax_(scores, row_indices, row_offsets, float(scale))
    if plan is not None:
        out = _pyops.spmm_batched_values_planned(v, row_indices, probs, row_offsets, column_indices, tokens, plan)
    else:
        out = ops.spmm_sputnik_batched_values(v, row_indices, probs, row_offsets, column_indices, tokens)
    return (out, probs) if return_probs else out
