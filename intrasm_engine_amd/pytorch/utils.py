"""CSR construction helpers of the path: dense -> CSR with the load-balancing row
swizzle, CSR transpose by a cached permutation, CSR -> dense.

They run as torch tensor operations on whatever device the input lives on (index
construction is set-up work outside the timed path, as in the reference, which
delegates it to xformers: pytorch/utils.py:143-153).  All index tensors are int32.
"""
from __future__ import annotations

import torch


def row_swizzle(row_offsets: torch.Tensor) -> torch.Tensor:
    """Rows ordered by decreasing number of nonzeros; ties keep ascending row order
    (a stable sort: the order among equal-length rows is fixed and documented here,
    it never affects results because every row writes its own output row)."""
    lens = torch.diff(row_offsets.to(torch.int64))
    return torch.argsort(lens, descending=True, stable=True).to(torch.int32)


def dense_to_sparse(matrix: torch.Tensor, device=None):
    """Dense 2-D matrix -> ``(values, row_indices, row_offsets, column_indices)``:
    ``values`` = row-major ``matrix[matrix != 0]`` (dtype kept), ``row_offsets`` =
    ``[0, cumsum(nnz per row)]``, ``column_indices`` ascending inside a row,
    ``row_indices`` = :func:`row_swizzle`."""
    assert matrix.dim() == 2
    if device is not None:
        matrix = matrix.to(device)
    mask = matrix != 0
    values = matrix[mask].contiguous()
    counts = mask.sum(dim=1, dtype=torch.int64)
    row_offsets = torch.zeros(matrix.shape[0] + 1, dtype=torch.int64, device=matrix.device)
    torch.cumsum(counts, 0, out=row_offsets[1:])
    column_indices = mask.nonzero()[:, 1].to(torch.int32).contiguous()
    row_offsets = row_offsets.to(torch.int32)
    if column_indices.is_cuda:
        from .ops import mark_canonical
        mark_canonical(row_offsets, column_indices, matrix.shape[1])   # (by construction: the operators need not look)
    return values, row_swizzle(row_offsets), row_offsets, column_indices


def sparse_to_dense(m: int, k: int, values, row_offsets, column_indices) -> torch.Tensor:
    lens = torch.diff(row_offsets.to(torch.int64))
    rows = torch.repeat_interleave(torch.arange(m, device=values.device), lens)
    out = torch.zeros((m, k), dtype=values.dtype, device=values.device)
    out[rows, column_indices.to(torch.int64)] = values
    return out


def transpose_info(m: int, k: int, row_offsets: torch.Tensor, column_indices: torch.Tensor):
    """Index arrays of the transposed matrix plus the permutation that carries values
    over: ``(row_indices_t, row_offsets_t, column_indices_t, perm)`` with
    ``values_t = values[perm]``.  Computed once per sparsity pattern and reused by every
    backward pass (the ``_transp_info`` argument of ``MySpMM``,
    layers_and_funcs/sputnik.py:45,117-122)."""
    dev = column_indices.device
    lens = torch.diff(row_offsets.to(torch.int64))
    rows = torch.repeat_interleave(torch.arange(m, device=dev, dtype=torch.int64), lens)
    cols = column_indices.to(torch.int64)
    perm = torch.argsort(cols * m + rows)           # keys are unique: (col, row) pairs
    column_indices_t = rows[perm].to(torch.int32).contiguous()
    counts = torch.bincount(cols, minlength=k)
    row_offsets_t = torch.zeros(k + 1, dtype=torch.int64, device=dev)
    torch.cumsum(counts, 0, out=row_offsets_t[1:])
    row_offsets_t = row_offsets_t.to(torch.int32)
    if column_indices_t.is_cuda:
        from .ops import mark_canonical
        mark_canonical(row_offsets_t, column_indices_t, m)   # (sorted by (column, row): ascending and distinct by construction, given distinct columns per row)
    return row_swizzle(row_offsets_t), row_offsets_t, column_indices_t, perm


def _transpose_with_info(values: torch.Tensor, _transp_info):
    """``(row_indices_t, values_t, row_offsets_t, column_indices_t)``; ``values`` may be
    (nnz) or (batch, nnz)."""
    row_indices_t, row_offsets_t, column_indices_t, perm = _transp_info
    values_t = values[..., perm].contiguous()
    return row_indices_t, values_t, row_offsets_t, column_indices_t


def to_int16_indices(column_indices: torch.Tensor, k: int) -> torch.Tensor:
    """Compressed column indices for the half kernels (the reference's ``short2``
    layout, sputnik_kernels.cpp:179-181); needs k <= 32768."""
    if k > 32768:
        raise ValueError("int16 column indices need k <= 32768")
    from .ops import carry_pattern_note
    return carry_pattern_note(column_indices, column_indices.to(torch.int16))
