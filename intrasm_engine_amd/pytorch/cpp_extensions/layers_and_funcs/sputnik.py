"""``MySpMM`` -- the trainable CSR x dense product of the path.

Forward  : out = A_csr @ b                       (spmm_sputnik_reuse_weight[_half])
Backward : d(values) = SDDMM(pattern, grad, b)   (sddmm_sputnik_atomic_upd_weight / _half)
           d(b)      = A_csr^T @ grad            (the same SpMM on the transposed CSR)
each optionally recorded into a forward / backward graph constructor.

Re-specified from the reference (layers_and_funcs/sputnik.py:19-149), whose version cannot
run as written: it returns a bare tensor where its base class expects a triple, reads
``ctx.need_input_grad`` (sic) and hands 1-D ``values`` to a helper that indexes 2-D.
Differences kept on purpose: inputs are ``b`` of shape (k, n) and the output is (m, n)
(the reference leaves the unit batch dimension on the output); ``values`` may be fp32 or
fp16/bf16 (the half operators are chosen by dtype).
"""
from __future__ import annotations

import torch

from ...utils import _transpose_with_info, transpose_info
from .utils import MyAutogradFunc, maybe_captured

ops = torch.ops.iex_ops


def _spmm(b3, row_indices, values, row_offsets, column_indices, m):
    if values.dtype == torch.float32:
        return ops.spmm_sputnik_reuse_weight(b3, row_indices, values, row_offsets, column_indices, m)
    return ops.spmm_sputnik_reuse_weight_half(b3, row_indices, values, row_offsets, column_indices, m)


def _sddmm(a3, b3, row_indices, row_offsets, column_indices):
    if a3.dtype == torch.float32:
        return ops.sddmm_sputnik_atomic_upd_weight(a3, b3, row_indices, row_offsets, column_indices)
    return ops.sddmm_sputnik_half(a3, b3, row_indices, row_offsets, column_indices)[0]


class MySpMM(MyAutogradFunc):
    """``MySpMM.apply(fwd_kwargs, b, row_indices, values, row_offsets, column_indices, m, _transp_info)``.

    ``_transp_info`` is the tuple of :func:`transpose_info` (or None: it is then computed
    on the fly, outside any capture); ``column_indices`` may be int16 for half values in the
    forward pass, the backward pass uses int32 indices (the transposed matrix has m columns)."""

    @staticmethod
    def num_inputs(**kwargs) -> int:
        return 7

    @staticmethod
    def num_saved_tensors(**ctx_kwargs) -> int:
        return 9

    @staticmethod
    def _forward(b, row_indices, values, row_offsets, column_indices, m, _transp_info, **kwargs):
        b3 = b.contiguous().unsqueeze(0)                 # batch of one, as the reference does (:54-56)
        k = b3.shape[1]
        if _transp_info is None:
            _transp_info = transpose_info(int(m), k, row_offsets, column_indices)
        with maybe_captured(kwargs["constructor"], kwargs["constructor_enabled"], kwargs["stream_beg"]):
            out = _spmm(b3, row_indices, values, row_offsets, column_indices, int(m))
        ctx_dict = {"m": int(m), "k": k, "backward_constructor": kwargs["backward_constructor"],
                    "constructor_enabled": kwargs["constructor_enabled"] and kwargs["backward_constructor"] is not None,
                    "stream_beg": kwargs["stream_beg"]}
        to_save = (b3, row_indices, values, row_offsets, column_indices, *_transp_info)
        return (out.squeeze(0),), ctx_dict, to_save

    @staticmethod
    def _backward(grad, b3, row_indices, values, row_offsets, column_indices, row_indices_t, row_offsets_t,
                  column_indices_t, perm, *, needs_input_grad, m, k, backward_constructor, constructor_enabled,
                  stream_beg):
        grad3 = grad.contiguous().unsqueeze(0)
        grad_dense = grad_sparse = None
        ci32 = column_indices if column_indices.dtype == torch.int32 else column_indices.to(torch.int32)
        if needs_input_grad[2]:
            # lhs = grad (m, tokens), rhs = b (k, tokens): rhs rows are indexed by the CSR column
            with maybe_captured(backward_constructor, constructor_enabled, stream_beg):
                grad_sparse = _sddmm(grad3, b3, row_indices, row_offsets, ci32)
        if needs_input_grad[0]:
            # gather outside the capture zone, as the reference notes for its transposes (:93-95)
            _, values_t, _, _ = _transpose_with_info(values, (row_indices_t, row_offsets_t, column_indices_t, perm))
            with maybe_captured(backward_constructor, constructor_enabled, stream_beg):
                grad_dense = _spmm(grad3, row_indices_t, values_t, row_offsets_t, column_indices_t, k).squeeze(0)
        return grad_dense, None, grad_sparse, None, None, None, None


def spmm(b, row_indices, values, row_offsets, column_indices, m, _transp_info=None, **fwd_kwargs):
    """Functional form of :class:`MySpMM`."""
    return MySpMM.apply(fwd_kwargs, b, row_indices, values, row_offsets, column_indices, m, _transp_info)
