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

Tunable parameters (``fwd_kwargs["params"]``): ``spmm_kernel`` and ``grad_dense_kernel`` name
an entry of :data:`SPMM_KERNELS` for the forward product and for the product with the
transposed matrix, ``grad_values_wpr`` is the wavefronts-per-row choice of the SDDMM.
"""
from __future__ import annotations

import torch

from ... import ops as _ops
from ...utils import _transpose_with_info, transpose_info
from .utils import MyAutogradFunc, TunableItemCfg, maybe_captured

ops = torch.ops.iex_ops

# name -> tuning bits of the SpMM entry point.  "auto" leaves the choice to the library.
SPMM_KERNELS: dict[str, dict] = {
    "auto": {},
    "row": {"force_variant": 1},
    "row_wpr4": {"force_variant": 1, "force_wpr": 4},
    "row_wpr8": {"force_variant": 1, "force_wpr": 8},
    "lds_rows2": {"force_variant": 2, "force_rpw": 2},
    "lds_rows4": {"force_variant": 2, "force_rpw": 4},
    "lds_rows8": {"force_variant": 2, "force_rpw": 8},
    # 16-bit types on the matrix cores
    "mfma4_lanes8": {"force_variant": 3, "force_lpg": 8},
    "mfma4_lanes16": {"force_variant": 3, "force_lpg": 16},
    "mfma8_windows1": {"force_variant": 4, "force_rpw": 1},
    "mfma8_windows2": {"force_variant": 4, "force_rpw": 2},
    "mfma8_windows4": {"force_variant": 4, "force_rpw": 4},
    "mfma8_windows5": {"force_variant": 4, "force_rpw": 5},
    # the same tile with the dense operand loaded straight into LDS, A expanded 64 columns at a time
    "mfma8_direct_windows1": {"force_variant": 6, "force_rpw": 1},
    "mfma8_direct_windows2": {"force_variant": 6, "force_rpw": 2},
    # the dense form of the sparse operand written into a workspace (the operator allocates it), then the dense GEMM
    "dense_form_gemm": {"force_variant": 7},
    # A with at most 128 columns and a wide output: the dense operand's tile in LDS, rows streamed
    "few_columns": {"force_variant": 8},
    # fp32 on the matrix cores: 32 x 128 tiles with 2, 4 or 8 windows, 16 x 128 tiles
    "mfma32_windows2": {"force_variant": 5, "force_nt": 4, "force_rpw": 2},
    "mfma32_windows4": {"force_variant": 5, "force_nt": 4, "force_rpw": 4},
    "mfma32_windows8": {"force_variant": 5, "force_nt": 4, "force_rpw": 8},
    "mfma32_rows16": {"force_variant": 5, "force_nt": 6, "force_rpw": 4},
    # the row kernel with 16, 8, 4, 2 or 1 wavefronts per row by the row's own length (the operator hands the pattern's
    # row-length histogram over); a wavefront gets at most 1, 2 or 4 chunks of 64 nonzeros
    "rows_by_length": {"force_variant": 11},
    "rows_by_length_1chunk": {"force_variant": 11, "force_rpw": 1},
    "rows_by_length_4chunks": {"force_variant": 11, "force_rpw": 3},
    # the library's choice for a launch that shares the chip with a gather-bound launch (a parallel branch of a graph):
    # fp32 products that are a tie between the row kernel and the matrix cores then take the matrix cores
    "auto_beside_gather_kernel": {"beside_gather_kernel": True},
}


def spmm_kernel_choices(dtype: torch.dtype, n: int, k: int | None = None, m: int | None = None) -> list[str]:
    """The entries of :data:`SPMM_KERNELS` that can run a product with ``n`` dense columns of
    ``dtype`` (a family that cannot would silently fall back and only repeat a measurement).
    The dense-form path refuses shapes it cannot serve instead of falling back, and the backward
    pass runs the same choice on the transposed matrix: it is offered when the sparse operand's
    ``k`` and ``m`` are given and multiples of 8."""
    names = ["auto", "row", "row_wpr4", "row_wpr8", "lds_rows2", "lds_rows4", "lds_rows8"]
    vec = 4 if dtype == torch.float32 else 8
    if k is not None and m is not None and max(k, m) <= 128 and n % vec == 0 and n >= 64 * vec:
        names.append("few_columns")      # (refuses other shapes; the backward product has m columns)
    if dtype in (torch.float16, torch.bfloat16) and n % 8 == 0:
        names += [k_ for k_ in SPMM_KERNELS if k_.startswith(("mfma4_", "mfma8_"))]
        if k is not None and m is not None and k % 8 == 0 and m % 8 == 0:
            names.append("dense_form_gemm")
    if dtype == torch.float32 and n % 4 == 0:
        names += [k for k in SPMM_KERNELS if k.startswith("mfma32_")] + ["auto_beside_gather_kernel"]
    if n % vec == 0:
        names += [k for k in SPMM_KERNELS if k.startswith("rows_by_length")]    # (full 128-bit vectors; the backward product has the same n)
    return names


def _spmm(b3, row_indices, values, row_offsets, column_indices, m, kernel="auto"):
    with _ops.kernel_params(spmm=SPMM_KERNELS[kernel] or None):   # "auto" keeps an enclosing block's choice
        if values.dtype == torch.float32:
            return ops.spmm_sputnik_reuse_weight(b3, row_indices, values, row_offsets, column_indices, m)
        return ops.spmm_sputnik_reuse_weight_half(b3, row_indices, values, row_offsets, column_indices, m)


def _sddmm(a3, b3, row_indices, row_offsets, column_indices, wpr=0):
    with _ops.kernel_params(sddmm={"force_wpr": wpr} if wpr else None):
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

    @classmethod
    def param_names(cls):
        return ("spmm_kernel", "grad_dense_kernel", "grad_values_wpr")

    @classmethod
    def check_params_sanity(cls, params: dict) -> None:
        super().check_params_sanity(params)
        for key in ("spmm_kernel", "grad_dense_kernel"):
            if params.get(key, "auto") not in SPMM_KERNELS:
                raise ValueError(f"{key}: unknown kernel {params[key]!r}")
        if params.get("grad_values_wpr", 0) not in (0, 1, 4):
            raise ValueError("grad_values_wpr must be 0 (choose), 1 or 4")

    @classmethod
    def get_search_space(cls, sample_inputs, sample_grads=None):
        b, values = sample_inputs[0], sample_inputs[2]
        names = spmm_kernel_choices(values.dtype, b.shape[-1], b.shape[-2], int(sample_inputs[5]))
        return {"spmm_kernel": TunableItemCfg("choice", names),
                "grad_dense_kernel": TunableItemCfg("choice", names),
                "grad_values_wpr": TunableItemCfg("choice", [0, 1, 4])}

    @classmethod
    def differentiable_inputs(cls, sample_inputs):
        return (True, False, True, False, False, False, False)

    @staticmethod
    def _forward(b, row_indices, values, row_offsets, column_indices, m, _transp_info, **kwargs):
        params = kwargs.get("params") or {}
        b3 = b.contiguous().unsqueeze(0)                 # batch of one, as the reference does (:54-56)
        k = b3.shape[1]
        if _transp_info is None:
            _transp_info = transpose_info(int(m), k, row_offsets, column_indices)
        with maybe_captured(kwargs["constructor"], kwargs["constructor_enabled"], kwargs["stream_beg"]):
            out = _spmm(b3, row_indices, values, row_offsets, column_indices, int(m), params.get("spmm_kernel", "auto"))
        ctx_dict = {"m": int(m), "k": k, "backward_constructor": kwargs["backward_constructor"],
                    "constructor_enabled": kwargs["constructor_enabled"] and kwargs["backward_constructor"] is not None,
                    "stream_beg": kwargs["stream_beg"], "params": params}
        to_save = (b3, row_indices, values, row_offsets, column_indices, *_transp_info)
        return (out.squeeze(0),), ctx_dict, to_save

    @staticmethod
    def _backward(grad, b3, row_indices, values, row_offsets, column_indices, row_indices_t, row_offsets_t,
                  column_indices_t, perm, *, needs_input_grad, m, k, backward_constructor, constructor_enabled,
                  stream_beg, params):
        grad3 = grad.contiguous().unsqueeze(0)
        grad_dense = grad_sparse = None
        ci32 = column_indices if column_indices.dtype == torch.int32 else _ops.carry_pattern_note(column_indices, column_indices.to(torch.int32))
        if needs_input_grad[2]:
            # lhs = grad (m, tokens), rhs = b (k, tokens): rhs rows are indexed by the CSR column
            with maybe_captured(backward_constructor, constructor_enabled, stream_beg):
                grad_sparse = _sddmm(grad3, b3, row_indices, row_offsets, ci32, params.get("grad_values_wpr", 0))
        if needs_input_grad[0]:
            # gather outside the capture zone, as the reference notes for its transposes (:93-95)
            _, values_t, _, _ = _transpose_with_info(values, (row_indices_t, row_offsets_t, column_indices_t, perm))
            with maybe_captured(backward_constructor, constructor_enabled, stream_beg):
                grad_dense = _spmm(grad3, row_indices_t, values_t, row_offsets_t, column_indices_t, k,
                                   params.get("grad_dense_kernel", "auto")).squeeze(0)
        return grad_dense, None, grad_sparse, None, None, None, None


def spmm(b, row_indices, values, row_offsets, column_indices, m, _transp_info=None, **fwd_kwargs):
    """Functional form of :class:`MySpMM`."""
    return MySpMM.apply(fwd_kwargs, b, row_indices, values, row_offsets, column_indices, m, _transp_info)
