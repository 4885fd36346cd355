"""``MyLinear`` -- the dense companion of ``MySpMM``: ``input @ weight.T`` with the weight in
torch.nn.Linear layout (out_features, in_features), on the MFMA GEMM of this package
(the reference uses ``input.mm(weight.t())`` on cuBLAS, layers_and_funcs/torch.py:6-31).
fp16 / bf16 only; in_features and out_features must be multiples of 8.

Tunable parameters (``fwd_kwargs["params"]``): ``gemm_tile``, ``grad_input_tile`` and
``grad_weight_tile`` name an entry of :data:`GEMM_TILES` for the three products."""
from __future__ import annotations

import torch

from ... import ops as _ops
from .utils import MyAutogradFunc, TunableItemCfg, maybe_captured

ops = torch.ops.iex_ops

# name -> tile-shape code of the GEMM entry point (workgroup tile, K step)
GEMM_TILES: dict[str, int] = {"auto": 0, "128x128": 5, "128x256": 6, "256x256": 7, "128x128_8waves_k64": 8, "64x128_8waves_k64": 9,
                              # operands staged through registers on their way to LDS
                              "staged_128x128": 1, "staged_128x256": 2, "staged_256x256": 3, "staged_128x128_k64": 4}


def _gemm(a, b, trans_b, tile="auto"):
    with _ops.kernel_params(gemm={"tile": GEMM_TILES[tile]} if GEMM_TILES[tile] else None):
        return ops.gemm_mfma(a, b, trans_b)


class MyLinear(MyAutogradFunc):
    """``MyLinear.apply(fwd_kwargs, input, weight)``."""

    @staticmethod
    def num_inputs(**kwargs) -> int:
        return 2

    @staticmethod
    def num_saved_tensors(**ctx_kwargs) -> int:
        return 2

    @classmethod
    def param_names(cls):
        return ("gemm_tile", "grad_input_tile", "grad_weight_tile")

    @classmethod
    def check_params_sanity(cls, params: dict) -> None:
        super().check_params_sanity(params)
        for key, value in params.items():
            if value not in GEMM_TILES:
                raise ValueError(f"{key}: unknown tile {value!r}")

    @classmethod
    def get_search_space(cls, sample_inputs, sample_grads=None):
        tiles = list(GEMM_TILES)
        return {name: TunableItemCfg("choice", tiles) for name in cls.param_names()}

    @staticmethod
    def _forward(input, weight, **kwargs):
        params = kwargs.get("params") or {}
        input = input.contiguous()
        weight = weight.contiguous()
        with maybe_captured(kwargs["constructor"], kwargs["constructor_enabled"], kwargs["stream_beg"]):
            output = _gemm(input, weight, True, params.get("gemm_tile", "auto"))
        ctx_dict = {"backward_constructor": kwargs["backward_constructor"],
                    "constructor_enabled": kwargs["constructor_enabled"] and kwargs["backward_constructor"] is not None,
                    "stream_beg": kwargs["stream_beg"], "params": params}
        return (output,), ctx_dict, (input, weight)

    @staticmethod
    def _backward(grad_output, input, weight, *, needs_input_grad, backward_constructor, constructor_enabled,
                  stream_beg, params):
        grad_output = grad_output.contiguous()
        grad_input = grad_weight = None
        if needs_input_grad[0]:
            with maybe_captured(backward_constructor, constructor_enabled, stream_beg):
                grad_input = _gemm(grad_output, weight, False, params.get("grad_input_tile", "auto"))
        if needs_input_grad[1]:
            go_t = grad_output.t().contiguous()          # outside the capture zone
            with maybe_captured(backward_constructor, constructor_enabled, stream_beg):
                grad_weight = _gemm(go_t, input, False, params.get("grad_weight_tile", "auto"))
        return grad_input, grad_weight


def linear(input, weight, **fwd_kwargs):
    return MyLinear.apply(fwd_kwargs, input, weight)
