"""``MyLinear`` -- the dense companion of ``MySpMM``: ``input @ weight.T`` with the weight in
torch.nn.Linear layout (out_features, in_features), on the MFMA GEMM of this package
(the reference uses ``input.mm(weight.t())`` on cuBLAS, layers_and_funcs/torch.py:6-31).
fp16 / bf16 only; in_features and out_features must be multiples of 8."""
from __future__ import annotations

import torch

from .utils import MyAutogradFunc, maybe_captured

ops = torch.ops.iex_ops


class MyLinear(MyAutogradFunc):
    """``MyLinear.apply(fwd_kwargs, input, weight)``."""

    @staticmethod
    def num_inputs(**kwargs) -> int:
        return 2

    @staticmethod
    def num_saved_tensors(**ctx_kwargs) -> int:
        return 2

    @staticmethod
    def _forward(input, weight, **kwargs):
        input = input.contiguous()
        weight = weight.contiguous()
        with maybe_captured(kwargs["constructor"], kwargs["constructor_enabled"], kwargs["stream_beg"]):
            output = ops.gemm_mfma(input, weight, True)
        ctx_dict = {"backward_constructor": kwargs["backward_constructor"],
                    "constructor_enabled": kwargs["constructor_enabled"] and kwargs["backward_constructor"] is not None,
                    "stream_beg": kwargs["stream_beg"]}
        return (output,), ctx_dict, (input, weight)

    @staticmethod
    def _backward(grad_output, input, weight, *, needs_input_grad, backward_constructor, constructor_enabled,
                  stream_beg):
        grad_output = grad_output.contiguous()
        grad_input = grad_weight = None
        if needs_input_grad[0]:
            with maybe_captured(backward_constructor, constructor_enabled, stream_beg):
                grad_input = ops.gemm_mfma(grad_output, weight, False)
        if needs_input_grad[1]:
            go_t = grad_output.t().contiguous()          # outside the capture zone
            with maybe_captured(backward_constructor, constructor_enabled, stream_beg):
                grad_weight = ops.gemm_mfma(go_t, input, False)
        return grad_input, grad_weight


def linear(input, weight, **fwd_kwargs):
    return MyLinear.apply(fwd_kwargs, input, weight)
