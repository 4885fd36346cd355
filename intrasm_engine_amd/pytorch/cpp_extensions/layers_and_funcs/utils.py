"""Contract shared by the autograd functions of the path.

Re-specification of the reference's ``MyAutogradFunc``
(layers_and_funcs/utils.py:11-144) restricted to what its operators use: a function is
written as a pair of pure static methods

    _forward(*inputs, **fwd_kwargs)  -> (outputs, ctx_dict, tensors_to_save)
    _backward(*grads_and_saved, **ctx_dict) -> gradients, one per input

so that two or three of them can later share one autograd node, and ``apply`` is called
as ``Func.apply(fwd_kwargs, *inputs)``.  ``fwd_kwargs`` carries the capture options of
the reference (``constructor``, ``backward_constructor``, ``num_streams``,
``constructor_enabled``, ``stream_beg``; layers_and_funcs/sputnik.py:48-53).  The tuner
hooks of the reference (search spaces, ``build_and_test``) are not part of this path.
"""
from __future__ import annotations

import contextlib

import torch

DEFAULT_FWD_KWARGS = {
    "constructor": None,
    "backward_constructor": None,
    "num_streams": 1,
    "constructor_enabled": False,
    "stream_beg": 0,
}


def normalise_kwargs(kwargs: dict | None) -> dict:
    out = dict(DEFAULT_FWD_KWARGS)
    if kwargs:
        unknown = set(kwargs) - set(DEFAULT_FWD_KWARGS)
        if unknown:
            raise TypeError(f"unknown forward options: {sorted(unknown)}")
        out.update(kwargs)
    assert out["num_streams"] == 1
    if out["constructor_enabled"] and out["constructor"] is None:
        raise ValueError("constructor_enabled needs a constructor")
    return out


@contextlib.contextmanager
def maybe_captured(constructor, enabled: bool, stream_beg: int):
    """Run the body on registered stream ``stream_beg`` of ``constructor`` inside a
    ``capture_library_call_begin/end`` pair, or plainly when capture is off."""
    if not enabled or constructor is None:
        yield
        return
    with constructor.registeredStreams[stream_beg]:
        constructor.capture_library_call_begin()
        try:
            yield
        finally:
            constructor.capture_library_call_end()


class MyAutogradFunc(torch.autograd.Function):
    @staticmethod
    def num_inputs(**fwd_kwargs) -> int:
        raise NotImplementedError

    @staticmethod
    def num_saved_tensors(**ctx_kwargs) -> int:
        raise NotImplementedError

    @staticmethod
    def _forward(*args, **fwd_kwargs):
        raise NotImplementedError

    @staticmethod
    def _backward(*grads_and_saved, **ctx_dict):
        raise NotImplementedError

    @classmethod
    def forward(cls, ctx, fwd_kwargs, *inputs):
        kwargs = normalise_kwargs(fwd_kwargs)
        outputs, ctx_dict, to_save = cls._forward(*inputs, **kwargs)
        ctx.ctx_dict = ctx_dict
        ctx.num_outputs = len(outputs)
        ctx.save_for_backward(*to_save)
        return outputs[0] if len(outputs) == 1 else tuple(outputs)

    @classmethod
    def backward(cls, ctx, *grads):
        grad_inputs = cls._backward(*grads, *ctx.saved_tensors, needs_input_grad=ctx.needs_input_grad[1:],
                                    **ctx.ctx_dict)
        return (None, *grad_inputs)
