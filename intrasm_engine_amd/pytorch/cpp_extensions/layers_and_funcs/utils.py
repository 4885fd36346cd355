"""Contract shared by the autograd functions of the path.

Re-specification of the reference's ``MyAutogradFunc``
(layers_and_funcs/utils.py:11-144): a function is written as a pair of pure static methods

    _forward(*inputs, **fwd_kwargs)  -> (outputs, ctx_dict, tensors_to_save)
    _backward(*grads_and_saved, **ctx_dict) -> gradients, one per input

so that two or three of them can share one autograd node, and ``apply`` is called
as ``Func.apply(fwd_kwargs, *inputs)``.  ``fwd_kwargs`` carries the capture options of
the reference (``constructor``, ``backward_constructor``, ``num_streams``,
``constructor_enabled``, ``stream_beg``; layers_and_funcs/sputnik.py:48-53) and ``params``, a
point of the function's search space: which kernel variant each launch of the forward and
backward pass uses (the reference's tuner hooks, :61-144: ``get_search_space``,
``check_params_sanity``, ``get_test_fwd_kwargs``, ``build_and_test``; there ``build_and_test``
stops at a TODO before timing anything, here it replays the recorded graphs and returns
milliseconds).
"""
from __future__ import annotations

import contextlib
import statistics
from dataclasses import dataclass, field
from typing import Any, Optional

import torch

DEFAULT_FWD_KWARGS = {
    "constructor": None,
    "backward_constructor": None,
    "num_streams": 1,
    "constructor_enabled": False,
    "stream_beg": 0,
    "params": None,
}


@dataclass
class TunableItemCfg:
    """One dimension of a search space: ``_value`` lists the choices (the shape of SparTA's
    class of the same name, which the reference imports, :3; only ``choice`` items exist)."""
    _type: str = "choice"
    _value: list = field(default_factory=list)

    def __post_init__(self):
        if self._type != "choice":
            raise ValueError(f"unsupported tunable item type {self._type!r}")
        if len(self._value) == 0:
            raise ValueError("a tunable item needs at least one choice")


def assert_params_unpacked(params: dict) -> None:
    """A point handed to a single function must not carry the ``space_<i>.`` prefixes of a group
    (reference :6-8)."""
    for key in params:
        assert not key.startswith("space_"), f"parameter {key!r} still carries a group prefix"


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


def time_constructor(constructor, repeats: int = 5, warmup: int = 1) -> float:
    """Median milliseconds of one launch of what ``constructor`` recorded (0.0 for an empty one)."""
    if constructor.constructor.num_nodes() == 0:
        return 0.0
    constructor.instantiate_graph_exec()
    times = []
    try:
        for _ in range(warmup):
            constructor.execute_graph()
        constructor.synchronize()
        for _ in range(repeats):
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record()          # the current stream is the constructor's primary stream
            constructor.execute_graph()
            end.record()
            constructor.synchronize()
            times.append(start.elapsed_time(end))
    finally:
        constructor.destroy_graph_exec()
    return statistics.median(times)


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

    # ------------------------------------------------------------------ tuning hooks
    @classmethod
    def get_search_space(cls, sample_inputs: list, sample_grads: Optional[list]) -> dict[str, TunableItemCfg]:
        """{parameter name: choices}.  Every combination must be a legal ``params``."""
        raise NotImplementedError

    @classmethod
    def check_params_sanity(cls, params: dict) -> None:
        """Raises unless ``params`` is a point of this function's search space (names only: the
        legal values depend on the operands)."""
        assert_params_unpacked(params)
        unknown = set(params) - set(cls.param_names())
        if unknown:
            raise ValueError(f"{cls.__name__}: unknown parameters {sorted(unknown)}")

    @classmethod
    def param_names(cls) -> tuple[str, ...]:
        raise NotImplementedError

    @classmethod
    def get_test_fwd_kwargs(cls, params: dict, constructor=None, backward_constructor=None,
                            stream_beg: int = 0) -> dict[str, Any]:
        """``{"fwd_kwargs_1": options}`` that run the function at ``params``; recorded into the
        two constructors when given (reference :113-118)."""
        cls.check_params_sanity(params)
        return {"fwd_kwargs_1": {"constructor": constructor, "backward_constructor": backward_constructor,
                                 "constructor_enabled": constructor is not None, "stream_beg": stream_beg,
                                 "params": dict(params)}}

    @classmethod
    def differentiable_inputs(cls, sample_inputs: list) -> tuple[bool, ...]:
        """Which inputs get a gradient during tuning: floating-point tensors by default."""
        return tuple(isinstance(t, torch.Tensor) and t.is_floating_point() for t in sample_inputs)

    @classmethod
    def build_and_test(cls, sample_inputs: list, sample_grads: Optional[list], params: dict,
                       repeats: int = 5) -> float:
        """Records the forward pass and the backward pass at ``params`` into one graph each,
        replays both and returns the sum of their median launch times in milliseconds
        (reference :120-144)."""
        from ..cuda_graph_constructor import TorchCUDAGraphConstructor

        fwd, bwd = TorchCUDAGraphConstructor(), TorchCUDAGraphConstructor()
        kwargs = normalise_kwargs(cls.get_test_fwd_kwargs(params, fwd, bwd)["fwd_kwargs_1"])
        with torch.no_grad():
            outputs, ctx_dict, to_save = cls._forward(*sample_inputs, **kwargs)
            if sample_grads is None:
                sample_grads = [torch.randn_like(o) for o in outputs]
            grads = cls._backward(*sample_grads, *to_save, needs_input_grad=cls.differentiable_inputs(sample_inputs),
                                  **ctx_dict)
        latency = time_constructor(fwd, repeats) + time_constructor(bwd, repeats)
        del outputs, grads
        return latency
