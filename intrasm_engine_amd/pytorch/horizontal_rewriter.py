"""Two or three operators of the path as ONE autograd node on parallel graph branches, and the
layers that replay what such a node recorded.

Re-specified from the reference (pytorch/horizontal_rewriter.py:76-408).  Its version cannot run
as written: ``apply`` is called with keyword arguments (torch forbids them), dictionaries are
stored with ``ctx[...]`` item assignment, the second and third ``_backward`` receive ``ctx`` as
a gradient, and ``ModuleToReplay.forward`` / ``build_and_test`` are left open.  What it means to
do is kept:

* :func:`make_kernel_pair_or_triple_autograd_function` concatenates the inputs, outputs, saved
  tensors and context dictionaries of two or three :class:`MyAutogradFunc` classes (:76-311).
  Each part keeps its own forward options ``fwd_kwargs_<i>`` (:232-262), so each can be recorded
  on its own stream (``stream_beg``) of one graph constructor: the parts have no data dependence
  and become parallel branches of the graph.
* :class:`CUDAGraphModuleNextLayerFunction` replays the forward constructor behind the recorded
  node (:338-360); :class:`CUDAGraphModulePreviousLayerFunction` sits in front of it and replays
  the backward constructor when the gradients come back (:314-335).
* :class:`ConstructorEnabledLayer` wires previous layer -> module -> next layer (:377-408).

Calling convention, as everywhere in this package: options first, tensors after,
``Func.apply(options, *tensors)``.

Differences kept on purpose.  One constructor with one registered stream per part replaces the
reference's list of constructors of which only the first is ever replayed (:391-406): branches
can only overlap inside ONE graph.  The weights pass through the previous layer together with
the activations, so that their gradients too are replayed into before autograd accumulates them.
"""
from __future__ import annotations

from typing import Any, Optional, Sequence

import torch
from torch import nn

from .cpp_extensions.cuda_graph_constructor import TorchCUDAGraphConstructor
from .cpp_extensions.layers_and_funcs.utils import MyAutogradFunc, normalise_kwargs


def simple_combine_search_space(space_1: dict, space_2: dict, space_3: Optional[dict] = None) -> dict:
    """Prefix the keys of each part's search space with ``space_<i>.`` (reference :10-23)."""
    out = {}
    for i, space in enumerate((space_1, space_2, space_3 or {}), start=1):
        for key, value in space.items():
            out[f"space_{i}.{key}"] = value
    return out


def simple_unpack_params(params: dict[str, Any]) -> tuple[dict, ...]:
    """Inverse of :func:`simple_combine_search_space` for one parameter assignment: two
    dictionaries, or three when any ``space_3.`` key is present (reference :26-47)."""
    parts: list[dict] = [{}, {}, {}]
    for key, value in params.items():
        for i in range(3):
            prefix = f"space_{i + 1}."
            if key.startswith(prefix):
                parts[i][key[len(prefix):]] = value
                break
        else:
            raise ValueError(f"Unknown key {key}")
    return tuple(parts) if parts[2] else (parts[0], parts[1])


def make_kernel_pair_or_triple_autograd_function(
    func1: type[MyAutogradFunc], func2: type[MyAutogradFunc], func3: Optional[type[MyAutogradFunc]] = None
) -> type[MyAutogradFunc]:
    """Returns an autograd function ``F`` with

        F.apply({"fwd_kwargs_1": {...}, "fwd_kwargs_2": {...}[, "fwd_kwargs_3": {...}]},
                *inputs_of_func1, *inputs_of_func2[, *inputs_of_func3])
            -> (*outputs_of_func1, *outputs_of_func2[, *outputs_of_func3])

    Missing ``fwd_kwargs_<i>`` means default options (eager, current stream)."""
    funcs = (func1, func2) if func3 is None else (func1, func2, func3)

    class KernelPairOrTripleAutogradFunction(MyAutogradFunc):
        parts = funcs

        @staticmethod
        def num_inputs(**fwd_kwargs) -> int:
            return sum(f.num_inputs() for f in funcs)

        @staticmethod
        def num_saved_tensors(**ctx_kwargs) -> int:
            return sum(f.num_saved_tensors() for f in funcs)

        @classmethod
        def check_fwd_kwargs_sanity(cls, fwd_kwargs: dict[str, Any]) -> list[dict]:
            known = {f"fwd_kwargs_{i + 1}" for i in range(len(funcs))}
            unknown = set(fwd_kwargs or {}) - known
            if unknown:
                raise TypeError(f"unknown forward options: {sorted(unknown)} (expected {sorted(known)})")
            return [normalise_kwargs((fwd_kwargs or {}).get(f"fwd_kwargs_{i + 1}")) for i in range(len(funcs))]

        # ---- tuning hooks: the group's search space is the product of its parts' (reference :109-205)
        @classmethod
        def _split(cls, items: Optional[Sequence], counts: Sequence[int]) -> list:
            if items is None:
                return [None] * len(counts)
            out, beg = [], 0
            for n in counts:
                out.append(list(items[beg:beg + n]))
                beg += n
            return out

        @classmethod
        def get_search_space(cls, sample_inputs, sample_grads=None):
            ins = cls._split(sample_inputs, [f.num_inputs() for f in funcs])
            grads = cls._split(sample_grads, [1] * len(funcs))
            return simple_combine_search_space(*(f.get_search_space(i, g) for f, i, g in zip(funcs, ins, grads)))

        @classmethod
        def _unpack(cls, params: dict) -> list[dict]:
            parts = list(simple_unpack_params(params))
            if len(parts) > len(funcs):
                raise ValueError("parameters for a third operator given to a pair")
            return parts + [{}] * (len(funcs) - len(parts))

        @classmethod
        def check_params_sanity(cls, params: dict) -> None:
            for f, part in zip(funcs, cls._unpack(params)):
                f.check_params_sanity(part)

        @classmethod
        def get_test_fwd_kwargs(cls, params: dict, constructor=None, backward_constructor=None,
                                stream_beg: int = 0) -> dict[str, Any]:
            """Part i at its share of ``params`` on stream ``stream_beg + i`` (reference :168-189)."""
            return {f"fwd_kwargs_{i + 1}": f.get_test_fwd_kwargs(part, constructor, backward_constructor,
                                                                   stream_beg + i)["fwd_kwargs_1"]
                    for i, (f, part) in enumerate(zip(funcs, cls._unpack(params)))}

        @classmethod
        def build_and_test(cls, sample_inputs, sample_grads, params: dict, repeats: int = 5) -> float:
            """Both passes of every part recorded on parallel branches of one forward and one backward
            graph; returns the sum of the two median launch times in milliseconds (the reference
            leaves this open, :207-236)."""
            from .cpp_extensions.layers_and_funcs.utils import time_constructor

            fwd, bwd = TorchCUDAGraphConstructor(), TorchCUDAGraphConstructor()
            fwd.register_new_streams(len(funcs) - 1)
            bwd.register_new_streams(len(funcs) - 1)
            kwargs = cls.check_fwd_kwargs_sanity(cls.get_test_fwd_kwargs(params, fwd, bwd))
            ins = cls._split(sample_inputs, [f.num_inputs() for f in funcs])
            grads = cls._split(sample_grads, [1] * len(funcs))
            keep = []
            with torch.no_grad():
                for f, kw, i, g in zip(funcs, kwargs, ins, grads):
                    outputs, ctx_dict, to_save = f._forward(*i, **kw)
                    g = g if g is not None else [torch.randn_like(o) for o in outputs]
                    keep.append((outputs, f._backward(*g, *to_save, needs_input_grad=f.differentiable_inputs(i),
                                                      **ctx_dict)))
            latency = time_constructor(fwd, repeats) + time_constructor(bwd, repeats)
            del keep
            return latency

        @classmethod
        def forward(cls, ctx, fwd_kwargs, *inputs):
            kwargs = cls.check_fwd_kwargs_sanity(fwd_kwargs)
            counts = [f.num_inputs(**kw) for f, kw in zip(funcs, kwargs)]
            if sum(counts) != len(inputs):
                raise TypeError(f"expected {sum(counts)} inputs ({' + '.join(map(str, counts))}), got {len(inputs)}")
            outputs: list[torch.Tensor] = []
            saved: list[torch.Tensor] = []
            ctx.parts = []  # (inputs, outputs, saved tensors, ctx_dict) per part
            beg = 0
            for f, kw, n in zip(funcs, kwargs, counts):
                outs, ctx_dict, to_save = f._forward(*inputs[beg:beg + n], **kw)
                ctx.parts.append((n, len(outs), len(to_save), ctx_dict))
                outputs.extend(outs)
                saved.extend(to_save)
                beg += n
            ctx.save_for_backward(*saved)
            return tuple(outputs)

        @classmethod
        def backward(cls, ctx, *grads):
            saved = ctx.saved_tensors
            needs = ctx.needs_input_grad[1:]
            grad_inputs: list = []
            ib = ob = sb = 0
            for f, (n_in, n_out, n_saved, ctx_dict) in zip(funcs, ctx.parts):
                part = f._backward(*grads[ob:ob + n_out], *saved[sb:sb + n_saved],
                                   needs_input_grad=needs[ib:ib + n_in], **ctx_dict)
                assert len(part) == n_in, f"{f.__name__}._backward returned {len(part)} gradients for {n_in} inputs"
                grad_inputs.extend(part)
                ib, ob, sb = ib + n_in, ob + n_out, sb + n_saved
            return (None, *grad_inputs)

    names = "_".join(f.__name__ for f in funcs)
    KernelPairOrTripleAutogradFunction.__name__ = KernelPairOrTripleAutogradFunction.__qualname__ = f"KernelGroup_{names}"
    return KernelPairOrTripleAutogradFunction


def _replay(constructor: TorchCUDAGraphConstructor) -> None:
    """Instantiate, launch on the primary stream, wait, destroy (reference :329-333, :353-356)."""
    constructor.instantiate_graph_exec()
    try:
        constructor.execute_graph()
        constructor.synchronize()
    finally:
        constructor.destroy_graph_exec()


class CUDAGraphModulePreviousLayerFunction(torch.autograd.Function):
    """Identity in the forward pass; in the backward pass replays the graph that the node behind
    it recorded into ``options["backward_constructor"]``, which fills the gradient tensors it is
    handed, then passes them on (reference :314-335).
    ``CUDAGraphModulePreviousLayerFunction.apply({"backward_constructor": c}, *tensors)``."""

    @staticmethod
    def forward(ctx, options, *tensors):
        ctx.backward_constructor = options["backward_constructor"]
        return tuple(t.view_as(t) for t in tensors)

    @staticmethod
    def backward(ctx, *grads):
        _replay(ctx.backward_constructor)
        return (None, *grads)


class CUDAGraphModuleNextLayerFunction(torch.autograd.Function):
    """Replays ``options["forward_constructor"]`` in the forward pass, which fills the tensors
    it is handed (the outputs of the recorded node); identity in the backward pass (reference
    :338-360).  ``CUDAGraphModuleNextLayerFunction.apply({"forward_constructor": c}, *tensors)``."""

    @staticmethod
    def forward(ctx, options, *tensors):
        _replay(options["forward_constructor"])
        return tuple(t.view_as(t) for t in tensors)

    @staticmethod
    def backward(ctx, *grads):
        return (None, *grads)


class ModuleToReplay(nn.Module):
    """A module whose forward records ``num_parallel_autograd_funcs`` independent operators as one
    node (``layer_func``), part i on stream i of the constructors it is given (reference
    :364-375).  Subclasses define ``weights()`` (tensors that need gradients) and ``forward``."""

    num_parallel_autograd_funcs: int
    layer_func: type[MyAutogradFunc]

    def weights(self) -> Sequence[torch.Tensor]:
        raise NotImplementedError

    def forward(self, inputs: Sequence[torch.Tensor], weights: Sequence[torch.Tensor], *,
                forward_constructor: Optional[TorchCUDAGraphConstructor],
                backward_constructor: Optional[TorchCUDAGraphConstructor]):
        raise NotImplementedError

    def part_kwargs(self, forward_constructor, backward_constructor) -> dict[str, dict]:
        """``fwd_kwargs_<i>``: record part i on registered stream i; eager when no constructor."""
        enabled = forward_constructor is not None
        return {
            f"fwd_kwargs_{i + 1}": {"constructor": forward_constructor, "backward_constructor": backward_constructor,
                                    "constructor_enabled": enabled, "stream_beg": i if enabled else 0}
            for i in range(self.num_parallel_autograd_funcs)
        }


class ConstructorEnabledLayer(nn.Module):
    """previous layer -> recorded module -> next layer (reference :377-408).  Every call builds a
    forward and a backward constructor with one stream per parallel operator; the forward graph
    is replayed before the outputs are returned, the backward graph when the gradients arrive at
    the previous layer.  ``forward(*inputs)`` returns the tuple of the module's outputs."""

    def __init__(self, layer_to_replay: ModuleToReplay):
        super().__init__()
        self.layer_to_replay = layer_to_replay

    def _constructor(self) -> TorchCUDAGraphConstructor:
        c = TorchCUDAGraphConstructor()
        c.register_new_streams(self.layer_to_replay.num_parallel_autograd_funcs - 1)
        return c

    def forward(self, *inputs):
        forward_constructor, backward_constructor = self._constructor(), self._constructor()
        weights = tuple(self.layer_to_replay.weights())
        passed = CUDAGraphModulePreviousLayerFunction.apply(
            {"backward_constructor": backward_constructor}, *inputs, *weights)
        outputs = self.layer_to_replay(passed[:len(inputs)], passed[len(inputs):],
                                       forward_constructor=forward_constructor,
                                       backward_constructor=backward_constructor)
        return CUDAGraphModuleNextLayerFunction.apply({"forward_constructor": forward_constructor}, *outputs)


class SparseDenseLinearPair(ModuleToReplay):
    """The pair the path is about: a CSR-weight product ``A_csr @ x_sparse`` (:class:`MySpMM`)
    beside a dense linear ``x_dense @ W.T`` (:class:`MyLinear`), fp16 or bf16.

    ``sparse_weight``: dense (m, k) tensor whose zeros define the pattern; ``dense_weight``:
    (out_features, in_features)."""

    num_parallel_autograd_funcs = 2

    def __init__(self, sparse_weight: torch.Tensor, dense_weight: torch.Tensor):
        super().__init__()
        from .cpp_extensions.layers_and_funcs.sputnik import MySpMM
        from .cpp_extensions.layers_and_funcs.torch import MyLinear
        from .utils import dense_to_sparse, transpose_info

        self.layer_func = make_kernel_pair_or_triple_autograd_function(MySpMM, MyLinear)
        values, row_indices, row_offsets, column_indices = dense_to_sparse(sparse_weight, sparse_weight.device)
        self.m, self.k = sparse_weight.shape
        self.values = nn.Parameter(values.to(sparse_weight.dtype))
        self.register_buffer("row_indices", row_indices)
        self.register_buffer("row_offsets", row_offsets)
        self.register_buffer("column_indices", column_indices)
        self._transp_info = transpose_info(self.m, self.k, row_offsets, column_indices)
        self.dense_weight = nn.Parameter(dense_weight.detach().clone())

    def weights(self):
        return (self.values, self.dense_weight)

    def forward(self, inputs, weights, *, forward_constructor=None, backward_constructor=None):
        x_sparse, x_dense = inputs
        values, dense_weight = weights
        return self.layer_func.apply(
            self.part_kwargs(forward_constructor, backward_constructor),
            x_sparse, self.row_indices, values, self.row_offsets, self.column_indices, self.m, self._transp_info,
            x_dense, dense_weight)
