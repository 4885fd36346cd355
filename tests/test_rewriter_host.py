"""Host logic of the operator-grouping module that needs no GPU: search-space key handling
(reference pytorch/horizontal_rewriter.py:10-47) and the bookkeeping of a grouped node."""
import pytest
import torch

from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.utils import MyAutogradFunc
from intrasm_engine_amd.pytorch.horizontal_rewriter import (
    make_kernel_pair_or_triple_autograd_function,
    simple_combine_search_space,
    simple_unpack_params,
)


def test_search_space_keys_round_trip():
    s1, s2, s3 = {"tile": [64, 128], "waves": [4, 8]}, {"tile": [32]}, {"windows": [1, 2, 4]}
    both = simple_combine_search_space(s1, s2)
    assert both == {"space_1.tile": [64, 128], "space_1.waves": [4, 8], "space_2.tile": [32]}
    assert simple_unpack_params({k: v[0] for k, v in both.items()}) == ({"tile": 64, "waves": 4}, {"tile": 32})
    three = simple_combine_search_space(s1, s2, s3)
    assert simple_unpack_params({k: v[-1] for k, v in three.items()}) == (
        {"tile": 128, "waves": 8}, {"tile": 32}, {"windows": 4})
    with pytest.raises(ValueError, match="Unknown key tile"):
        simple_unpack_params({"tile": 1})


class _Scale(MyAutogradFunc):
    """y = x * w (elementwise), CPU-capable stand-in with two inputs and two saved tensors."""

    @staticmethod
    def num_inputs(**kwargs):
        return 2

    @staticmethod
    def num_saved_tensors(**kwargs):
        return 2

    @staticmethod
    def _forward(x, w, **kwargs):
        return (x * w,), {"stream_beg": kwargs["stream_beg"]}, (x, w)

    @staticmethod
    def _backward(g, x, w, *, needs_input_grad, stream_beg):
        return (g * w if needs_input_grad[0] else None, g * x if needs_input_grad[1] else None)


class _Square(MyAutogradFunc):
    @staticmethod
    def num_inputs(**kwargs):
        return 1

    @staticmethod
    def num_saved_tensors(**kwargs):
        return 1

    @staticmethod
    def _forward(x, **kwargs):
        return (x * x,), {}, (x,)

    @staticmethod
    def _backward(g, x, *, needs_input_grad):
        return (2 * x * g,)


def test_grouped_node_splits_inputs_outputs_and_gradients():
    group = make_kernel_pair_or_triple_autograd_function(_Scale, _Square, _Scale)
    assert group.num_inputs() == 5 and group.num_saved_tensors() == 5
    assert "_Scale__Square__Scale" in group.__name__
    x1, w1, x2, x3 = (torch.arange(1.0, 4.0) * s for s in (1, 2, 3, 4))
    w3 = torch.full((3,), 0.5)
    leaves = [t.clone().requires_grad_(i != 1) for i, t in enumerate((x1, w1, x2, x3, w3))]
    y1, y2, y3 = group.apply({"fwd_kwargs_1": {"stream_beg": 0}}, *leaves)
    assert torch.equal(y1, x1 * w1) and torch.equal(y2, x2 * x2) and torch.equal(y3, x3 * w3)
    (y1.sum() + 2 * y2.sum() + 3 * y3.sum()).backward()
    assert torch.equal(leaves[0].grad, w1) and leaves[1].grad is None
    assert torch.equal(leaves[2].grad, 4 * x2)
    assert torch.equal(leaves[3].grad, 3 * w3) and torch.equal(leaves[4].grad, 3 * x3)
    with pytest.raises(TypeError, match="expected 5 inputs"):
        group.apply({}, *leaves[:4])
    with pytest.raises(TypeError, match="unknown forward options"):
        group.apply({"fwd_kwargs_1": {"tile": 3}}, *leaves)
