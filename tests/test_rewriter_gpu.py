"""Two or three operators as one autograd node on parallel graph branches, and the replay layers
around it (pytorch/horizontal_rewriter.py of the reference, re-specified).  The single operators
are checked against the CPU oracle in test_autograd_gpu.py; here the grouped node must give the
same bits as the operators one by one, eager and replayed, and the layer is checked against the
oracle once more end to end."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from intrasm_engine_amd.pytorch import utils as U
from intrasm_engine_amd.pytorch.cpp_extensions.cuda_graph_constructor import TorchCUDAGraphConstructor
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.sputnik import MySpMM, spmm
from intrasm_engine_amd.pytorch.cpp_extensions.layers_and_funcs.torch import MyLinear, linear
from intrasm_engine_amd.pytorch.horizontal_rewriter import (
    CUDAGraphModuleNextLayerFunction,
    CUDAGraphModulePreviousLayerFunction,
    ConstructorEnabledLayer,
    SparseDenseLinearPair,
    make_kernel_pair_or_triple_autograd_function,
)
from _util import assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu
KERNEL_NODE = 0


class _Case:
    """A CSR matrix with half values and a dense linear of unrelated shape, with gradients."""

    def __init__(self, dev, seed=0, dtype=torch.float16):
        g = torch.Generator().manual_seed(seed)
        self.a = W.config2_matrix(0.90, m=256, k=384, seed=seed + 1)
        self.ri, v, self.ro, self.ci = to_dev(self.a, dev, dtype)
        self.info = U.transpose_info(self.a.m, self.a.k, self.ro, self.ci)
        self.v = v
        self.b = torch.randn(self.a.k, 128, generator=g).to(dev).to(dtype)
        self.x = torch.randn(192, 64, generator=g).to(dev).to(dtype)
        self.w = torch.randn(80, 64, generator=g).to(dev).to(dtype)
        self.g_sparse = torch.randn(self.a.m, 128, generator=g).to(dev).to(dtype)
        self.g_dense = torch.randn(192, 80, generator=g).to(dev).to(dtype)

    def leaves(self):
        return [t.detach().clone().requires_grad_(True) for t in (self.b, self.v, self.x, self.w)]

    def spmm_inputs(self, b, v):
        return (b, self.ri, v, self.ro, self.ci, self.a.m, self.info)

    def one_by_one(self):
        b, v, x, w = self.leaves()
        y1 = spmm(*self.spmm_inputs(b, v))
        y2 = linear(x, w)
        torch.autograd.backward([y1, y2], [self.g_sparse, self.g_dense])
        return (y1.detach(), y2.detach()), tuple(t.grad for t in (b, v, x, w))


def test_pair_node_equals_the_two_operators(dev):
    case = _Case(dev)
    want_out, want_grads = case.one_by_one()
    pair = make_kernel_pair_or_triple_autograd_function(MySpMM, MyLinear)
    assert pair.num_inputs() == 9 and pair.num_saved_tensors() == 11
    b, v, x, w = case.leaves()
    y1, y2 = pair.apply({}, *case.spmm_inputs(b, v), x, w)
    torch.autograd.backward([y1, y2], [case.g_sparse, case.g_dense])
    assert torch.equal(y1, want_out[0]) and torch.equal(y2, want_out[1])
    for got, want in zip((b.grad, v.grad, x.grad, w.grad), want_grads):
        assert torch.equal(got, want)
    # only one output used downstream: the other part receives a zero gradient
    b, v, x, w = case.leaves()
    y1, y2 = pair.apply({}, *case.spmm_inputs(b, v), x, w)
    y2.backward(case.g_dense)
    assert torch.equal(x.grad, want_grads[2]) and torch.equal(w.grad, want_grads[3])
    assert not b.grad.any() and not v.grad.any()
    with pytest.raises(TypeError, match="expected 9 inputs"):
        pair.apply({}, x, w)
    with pytest.raises(TypeError, match="unknown forward options"):
        pair.apply({"fwd_kwargs_3": {}}, *case.spmm_inputs(b, v), x, w)


def test_pair_recorded_as_parallel_branches(dev):
    """Part i on stream i of one constructor: the forward graph holds two kernel nodes with no
    path between them, the backward graph four (two per operator); replays reproduce eager."""
    case = _Case(dev, seed=3)
    want_out, want_grads = case.one_by_one()
    pair = make_kernel_pair_or_triple_autograd_function(MySpMM, MyLinear)
    fwd, bwd = TorchCUDAGraphConstructor(), TorchCUDAGraphConstructor()
    fwd.register_new_stream()
    bwd.register_new_stream()
    opts = {f"fwd_kwargs_{i + 1}": {"constructor": fwd, "backward_constructor": bwd, "constructor_enabled": True,
                                    "stream_beg": i} for i in range(2)}
    b, v, x, w = case.leaves()
    y1, y2 = pair.apply(opts, *case.spmm_inputs(b, v), x, w)
    types = fwd.constructor.node_types()
    assert types.count(KERNEL_NODE) == 2
    kernels = [i for i, t in enumerate(types) if t == KERNEL_NODE]
    assert not any(set(e) == set(kernels) for e in fwd.constructor.edges())
    fwd.instantiate_graph_exec()
    fwd.execute_graph()
    fwd.synchronize()
    assert torch.equal(y1.detach(), want_out[0]) and torch.equal(y2.detach(), want_out[1])
    torch.autograd.backward([y1, y2], [case.g_sparse, case.g_dense])
    assert bwd.constructor.node_types().count(KERNEL_NODE) == 4
    bwd.instantiate_graph_exec()
    bwd.execute_graph()
    bwd.synchronize()
    for got, want in zip((b.grad, v.grad, x.grad, w.grad), want_grads):
        assert torch.equal(got, want)
    fwd.destroy_graph_exec()
    bwd.destroy_graph_exec()


def test_triple_node(dev):
    case, other = _Case(dev, seed=5), _Case(dev, seed=6)
    want_out, want_grads = case.one_by_one()
    other_out, other_grads = other.one_by_one()
    triple = make_kernel_pair_or_triple_autograd_function(MySpMM, MyLinear, MySpMM)
    assert triple.num_inputs() == 16
    b, v, x, w = case.leaves()
    b3, v3, _, _ = other.leaves()
    y1, y2, y3 = triple.apply({"fwd_kwargs_2": {}}, *case.spmm_inputs(b, v), x, w, *other.spmm_inputs(b3, v3))
    torch.autograd.backward([y1, y2, y3], [case.g_sparse, case.g_dense, other.g_sparse])
    assert torch.equal(y1, want_out[0]) and torch.equal(y2, want_out[1]) and torch.equal(y3, other_out[0])
    for got, want in zip((b.grad, v.grad, x.grad, w.grad, b3.grad, v3.grad), (*want_grads, *other_grads[:2])):
        assert torch.equal(got, want)


def test_replay_layers_alone(dev):
    """The previous layer replays the backward constructor when gradients arrive, the next layer
    replays the forward constructor before handing its inputs on."""
    case = _Case(dev, seed=7)
    want_out, want_grads = case.one_by_one()
    fwd, bwd = TorchCUDAGraphConstructor(), TorchCUDAGraphConstructor()
    b, v, _, _ = case.leaves()
    b_in, v_in = CUDAGraphModulePreviousLayerFunction.apply({"backward_constructor": bwd}, b, v)
    y = spmm(*case.spmm_inputs(b_in, v_in), constructor=fwd, backward_constructor=bwd, constructor_enabled=True)
    (y,) = CUDAGraphModuleNextLayerFunction.apply({"forward_constructor": fwd}, y)
    assert torch.equal(y.detach(), want_out[0])
    y.backward(case.g_sparse)
    assert torch.equal(b.grad, want_grads[0]) and torch.equal(v.grad, want_grads[1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_constructor_enabled_layer(oracle, dev, dtype):
    rng = np.random.default_rng(11)
    m, k, tokens, fin, fout = 256, 384, 128, 64, 80
    sw = rng.standard_normal((m, k)).astype(np.float32) * (rng.random((m, k)) < 0.1)
    sw[5] = 0.0                                               # an empty row
    dw = rng.standard_normal((fout, fin)).astype(np.float32)
    xs = rng.standard_normal((k, tokens)).astype(np.float32)
    xd = rng.standard_normal((tokens, fin)).astype(np.float32)
    gs = rng.standard_normal((m, tokens)).astype(np.float32)
    gd = rng.standard_normal((tokens, fout)).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(dev).to(dtype)
    module = SparseDenseLinearPair(t(sw), t(dw))
    layer = ConstructorEnabledLayer(module)

    def run(fn):
        x1, x2 = t(xs).requires_grad_(True), t(xd).requires_grad_(True)
        module.zero_grad(set_to_none=True)
        y1, y2 = fn(x1, x2)
        torch.autograd.backward([y1, y2], [t(gs), t(gd)])
        return [u.detach().clone() for u in (y1, y2, x1.grad, x2.grad, module.values.grad, module.dense_weight.grad)]

    eager = run(lambda x1, x2: module((x1, x2), module.weights()))
    replayed = run(layer)
    for got, want in zip(replayed, eager):
        assert torch.equal(got, want)

    # end to end against the oracle: forward outputs and the gradient of the sparse values
    dwr, xsr, xdr, gsr = (rounded(a, dtype) for a in (dw, xs, xd, gs))
    ro, ci = module.row_offsets.cpu().numpy(), module.column_indices.cpu().numpy()
    ri, vals = module.row_indices.cpu().numpy(), module.values.detach().float().cpu().numpy()
    want1 = oracle.spmm(xsr[None], ri, vals, ro, ci, m)[0]
    scale1 = oracle.spmm_abs_scale(xsr[None], ri, vals, ro, ci, m)[0]
    assert_close(replayed[0].float().cpu().numpy(), want1, scale1, 1e-2, "sparse product")
    assert_close(replayed[1].float().cpu().numpy(), oracle.gemm(xdr, dwr, trans_b=True),
                 oracle.gemm(np.abs(xdr), np.abs(dwr), trans_b=True), 1e-2, "dense product")
    assert_close(replayed[4].float().cpu().numpy(), oracle.sddmm(gsr[None], xsr[None], ri, ro, ci),
                 oracle.sddmm_abs_scale(gsr[None], xsr[None], ri, ro, ci), 1e-2, "d(values)")

    # a second pass accumulates into the parameters' gradients only after its replay
    x1, x2 = t(xs).requires_grad_(True), t(xd).requires_grad_(True)
    y1, y2 = layer(x1, x2)
    torch.autograd.backward([y1, y2], [t(gs), t(gd)])
    assert_close(module.values.grad.float().cpu().numpy(), 2 * eager[4].float().cpu().numpy(),
                 2 * np.abs(eager[4].float().cpu().numpy()), 1e-2, "accumulated d(values)")
    assert_close(module.dense_weight.grad.float().cpu().numpy(), 2 * eager[5].float().cpu().numpy(),
                 2 * np.abs(eager[5].float().cpu().numpy()), 1e-2, "accumulated d(weight)")
