"""Graph builder: capture -> instantiate -> replay must reproduce eager results
(the invariant of the reference's tests/test_CUDAGraphConstructor.py:15-72 and
tests/test_CUDAGraphConstructor_event.py:12-150), plus structure and error paths."""
import numpy as np
import pytest
import torch

import intrasm_engine_amd
import intrasm_engine_amd.extensions as iex
from intrasm_engine_amd import interleaving as IL
from intrasm_engine_amd import workloads as W
from intrasm_engine_amd.pytorch.cpp_extensions.cuda_graph_constructor import TorchCUDAGraphConstructor
from _util import to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops
KERNEL_NODE, EMPTY_NODE = 0, 5          # hipGraphNodeTypeKernel, hipGraphNodeTypeEmpty


def _replay(torch_func, a, b):
    c_ref = torch_func(a, b)
    constructor = TorchCUDAGraphConstructor()
    constructor.capture_library_call_begin()
    c = torch_func(a, b)
    constructor.capture_library_call_end()
    constructor.instantiate_graph_exec()
    constructor.execute_graph()
    constructor.synchronize()
    constructor.destroy_graph_exec()
    assert torch.allclose(c, c_ref)
    return constructor


def test_replay_torch_matmul(dev):
    _replay(torch.matmul, torch.randn(512, 512, device=dev), torch.randn(512, 512, device=dev))


def test_replay_torch_matmul_batched_and_linear(dev):
    a, b = torch.randn(64, 512, 512, device=dev), torch.randn(512, 512, device=dev)
    _replay(torch.matmul, a, b)
    _replay(torch.nn.functional.linear, a, b)
    _replay(lambda x, w: torch.nn.functional.linear(x[2:34], w), a, b)


def test_replay_own_operators_several_times(dev):
    """Replays are repeated with eager work and synchronisations in between; every replay
    must reproduce the eager result after the inputs were overwritten in place."""
    a = W.config2_matrix(0.90, m=1024, k=1024)
    ri, v, ro, ci = to_dev(a, dev)
    b = torch.randn(1, 1024, 128, device=dev)
    ga = torch.randint(-3, 3, (256, 256), device=dev).bfloat16()
    gb = torch.randint(-3, 3, (256, 256), device=dev).bfloat16()
    constructor = TorchCUDAGraphConstructor()
    with constructor.get_primary_stream():
        with constructor:
            out = ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, a.m)
            c = ops.gemm_mfma(ga, gb, False)
    constructor.instantiate_graph_exec()
    for it in range(4):
        b.copy_(torch.randn(1, 1024, 128, device=dev))
        ga.copy_(torch.randint(-3, 3, (256, 256), device=dev).bfloat16())
        torch.cuda.synchronize()
        constructor.execute_graph()
        constructor.synchronize()
        assert torch.equal(out, ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, a.m)), it
        assert torch.equal(c, ops.gemm_mfma(ga, gb, False)), it
    constructor.destroy_graph_exec()


def test_replay_spmm_that_uses_a_workspace(dev):
    """A 16-bit product large enough for the dense-form path: the operator takes its workspace from
    the allocator inside the capture, so it must come from the capture's pool and stay out of the
    hands of tensors created between the replays."""
    from intrasm_engine_amd import _lib
    rng = np.random.default_rng(3)
    m = k = 2048
    n = 1024
    ro, ci = W.csr_from_row_lengths(rng, m, k, rng.binomial(k, 0.2, m))
    ri = torch.from_numpy(W.swizzle_from_offsets(ro)).to(dev)
    ro_t, ci_t = torch.from_numpy(ro).to(dev), torch.from_numpy(ci.astype(np.int16)).to(dev)
    from intrasm_engine_amd.pytorch import ops as pyops
    pyops.prepare_pattern(ro_t, ci_t, k)     # set-up code looks at a pattern once, outside any capture
    v = torch.randn(ci.shape[0], device=dev).half()
    b = torch.randn(1, k, n, device=dev).half()
    assert _lib.load().iex_spmm_workspace_bytes(_lib.F16, _lib.I16, 0, m, k, n, ci.shape[0], 1) == m * k * 2
    constructor = TorchCUDAGraphConstructor()
    with constructor.get_primary_stream():
        with constructor:
            out = ops.spmm_sputnik_reuse_weight_half(b, ri, v, ro_t, ci_t, m)
    constructor.instantiate_graph_exec()
    for it in range(4):
        b.copy_(torch.randn(1, k, n, device=dev).half())
        clutter = [torch.full((m * k,), float(it), device=dev, dtype=torch.float16) for _ in range(3)]
        torch.cuda.synchronize()
        constructor.execute_graph()
        constructor.synchronize()
        assert torch.equal(out, ops.spmm_sputnik_reuse_weight_half(b, ri, v, ro_t, ci_t, m)), it
        assert all(bool((t == float(it)).all()) for t in clutter), it
    constructor.destroy_graph_exec()


def test_two_branches_join_structure_and_results(dev, tmp_path):
    a = W.config2_matrix(0.95, m=512, k=512)
    ri, v, ro, ci = to_dev(a, dev)
    b = torch.randn(1, 512, 64, device=dev)
    ga = torch.randint(-3, 3, (128, 128), device=dev).half()
    gb = torch.randint(-3, 3, (128, 128), device=dev).half()
    n_rep = 3
    constructor, keep = IL.capture_interleaved([lambda: ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, a.m)] * n_rep,
                                               [lambda: ops.gemm_mfma(ga, gb, False)] * n_rep)
    g = constructor.constructor
    types = g.node_types()
    edges = g.edges()
    assert types.count(KERNEL_NODE) == 2 * n_rep
    assert types.count(EMPTY_NODE) == 2                      # root + join
    # root has two successors (one per branch), the join node two predecessors, and no edge
    # connects a kernel of one branch to a kernel of the other
    succ, pred = {}, {}
    for f, t in edges:
        succ.setdefault(f, []).append(t)
        pred.setdefault(t, []).append(f)
    roots = [i for i, ty in enumerate(types) if ty == EMPTY_NODE and i not in pred]
    joins = [i for i, ty in enumerate(types) if ty == EMPTY_NODE and i not in succ]
    assert len(roots) == 1 and len(joins) == 1
    assert len(succ[roots[0]]) == 2 and len(pred[joins[0]]) == 2
    assert len(edges) == 2 * n_rep + 2                       # two chains of n_rep kernels + join edges

    def chain(start):
        seen = []
        while types[start] == KERNEL_NODE:
            seen.append(start)
            (start,) = succ[start]
        return seen, start
    c0, e0 = chain(succ[roots[0]][0])
    c1, e1 = chain(succ[roots[0]][1])
    assert len(c0) == n_rep and len(c1) == n_rep and not set(c0) & set(c1) and e0 == e1 == joins[0]

    constructor.instantiate_graph_exec()
    constructor.execute_graph()
    constructor.synchronize()
    for t in keep[:n_rep]:
        assert torch.equal(t, ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, a.m))
    for t in keep[n_rep:]:
        assert torch.equal(t.double(), ga.double() @ gb.double())
    dot = tmp_path / "graph.dot"
    constructor.dump_graph(str(dot))
    assert dot.stat().st_size > 0
    constructor.print_graph()
    constructor.destroy_graph_exec()


def test_event_record_and_wait_nodes(dev):
    """Two streams ordered by an explicit event node: the second GEMM consumes the first
    one's output (tests/test_CUDAGraphConstructor_event.py pattern)."""
    constructor = TorchCUDAGraphConstructor()
    s1 = constructor.register_new_stream()
    s0 = constructor.get_primary_stream()
    a = torch.randint(-2, 3, (256, 256), device=dev).half()
    ev = torch.cuda.Event()
    ev.record()                       # torch creates the event lazily
    torch.cuda.synchronize()
    with s0:
        constructor.capture_library_call_begin()
        x = ops.gemm_mfma(a, a, False)
        constructor.capture_library_call_end()
    constructor.add_event_record_node(ev, s0.torch_stream)
    constructor.add_stream_wait_event_node(s1.torch_stream, ev)
    with s1:
        constructor.capture_library_call_begin()
        y = ops.gemm_mfma(x, a, True)
        constructor.capture_library_call_end()
    constructor.join([s1], s0)
    constructor.instantiate_graph_exec()
    for _ in range(2):
        constructor.execute_graph()
        constructor.synchronize()
        xr = (a.double() @ a.double())
        assert torch.equal(x.double(), xr.half().double())
        assert torch.equal(y, ops.gemm_mfma(x, a, True))
    constructor.destroy_graph_exec()
    with pytest.raises(AssertionError, match="Event uninitialized"):
        constructor.add_event_record_node(torch.cuda.Event(), s0.torch_stream)


def test_child_graphs_and_combine(dev):
    a = torch.randn(128, 128, device=dev)
    c1, k1 = IL.capture_serialized([lambda: a @ a])
    c2, k2 = IL.capture_serialized([lambda: a + 1])
    merged = c1.constructor.combine_graphs(c2.constructor)
    assert merged.num_nodes() == 2
    merged.instantiate_graph_exec()
    k1[0].zero_(), k2[0].zero_()
    merged.execute_graph(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.allclose(k1[0], a @ a) and torch.equal(k2[0], a + 1)
    merged.destroy_graph_exec()
    parent = iex.CUDAExperimentalGraphConstructor()
    parent.add_graph_as_child_node(c1.constructor)
    assert parent.num_nodes() == 2 and parent.num_edges() == 1


def test_error_paths(dev):
    constructor = TorchCUDAGraphConstructor()
    # capture on an unregistered stream
    with torch.cuda.stream(torch.cuda.Stream()):
        with pytest.raises(AssertionError, match="not registered"):
            constructor.capture_library_call_begin()
    # capture on the default stream is refused before anything starts
    with torch.cuda.stream(torch.cuda.default_stream()):
        n = iex.CUDAGraphCaptureNotifier()
        with pytest.raises(RuntimeError, match="non-default stream"):
            n.capture_begin(None)
    # launching before instantiation, instantiating twice
    with pytest.raises(RuntimeError, match="not instantiated"):
        constructor.execute_graph()
    constructor.instantiate_graph_exec()
    with pytest.raises(RuntimeError, match="already instantiated"):
        constructor.instantiate_graph_exec()
    constructor.destroy_graph_exec()
    constructor.destroy_graph_exec()    # idempotent
    # ending a capture that never began
    with pytest.raises(RuntimeError):
        constructor.capture_library_call_end()
    # the allocator is still usable afterwards
    assert torch.ones(4, device=dev).sum().item() == 4


def test_handle_round_trip(dev, capsys):
    s = torch.cuda.current_stream().cuda_stream
    assert iex.print_cudastream(s) == s
    assert iex.print_cudastream([s, s]) == [s, s]
    ev = torch.cuda.Event()
    ev.record()
    assert iex.print_cudaevent(ev.cuda_event) == ev.cuda_event
    with pytest.raises(RuntimeError, match="null"):
        iex.print_cudaevent(0)
    assert "stream" in capsys.readouterr().out


def test_current_stream_is_not_the_default_stream(dev):
    cs = intrasm_engine_amd.current_stream[torch.device("cuda:0")]
    assert cs.stream == torch.cuda.current_stream()
    assert cs.stream != torch.cuda.default_stream()


@pytest.mark.parametrize("tables_from", ["capture_pool", "plan", "pattern"])
def test_replay_sparse_attention_with_tables_in_the_captured_workspace(dev, tables_from):
    """The attention block on a mask with structure, captured: the workspace with the tables and lists of the two
    kernels for such masks comes from the capture's pool (the block's own plan), or is the caller's plan, filled before
    the capture, or is kept with the pattern since set-up code looked at it; the second product inside the capture
    reuses what the first wrote.  Replays with new q, k, v (and other allocations between them) equal the eager block
    bit for bit."""
    kept_plan = tables_from == "plan"
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    from intrasm_engine_amd.pytorch.sparse_attention import sparse_attention
    pattern, q_np, k_np, _ = W.config3(tokens=2048, heads=8, band=128, extra=8)     # (large and dense enough for the structured kernels to be picked)
    ri, _, ro, ci = to_dev(pattern, dev, tables=tables_from == "pattern")
    heads, tokens, d = q_np.shape
    q, k, v = (torch.randn(heads, tokens, d, device=dev).half() for _ in range(3))
    plan = None
    if kept_plan:
        plan = pyops.SddmmPlan()
        plan.variant = 3
        sparse_attention(q, k, v, ri, ro, ci, plan=plan)           # tables and lists are in the plan before the capture
    constructor = TorchCUDAGraphConstructor()
    with constructor.get_primary_stream():
        with constructor:
            out = sparse_attention(q, k, v, ri, ro, ci, plan=plan)
    assert "spmm_blocks_kernel" in _lib.last_kernels()
    constructor.instantiate_graph_exec()
    for it in range(4):
        for t in (q, k, v):
            t.copy_(torch.randn(heads, tokens, d, device=dev).half())
        clutter = [torch.full((1 << 22,), float(it), device=dev, dtype=torch.float16) for _ in range(3)]
        torch.cuda.synchronize()
        constructor.execute_graph()
        constructor.synchronize()
        eager_plan = None
        if kept_plan:                     # (the same kernels as the captured calls: the plan settles the SDDMM's)
            eager_plan = pyops.SddmmPlan()
            eager_plan.variant = 3
        assert torch.equal(out, sparse_attention(q, k, v, ri, ro, ci, plan=eager_plan)), it
        assert all(bool((t == float(it)).all()) for t in clutter), it
    constructor.destroy_graph_exec()
