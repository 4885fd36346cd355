"""Configurations 4 and 5 at their real sizes.

Config 5 (hidden 4096, MLP 11008, 16 x 512 = 8192 tokens, fp16, int16 column indices): each of the seven
projections' SpMM (q/k/v/o at 2:4, gate/up/down at 80 % unstructured) against the CPU oracle on a strided
sample of output rows (the oracle on 32 rows x 8192 columns is seconds of CPU work), for the kernel the
operator picks (dense form + GEMM) and for the one the workspace-free entry point picks; then the three
schedules of the whole layer (serialized, two-stream graph, fused) against each other, bit for bit.
Config 4: the two-branch graph (fp16 SpMM 11008 x 4096 at 90 % x 2048 tokens beside a bf16 GEMM
4096 x 4096 x 2048) replayed, both results against the oracle on a sample of rows and against the eager
operators bit for bit.
"""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import interleaving as IL
from intrasm_engine_amd import workloads as W
from _util import assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops
HIDDEN, HEADS, MLP, SEQS, L = 4096, 32, 11008, 16, 512
SAMPLE_STRIDE = {4096: 131, 11008: 349}         # 32 rows of either height


@pytest.fixture(scope="module")
def weights():
    return W.config5_weights()


def _sub_csr(c, rows):
    """The CSR matrix made of the given rows of c (natural order; the swizzle only schedules)."""
    lens = (c.row_offsets[1:] - c.row_offsets[:-1])[rows]
    ro = np.zeros(len(rows) + 1, dtype=np.int32)
    np.cumsum(lens, out=ro[1:])
    take = np.concatenate([np.arange(c.row_offsets[r], c.row_offsets[r + 1]) for r in rows])
    return ro, c.column_indices[take], c.values[take]


@pytest.mark.parametrize("name", ["q", "k", "v", "o", "gate", "up", "down"])
def test_config5_projection_against_the_oracle(dev, oracle, weights, name):
    from intrasm_engine_amd.pytorch import ops as pyops
    c = weights[name]
    g = torch.Generator().manual_seed(50 + ["q", "k", "v", "o", "gate", "up", "down"].index(name))
    x = torch.relu(torch.randn(1, c.k, SEQS * L, generator=g)).half()         # activations N(0,1) through ReLU
    x_np = x.float().numpy()
    xd = x.to(dev)
    rows = np.arange(0, c.m, SAMPLE_STRIDE[c.m])
    sro, sci, svals = _sub_csr(c, rows)
    sub = W.CSR(len(rows), c.k, svals, W.swizzle_from_offsets(sro), sro, sci)
    want = oracle.spmm(x_np, sub.row_indices, rounded(svals, torch.float16), sro, sci, sub.m)[0]
    scale = oracle.spmm_abs_scale(x_np, sub.row_indices, svals, sro, sci, sub.m)[0]
    pick = torch.from_numpy(rows).to(dev)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float16,), allow_i16=True)

    ri, v, ro, ci = to_dev(c, dev, torch.float16, torch.int16)
    out = ops.spmm_sputnik_reuse_weight_half(xd, ri, v, ro, ci, c.m)          # what the layer calls
    assert out.shape == (1, c.m, SEQS * L)
    assert_close(out[0][pick].float().cpu().numpy(), want, scale, 1e-2, f"{name}: operator")
    bare = pyops._spmm(xd, ri, v, ro, ci, c.m, no_workspace=True, **kw)       # the C launcher's path (no workspace)
    assert_close(bare[0][pick].float().cpu().numpy(), want, scale, 1e-2, f"{name}: without workspace")
    # the gather kernel on the same rows, through the sub-matrix (an independent family: fp32 FMA chain)
    sri, sv, sro_t, sci_t = to_dev(sub, dev, torch.float16, torch.int16)
    gather = pyops._spmm(xd, sri, sv, sro_t, sci_t, sub.m, force_variant=1, **kw)
    assert_close(gather[0].float().cpu().numpy(), want, scale, 1e-2, f"{name}: row kernel")


def test_config5_layer_three_schedules_agree(dev, weights):
    from intrasm_engine_amd.decoder_layer import SparseDecoderLayer
    layer = SparseDecoderLayer(weights, HIDDEN, HEADS, MLP, dev)
    x = torch.from_numpy(W.config5_activation(hidden=HIDDEN, tokens=SEQS * L)[0]).to(dev).half()
    half = SEQS * L // 2
    xa, xb = x[:, :half].contiguous(), x[:, half:].contiguous()
    ya, yb = layer.forward(xa, SEQS // 2), layer.forward(xb, SEQS // 2)
    full = layer.forward(x, SEQS)
    assert torch.isfinite(full).all() and float(full.float().abs().max()) > 0
    # a sequence attends only inside itself: the whole batch equals its halves up to the summation order
    # of the kernels picked for 8192 and for 4096 tokens
    tol = 1e-2 * float(full.float().abs().max())
    assert torch.allclose(full[:, :half].float(), ya.float(), rtol=1e-2, atol=tol)
    assert torch.allclose(full[:, half:].float(), yb.float(), rtol=1e-2, atol=tol)

    constructor, keep = layer.capture_serialized(x, SEQS)
    constructor.instantiate_graph_exec()
    for _ in range(2):
        constructor.execute_graph()
        constructor.synchronize()
        assert torch.equal(keep[0], full)
    constructor.destroy_graph_exec()
    del constructor, keep

    for what, capture in (("two streams", lambda: layer.capture_multistream(xa, xb, SEQS // 2)),
                          ("fused", lambda: layer.capture_fused(xa, xb, SEQS // 2, 0)),
                          ("fused, groups of 8", lambda: layer.capture_fused(xa, xb, SEQS // 2, 8))):
        constructor, keep = capture()
        constructor.instantiate_graph_exec()
        for _ in range(2):
            constructor.execute_graph()
            constructor.synchronize()
            outs = keep if isinstance(keep[0], torch.Tensor) else list(keep[0])
            assert torch.equal(outs[0], ya) and torch.equal(outs[1], yb), what
        constructor.destroy_graph_exec()
        del constructor, keep


def test_config4_two_branch_graph_results(dev, oracle):
    w, x, ga, gb = W.config4()
    ri, v, ro, ci = to_dev(w, dev, torch.float16, torch.int16)
    xt = torch.from_numpy(x).to(dev).half()
    gat, gbt = torch.from_numpy(ga).to(dev).bfloat16(), torch.from_numpy(gb).to(dev).bfloat16()
    eager_s = ops.spmm_sputnik_reuse_weight_half(xt, ri, v, ro, ci, w.m)
    eager_g = ops.gemm_mfma(gat, gbt, False)
    reps = 2
    constructor, keep = IL.capture_interleaved([lambda: ops.spmm_sputnik_reuse_weight_half(xt, ri, v, ro, ci, w.m)] * reps,
                                               [lambda: ops.gemm_mfma(gat, gbt, False)] * reps)
    constructor.instantiate_graph_exec()
    for _ in range(2):
        for t in keep:
            t.zero_()
        torch.cuda.synchronize()
        constructor.execute_graph()
        constructor.synchronize()
        for t in keep[:reps]:
            assert torch.equal(t, eager_s)
        for t in keep[reps:]:
            assert torch.equal(t, eager_g)
    constructor.destroy_graph_exec()
    # against the oracle: the sparse branch on a strided sample of rows, the dense branch on a sample of rows
    x16 = rounded(x, torch.float16)
    rows = np.arange(0, w.m, 349)
    sro, sci, svals = _sub_csr(w, rows)
    ident = np.arange(len(rows), dtype=np.int32)
    want = oracle.spmm(x16, ident, rounded(svals, torch.float16), sro, sci, len(rows))
    scale = oracle.spmm_abs_scale(x16, ident, svals, sro, sci, len(rows))
    assert_close(keep[0][0][torch.from_numpy(rows).to(dev)].float().cpu().numpy(), want[0], scale[0], 1e-2, "config 4 SpMM branch")
    grow = np.arange(0, 4096, 67)
    a16, b16 = rounded(ga[grow], torch.bfloat16), rounded(gb, torch.bfloat16)
    want_g = oracle.gemm(a16, b16)
    scale_g = np.abs(a16).astype(np.float64) @ np.abs(b16).astype(np.float64)
    assert_close(keep[reps][torch.from_numpy(grow).to(dev)].float().cpu().numpy(), want_g, scale_g, 1e-2, "config 4 GEMM branch")
