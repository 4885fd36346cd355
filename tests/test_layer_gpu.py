"""The sparse decoder layer of configuration 5 at a small shape: the operator chain against
a dense fp32 PyTorch reference, and the three execution variants against each other."""
import math

import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from intrasm_engine_amd.decoder_layer import SparseDecoderLayer
from intrasm_engine_amd.pytorch.utils import sparse_to_dense

pytestmark = pytest.mark.gpu
HIDDEN, HEADS, MLP, SEQS, L = 256, 4, 512, 4, 64


def reference_forward(weights_dense: dict, x: torch.Tensor, heads: int, seqs: int) -> torch.Tensor:
    """The same layer with dense fp32 matrices and plain PyTorch (for tests at small sizes).
    weights_dense: name -> (m, k) fp32 tensor; x: (hidden, tokens) fp32."""
    hidden = x.shape[0]
    hd = hidden // heads
    L = x.shape[1] // seqs

    def split(t):
        return t.view(heads, hd, seqs, L).permute(2, 0, 3, 1).reshape(seqs * heads, L, hd)

    q, k, v = (weights_dense[n] @ x for n in ("q", "k", "v"))
    Q, K, V = split(q), split(k), split(v)
    P = torch.softmax((Q @ K.transpose(1, 2)) / math.sqrt(hd), dim=-1)
    O = (P @ V).view(seqs, heads, L, hd).permute(1, 3, 0, 2).reshape(hidden, seqs * L)
    h = x + weights_dense["o"] @ O
    act = torch.nn.functional.silu(weights_dense["gate"] @ h) * (weights_dense["up"] @ h)
    return h + weights_dense["down"] @ act


def _layer(dev):
    weights = {}
    for i, name in enumerate(("q", "k", "v", "o")):
        weights[name] = W.pruned_weight(100 + i, HIDDEN, HIDDEN, "2:4", sigma=0.06)
    weights["gate"] = W.pruned_weight(104, MLP, HIDDEN, 0.80, sigma=0.06)
    weights["up"] = W.pruned_weight(105, MLP, HIDDEN, 0.80, sigma=0.06)
    weights["down"] = W.pruned_weight(106, HIDDEN, MLP, 0.80, sigma=0.06)
    return SparseDecoderLayer(weights, HIDDEN, HEADS, MLP, dev), weights


def test_layer_matches_dense_fp32_reference(dev):
    layer, weights = _layer(dev)
    x = torch.relu(torch.randn(HIDDEN, SEQS * L, generator=torch.Generator().manual_seed(0))).half().to(dev)
    y = layer.forward(x, SEQS)
    dense = {n: sparse_to_dense(c.m, c.k, torch.from_numpy(c.values).to(dev).half().float(),
                                torch.from_numpy(c.row_offsets).to(dev), torch.from_numpy(c.column_indices).to(dev))
             for n, c in weights.items()}
    want = reference_forward(dense, x.float(), HEADS, SEQS)
    assert y.shape == want.shape and torch.isfinite(y).all()
    err = (y.float() - want).abs().max().item()
    assert err <= 2e-2 * want.abs().max().item(), err       # fp16 chain of 9 operators


def test_three_variants_agree(dev):
    layer, _ = _layer(dev)
    g = torch.Generator().manual_seed(1)
    x = torch.relu(torch.randn(HIDDEN, SEQS * L, generator=g)).half().to(dev)
    half = SEQS * L // 2
    xa, xb = x[:, :half].contiguous(), x[:, half:].contiguous()
    ya, yb = layer.forward(xa, SEQS // 2), layer.forward(xb, SEQS // 2)
    # a sequence only attends inside itself: the full batch equals the two halves (up to the
    # summation order, which depends on how many nonzeros a wave handles at once for a given n)
    full = layer.forward(x, SEQS)
    assert torch.allclose(full[:, :half].float(), ya.float(), rtol=1e-2, atol=1e-2)
    assert torch.allclose(full[:, half:].float(), yb.float(), rtol=1e-2, atol=1e-2)

    for capture in (lambda: layer.capture_multistream(xa, xb, SEQS // 2),
                    lambda: layer.capture_fused(xa, xb, SEQS // 2, 0),
                    lambda: layer.capture_fused(xa, xb, SEQS // 2, 8),
                    lambda: layer.capture_fused(xa, xb, SEQS // 2)):
        constructor, keep = capture()
        constructor.instantiate_graph_exec()
        for _ in range(2):
            constructor.execute_graph()
            constructor.synchronize()
            outs = keep if isinstance(keep[0], torch.Tensor) else list(keep[0])
            assert torch.equal(outs[0], ya) and torch.equal(outs[1], yb)
        constructor.destroy_graph_exec()

    constructor, keep = layer.capture_serialized(x, SEQS)
    constructor.instantiate_graph_exec()
    constructor.execute_graph()
    constructor.synchronize()
    assert torch.equal(keep[0], full)
    constructor.destroy_graph_exec()
