"""Seeded synthetic inputs for the five benchmark configurations.

Everything is generated on the CPU with ``numpy.random.Generator(PCG64(seed))`` so the
same arrays can be rebuilt on any machine; callers move them to the device.  Index
arrays are int32 (``column_indices`` optionally int16 for the half kernels) and every
CSR produced here has strictly ascending columns inside each row.

Tuple order everywhere: ``(values, row_indices, row_offsets, column_indices)``, the
order of the reference's ``dense_to_sparse`` (pytorch/utils.py:147-153).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np


@dataclass
class CSR:
    m: int
    k: int
    values: np.ndarray          # (nnz,) float32 (callers cast to fp16 where needed)
    row_indices: np.ndarray     # (m,) int32, rows by decreasing length, stable
    row_offsets: np.ndarray     # (m+1,) int32
    column_indices: np.ndarray  # (nnz,) int32
    meta: dict = field(default_factory=dict)

    @property
    def nnz(self) -> int:
        return int(self.column_indices.shape[0])

    @property
    def sparsity(self) -> float:
        return 1.0 - self.nnz / (self.m * self.k)


def swizzle_from_offsets(row_offsets: np.ndarray) -> np.ndarray:
    """Rows ordered by decreasing nnz, ties in ascending row order."""
    lens = np.diff(row_offsets.astype(np.int64))
    return np.argsort(-lens, kind="stable").astype(np.int32)


def csr_from_row_lengths(rng: np.random.Generator, m: int, k: int, lens: np.ndarray):
    """Pattern with ``lens[r]`` distinct, sorted, uniformly drawn columns in row r."""
    lens = np.asarray(lens, dtype=np.int64)
    assert lens.shape == (m,) and lens.min() >= 0 and lens.max() <= k
    row_offsets = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(lens, out=row_offsets[1:])
    cols = np.empty(int(row_offsets[-1]), dtype=np.int32)
    # rank trick: the L smallest keys of a row of iid uniforms are a uniform L-subset
    step = max(1, (1 << 24) // max(k, 1))
    for r0 in range(0, m, step):
        r1 = min(m, r0 + step)
        keys = rng.random((r1 - r0, k), dtype=np.float32)
        order = np.argsort(keys, axis=1, kind="stable")
        for r in range(r0, r1):
            sel = np.sort(order[r - r0, : lens[r]])
            cols[row_offsets[r]: row_offsets[r + 1]] = sel
    return row_offsets.astype(np.int32), cols


def csr_from_mask(mask: np.ndarray, values_dense: np.ndarray | None = None):
    """Boolean (m,k) mask -> (row_offsets, column_indices[, values])."""
    m, k = mask.shape
    lens = mask.sum(axis=1).astype(np.int64)
    row_offsets = np.zeros(m + 1, dtype=np.int64)
    np.cumsum(lens, out=row_offsets[1:])
    cols = np.nonzero(mask)[1].astype(np.int32)
    vals = values_dense[mask].astype(np.float32) if values_dense is not None else None
    return row_offsets.astype(np.int32), cols, vals


def _nonzero_normal(rng, size, sigma):
    v = (rng.standard_normal(size, dtype=np.float32) * np.float32(sigma)).astype(np.float32)
    zero = v == 0
    while zero.any():
        v[zero] = (rng.standard_normal(int(zero.sum()), dtype=np.float32) * np.float32(sigma))
        zero = v == 0
    return v


def _nonzero_after_fp16(rng, size, sigma):
    """N(0, sigma) values none of which rounds to zero in fp16 (keeps nnz honest)."""
    v = _nonzero_normal(rng, size, sigma)
    tiny = v.astype(np.float16) == 0
    while tiny.any():
        v[tiny] = _nonzero_normal(rng, int(tiny.sum()), sigma)
        tiny = v.astype(np.float16) == 0
    return v


# --------------------------------------------------------------------------- C1
def config1(seed: int = 0, m: int = 1024, k: int = 1024, n: int = 256, kd: int = 64,
            sparsity: float = 0.90):
    """fp32 SpMM 1024x1024 @ 90 % (exactly round(k*(1-s)) nonzeros per row, uniform
    columns, values N(0,1)) times B 1024x256, plus the paired SDDMM operands
    (lhs 1024x64, rhs 1024x64, mask = A's pattern)."""
    rng = np.random.default_rng(seed)
    per_row = int(round(k * (1.0 - sparsity)))
    ro, ci = csr_from_row_lengths(rng, m, k, np.full(m, per_row))
    vals = _nonzero_normal(rng, ci.shape[0], 1.0)
    a = CSR(m, k, vals, swizzle_from_offsets(ro), ro, ci, {"config": "C1", "seed": seed})
    b = rng.standard_normal((1, k, n), dtype=np.float32)
    lhs = rng.standard_normal((1, m, kd), dtype=np.float32)
    rhs = rng.standard_normal((1, k, kd), dtype=np.float32)
    return a, b, lhs, rhs


# --------------------------------------------------------------------------- C2
C2_SPARSITIES = (0.70, 0.80, 0.90, 0.95, 0.98)
C2_NS = (64, 128, 256)


def geometric_row_lengths(rng, m, k, sparsity, even=False):
    """Row lengths ~ Geometric(p = 1/mean) clipped to [1,k], then rescaled and
    corrected so that they sum to round(m*k*(1-s)) exactly (each even if ``even``)."""
    target = int(round(m * k * (1.0 - sparsity)))
    mean = k * (1.0 - sparsity)
    unit = 2 if even else 1
    lo = unit
    lens = np.clip(rng.geometric(1.0 / mean, size=m), 1, k).astype(np.float64)
    lens = np.clip(np.rint(lens * (target / lens.sum()) / unit) * unit, lo, k - (k % unit)).astype(np.int64)
    target -= target % unit
    diff = target - int(lens.sum())
    order = rng.permutation(m)
    i = 0
    while diff != 0:
        r = order[i % m]
        i += 1
        if diff > 0 and lens[r] + unit <= k:
            lens[r] += unit
            diff -= unit
        elif diff < 0 and lens[r] - unit >= lo:
            lens[r] -= unit
            diff += unit
    return lens


def config2_matrix(sparsity: float, seed: int | None = None, m: int = 4096, k: int = 4096,
                   even_rows: bool = False, sigma: float = 0.02):
    """One matrix of the sweep: geometric (imbalanced) row lengths, sorted uniform
    columns, values N(0, sigma=0.02) none of which vanishes in fp16."""
    if seed is None:
        seed = 1 + C2_SPARSITIES.index(sparsity) if sparsity in C2_SPARSITIES else 1
    rng = np.random.default_rng(seed)
    lens = geometric_row_lengths(rng, m, k, sparsity, even=even_rows)
    ro, ci = csr_from_row_lengths(rng, m, k, lens)
    vals = _nonzero_after_fp16(rng, ci.shape[0], sigma)
    return CSR(m, k, vals, swizzle_from_offsets(ro), ro, ci,
               {"config": "C2", "seed": seed, "sparsity": sparsity})


def config2_dense(n: int, k: int = 4096, seed: int = 100):
    rng = np.random.default_rng(seed + n)
    return rng.standard_normal((1, k, n), dtype=np.float32)


# --------------------------------------------------------------------------- C3
def config3(seed: int = 10, tokens: int = 4096, head_dim: int = 64, heads: int = 16,
            band: int = 256, extra: int = 32):
    """Sparse-attention mask: |i-j| < band/2 plus ``extra`` uniform columns per row
    (duplicates merged).  Q, K, V are (heads, tokens, head_dim) N(0,1)."""
    rng = np.random.default_rng(seed)
    idx = np.arange(tokens)
    mask = np.abs(idx[:, None] - idx[None, :]) < (band // 2)
    if extra > 0:
        ext = rng.integers(0, tokens, size=(tokens, extra))
        mask[np.repeat(idx, extra), ext.ravel()] = True
    ro, ci, _ = csr_from_mask(mask)
    pattern = CSR(tokens, tokens, np.ones(ci.shape[0], np.float32), swizzle_from_offsets(ro), ro, ci,
                  {"config": "C3", "seed": seed})
    q = rng.standard_normal((heads, tokens, head_dim), dtype=np.float32)
    kk = rng.standard_normal((heads, tokens, head_dim), dtype=np.float32)
    v = rng.standard_normal((heads, tokens, head_dim), dtype=np.float32)
    return pattern, q, kk, v


# --------------------------------------------------------------------------- C4 / C5
def magnitude_prune(w: np.ndarray, sparsity: float):
    """Global unstructured magnitude pruning: keep |w| strictly above the quantile."""
    thr = np.quantile(np.abs(w).ravel(), sparsity, method="higher")
    mask = np.abs(w) > thr
    return mask


def two_four_mask(w: np.ndarray):
    """Keep the 2 largest |w| of every 4 consecutive entries along the last axis."""
    m, k = w.shape
    assert k % 4 == 0
    g = np.abs(w).reshape(m, k // 4, 4)
    order = np.argsort(-g, axis=2, kind="stable")
    mask = np.zeros_like(g, dtype=bool)
    np.put_along_axis(mask, order[:, :, :2], True, axis=2)
    return mask.reshape(m, k)


def pruned_weight(seed: int, m: int, k: int, sparsity: float | str, sigma: float = 0.02):
    """Random-init N(0, sigma) fp16-representable weight, pruned (``"2:4"`` or a
    global magnitude quantile) and returned as CSR."""
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((m, k), dtype=np.float32) * np.float32(sigma))
    w = w.astype(np.float16).astype(np.float32)
    w[w == 0] = np.float32(sigma)
    mask = two_four_mask(w) if sparsity == "2:4" else magnitude_prune(w, float(sparsity))
    ro, ci, vals = csr_from_mask(mask, w)
    return CSR(m, k, vals, swizzle_from_offsets(ro), ro, ci, {"seed": seed, "sparsity": sparsity})


def config4(seed: int = 20, m: int = 11008, k: int = 4096, tokens: int = 2048,
            gm: int = 4096, gk: int = 4096, sparsity: float = 0.90):
    """Sparse branch: 11008x4096 @ 90 % magnitude-pruned weight times X (4096 x tokens);
    dense branch: (gm x gk) @ (gk x tokens)."""
    rng = np.random.default_rng(seed + 1)
    w = pruned_weight(seed, m, k, sparsity)
    w.meta["config"] = "C4"
    x = rng.standard_normal((1, k, tokens), dtype=np.float32)
    ga = rng.standard_normal((gm, gk), dtype=np.float32)
    gb = rng.standard_normal((gk, tokens), dtype=np.float32)
    return w, x, ga, gb


def config5_weights(seed: int = 30, hidden: int = 4096, mlp: int = 11008):
    """LLaMA-7B-shaped layer weights: q/k/v/o 2:4, gate/up/down 80 % unstructured."""
    out = {}
    for i, name in enumerate(("q", "k", "v", "o")):
        out[name] = pruned_weight(seed + i, hidden, hidden, "2:4")
    out["gate"] = pruned_weight(seed + 4, mlp, hidden, 0.80)
    out["up"] = pruned_weight(seed + 5, mlp, hidden, 0.80)
    out["down"] = pruned_weight(seed + 6, hidden, mlp, 0.80)
    return out


def config5_activation(seed: int = 37, hidden: int = 4096, tokens: int = 16 * 512):
    """ReLU(N(0,1)) activations, stored feature-major (hidden, tokens) so that every
    projection is ``W_csr @ X``."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((1, hidden, tokens), dtype=np.float32)
    return np.maximum(x, 0.0)


# ------------------------------------------------------------------ work model
def spmm_bytes(m, k, n, nnz, batch=1, sv=4, si=4, per_batch_values=False):
    """Compulsory HBM traffic of one SpMM call: values + column indices once,
    row_offsets, the row swizzle, B read once, C written once."""
    vbytes = (batch if per_batch_values else 1) * nnz * sv
    return vbytes + nnz * si + (m + 1) * 4 + m * 4 + batch * (k * n + m * n) * sv


def spmm_flops(nnz, n, batch=1):
    return 2 * nnz * n * batch


def sddmm_bytes(m, k, n, nnz, batch=1, sv=4, sum_over_batch=True):
    out_elems = nnz if sum_over_batch else batch * nnz
    return nnz * 4 + (m + 1) * 4 + m * 4 + batch * (m * k + n * k) * sv + out_elems * sv


def sddmm_flops(nnz, k, batch=1):
    return 2 * nnz * k * batch


def gemm_bytes(M, N, K, sv=2):
    return (M * K + K * N + M * N) * sv


def gemm_flops(M, N, K):
    return 2 * M * N * K
