"""Pins the CPU oracle to things that are NOT its own formula.

The reference holds no golden vector for SpMM / SDDMM (its tests only look the operators
up); the one worked sparse example it contains is the 3x4 matrix of
tests/test_cuda_python_interop.py:79-86.  Everything else is pinned by independent
implementations (scipy CSR, torch.sparse, numpy float64 matmul on the scattered matrix),
brute-force Python loops on tiny inputs, special cases that reduce to textbook
operations, and invariants chosen so that a dropped term, a transposed operand or a
wrong index breaks at least one of them.
"""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from intrasm_engine_amd import workloads as W


def _random_csr(rng, m, k, density, empty_rows=()):
    mask = rng.random((m, k)) < density
    for r in empty_rows:
        mask[r] = False
    dense = np.where(mask, rng.standard_normal((m, k)), 0.0).astype(np.float32)
    return dense


# ------------------------------------------------------------------ CSR build
@pytest.mark.parametrize("shape,density", [((7, 5), 0.5), ((64, 33), 0.1), ((33, 64), 0.9), ((16, 16), 0.0)])
def test_dense_to_csr_matches_scipy(oracle, shape, density):
    rng = np.random.default_rng(3)
    dense = _random_csr(rng, *shape, density, empty_rows=(0,) if shape[0] > 8 else ())
    values, ri, ro, ci = oracle.dense_to_csr(dense)
    ref = sp.csr_matrix(dense)
    ref.sort_indices()
    assert np.array_equal(ro, ref.indptr)
    assert np.array_equal(ci, ref.indices)
    assert np.array_equal(values, ref.data)
    # swizzle: permutation, non-increasing length, ties in ascending row order
    lens = np.diff(ro)
    assert sorted(ri.tolist()) == list(range(shape[0]))
    assert (np.diff(lens[ri]) <= 0).all()
    for a, b in zip(ri[:-1], ri[1:]):
        if lens[a] == lens[b]:
            assert a < b
    # round trip is exact
    assert np.array_equal(oracle.csr_to_dense(shape[0], shape[1], values, ro, ci), dense.astype(np.float64))


def test_csr_transpose_matches_scipy(oracle):
    rng = np.random.default_rng(4)
    dense = _random_csr(rng, 37, 53, 0.2, empty_rows=(5,))
    values, ri, ro, ci = oracle.dense_to_csr(dense)
    ro_t, ci_t, perm = oracle.csr_transpose(37, 53, ro, ci)
    ref = sp.csr_matrix(dense).T.tocsr()
    ref.sort_indices()
    assert np.array_equal(ro_t, ref.indptr)
    assert np.array_equal(ci_t, ref.indices)
    assert np.array_equal(values[perm], ref.data)
    # transposing twice is the identity
    ro_tt, ci_tt, perm2 = oracle.csr_transpose(53, 37, ro_t, ci_t)
    assert np.array_equal(ro_tt, ro) and np.array_equal(ci_tt, ci)
    assert np.array_equal(perm[perm2], np.arange(len(ci)))


# ----------------------------------------------------------------------- SpMM
def test_spmm_reference_3x4_example(oracle):
    """The sparse example of the reference's tests/test_cuda_python_interop.py:79-86:
    CSC data [0,1,3,2], indices [0,0,2,1], indptr [0,1,2,3,4], shape 3x4, i.e. the matrix
    [[0,1,0,0],[0,0,0,2],[0,0,3,0]] (the stored 0 is kept), times [[1,1],[2,2],[3,3],[4,4]]."""
    x = sp.csc_matrix((np.array([0, 1, 3, 2], float), np.array([0, 0, 2, 1]), np.array([0, 1, 2, 3, 4])), shape=(3, 4))
    assert np.array_equal(x.toarray(), [[0, 1, 0, 0], [0, 0, 0, 2], [0, 0, 3, 0]])
    y = np.array([[1, 2, 3, 4], [1, 2, 3, 4]], float).T
    values, ri, ro, ci = oracle.dense_to_csr(x.toarray())
    out = oracle.spmm(y[None], ri, values, ro, ci, 3)[0]
    assert np.array_equal(out, [[2, 2], [8, 8], [9, 9]])      # worked by hand
    assert np.array_equal(out, x @ y)


@pytest.mark.parametrize("m,k,n,density,batch", [(9, 7, 5, 0.4, 1), (50, 40, 33, 0.15, 3), (40, 64, 64, 0.9, 2)])
def test_spmm_matches_scipy_torch_and_dense(oracle, m, k, n, density, batch):
    rng = np.random.default_rng(5)
    dense_a = _random_csr(rng, m, k, density, empty_rows=(1,))
    values, ri, ro, ci = oracle.dense_to_csr(dense_a)
    b = rng.standard_normal((batch, k, n)).astype(np.float32)
    out = oracle.spmm(b, ri, values, ro, ci, m)
    a_sp = sp.csr_matrix((values.astype(np.float64), ci, ro), shape=(m, k))
    a_t = torch.sparse_csr_tensor(torch.from_numpy(ro).long(), torch.from_numpy(ci).long(),
                                  torch.from_numpy(values).double(), size=(m, k))
    for z in range(batch):
        assert np.allclose(out[z], a_sp @ b[z].astype(np.float64), rtol=1e-12, atol=1e-12)
        assert np.allclose(out[z], dense_a.astype(np.float64) @ b[z].astype(np.float64), rtol=1e-12, atol=1e-12)
        assert np.allclose(out[z], (a_t @ torch.from_numpy(b[z]).double()).numpy(), rtol=1e-12, atol=1e-12)
    assert (out[:, 1] == 0).all()  # the empty row


def test_spmm_brute_force_tiny(oracle):
    rng = np.random.default_rng(6)
    m, k, n = 4, 5, 3
    ro = np.array([0, 2, 2, 5, 6], np.int32)
    ci = np.array([1, 4, 0, 2, 3, 4], np.int32)
    vals = rng.integers(-3, 4, 6).astype(np.float32)
    b = rng.integers(-3, 4, (2, k, n)).astype(np.float32)
    ri = np.array([2, 0, 3, 1], np.int32)
    want = np.zeros((2, m, n))
    for z in range(2):
        for r in range(m):
            for j in range(ro[r], ro[r + 1]):
                for c in range(n):
                    want[z, r, c] += float(vals[j]) * float(b[z, ci[j], c])
    assert np.array_equal(oracle.spmm(b, ri, vals, ro, ci, m), want)
    assert np.array_equal(oracle.spmm_f32(b, ri, vals, ro, ci, m), want.astype(np.float32))


def test_spmm_special_cases(oracle):
    rng = np.random.default_rng(7)
    k, n = 12, 10
    b = rng.standard_normal((1, k, n)).astype(np.float32)
    # identity -> copy
    v, ri, ro, ci = oracle.dense_to_csr(np.eye(k, dtype=np.float32))
    assert np.array_equal(oracle.spmm(b, ri, v, ro, ci, k)[0], b[0].astype(np.float64))
    # permutation -> row gather
    perm = rng.permutation(k)
    p = np.zeros((k, k), np.float32)
    p[np.arange(k), perm] = 1
    v, ri, ro, ci = oracle.dense_to_csr(p)
    assert np.array_equal(oracle.spmm(b, ri, v, ro, ci, k)[0], b[0][perm].astype(np.float64))
    # one nonzero per row -> scaled gather
    p2 = p * np.arange(1, k + 1, dtype=np.float32)[:, None]
    v, ri, ro, ci = oracle.dense_to_csr(p2)
    assert np.array_equal(oracle.spmm(b, ri, v, ro, ci, k)[0],
                          b[0][perm].astype(np.float64) * np.arange(1, k + 1)[:, None])
    # fully dense -> GEMM
    d = rng.standard_normal((6, k)).astype(np.float32)
    v, ri, ro, ci = oracle.dense_to_csr(d)
    assert np.allclose(oracle.spmm(b, ri, v, ro, ci, 6)[0], d.astype(np.float64) @ b[0].astype(np.float64), rtol=1e-13)
    assert np.allclose(oracle.spmm(b, ri, v, ro, ci, 6)[0], oracle.gemm(d, b[0]), rtol=1e-13)
    # all-empty matrix -> zeros
    v, ri, ro, ci = oracle.dense_to_csr(np.zeros((5, k), np.float32))
    assert (oracle.spmm(b, ri, v, ro, ci, 5) == 0).all()


def test_spmm_invariants(oracle):
    rng = np.random.default_rng(8)
    m, k, n = 30, 20, 8
    dense_a = _random_csr(rng, m, k, 0.3)
    v, ri, ro, ci = oracle.dense_to_csr(dense_a)
    b = rng.standard_normal((3, k, n)).astype(np.float32)
    base = oracle.spmm(b, ri, v, ro, ci, m)
    # any permutation of the swizzle gives the same result (it only schedules)
    assert np.array_equal(oracle.spmm(b, rng.permutation(m).astype(np.int32), v, ro, ci, m), base)
    # batch entries are independent
    assert np.array_equal(oracle.spmm(b[1:2], ri, v, ro, ci, m)[0], base[1])
    # linear in values (exact in double for power-of-two scaling)
    assert np.array_equal(oracle.spmm(b, ri, 2 * v, ro, ci, m), 2 * base)
    # per-batch values = one call per batch entry
    vb = np.stack([v, 2 * v, -v])
    per = oracle.spmm(b, ri, vb, ro, ci, m)
    assert np.array_equal(per[0], base[0]) and np.array_equal(per[1], 2 * base[1]) and np.array_equal(per[2], -base[2])
    # accumulate mode adds to what the output holds
    init = rng.standard_normal(base.shape)
    assert np.allclose(oracle.spmm(b, ri, v, ro, ci, m, out_init=init), init + base, rtol=1e-13, atol=1e-13)
    # bias + relu epilogue
    bias = rng.standard_normal(m).astype(np.float32)
    assert np.allclose(oracle.spmm(b, ri, v, ro, ci, m, bias=bias, relu=True),
                       np.maximum(base + bias.astype(np.float64)[None, :, None], 0), rtol=1e-13, atol=1e-13)
    # float-accumulate port agrees with the double one to fp32 accuracy
    scale = oracle.spmm_abs_scale(b, ri, v, ro, ci, m)
    assert (np.abs(oracle.spmm_f32(b, ri, v, ro, ci, m) - base) <= 1e-6 * scale + 1e-30).all()


# ---------------------------------------------------------------------- SDDMM
@pytest.mark.parametrize("m,n,k,density,batch", [(9, 7, 5, 0.4, 1), (40, 30, 64, 0.2, 3)])
def test_sddmm_matches_dense(oracle, m, n, k, density, batch):
    rng = np.random.default_rng(9)
    mask = _random_csr(rng, m, n, density, empty_rows=(2,))
    _, ri, ro, ci = oracle.dense_to_csr(mask)
    a = rng.standard_normal((batch, m, k)).astype(np.float32)
    b = rng.standard_normal((batch, n, k)).astype(np.float32)
    rows = np.repeat(np.arange(m), np.diff(ro))
    full = np.einsum("zmk,znk->zmn", a.astype(np.float64), b.astype(np.float64))  # a @ b^T: b is (n,k)
    per = oracle.sddmm(a, b, ri, ro, ci, sum_over_batch=False)
    assert np.allclose(per, full[:, rows, ci], rtol=1e-12, atol=1e-12)
    summed = oracle.sddmm(a, b, ri, ro, ci, sum_over_batch=True)
    assert np.allclose(summed, full[:, rows, ci].sum(0), rtol=1e-12, atol=1e-12)
    assert np.allclose(oracle.sddmm_f32(a, b, ri, ro, ci, sum_over_batch=False), per, rtol=1e-4, atol=1e-4)
    init = rng.standard_normal(summed.shape)
    assert np.allclose(oracle.sddmm(a, b, ri, ro, ci, out_init=init), init + summed, rtol=1e-12, atol=1e-12)


def test_sddmm_special_masks(oracle):
    rng = np.random.default_rng(10)
    m, k = 12, 16
    a = rng.standard_normal((1, m, k)).astype(np.float32)
    b = rng.standard_normal((1, m, k)).astype(np.float32)
    # full mask -> dense GEMM with B transposed
    _, ri, ro, ci = oracle.dense_to_csr(np.ones((m, m), np.float32))
    assert np.allclose(oracle.sddmm(a, b, ri, ro, ci).reshape(m, m), oracle.gemm(a[0], b[0], trans_b=True), rtol=1e-13)
    # diagonal mask -> row-wise dot products
    _, ri, ro, ci = oracle.dense_to_csr(np.eye(m, dtype=np.float32))
    assert np.allclose(oracle.sddmm(a, b, ri, ro, ci), (a[0].astype(np.float64) * b[0]).sum(1), rtol=1e-13)
    # a transposed operand would fail this: non-square, asymmetric
    a2 = rng.standard_normal((1, 3, k)).astype(np.float32)
    b2 = rng.standard_normal((1, 5, k)).astype(np.float32)
    _, ri, ro, ci = oracle.dense_to_csr(np.array([[0, 0, 0, 0, 1], [1, 0, 0, 0, 0], [0, 0, 1, 1, 0]], np.float32))
    want = [a2[0, 0].astype(np.float64) @ b2[0, 4], a2[0, 1].astype(np.float64) @ b2[0, 0],
            a2[0, 2].astype(np.float64) @ b2[0, 2], a2[0, 2].astype(np.float64) @ b2[0, 3]]
    assert np.allclose(oracle.sddmm(a2, b2, ri, ro, ci), want, rtol=1e-13)


def test_sddmm_is_the_values_gradient_of_spmm(oracle):
    """d/d(values) sum(G * (A @ B)) = SDDMM(mask, G, B^T-rows): the relation MySpMM's backward
    relies on (layers_and_funcs/sputnik.py:103-114).  Checked against torch autograd on the
    dense formulation."""
    rng = np.random.default_rng(11)
    m, k, n = 10, 8, 6
    dense_a = _random_csr(rng, m, k, 0.4)
    v, ri, ro, ci = oracle.dense_to_csr(dense_a)
    b = rng.standard_normal((k, n)).astype(np.float32)
    g = rng.standard_normal((m, n)).astype(np.float32)
    at = torch.tensor(dense_a, dtype=torch.float64, requires_grad=True)
    ((at @ torch.tensor(b, dtype=torch.float64)) * torch.tensor(g, dtype=torch.float64)).sum().backward()
    rows = np.repeat(np.arange(m), np.diff(ro))
    want = at.grad.numpy()[rows, ci]
    # lhs = grad (m, n_tokens), rhs = b (k, n_tokens): rhs rows are indexed by the CSR column
    got = oracle.sddmm(g[None], b[None], ri, ro, ci)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)


# ----------------------------------------------------------------------- GEMM
def test_gemm_matches_numpy_and_integer_exactness(oracle):
    rng = np.random.default_rng(12)
    a = rng.standard_normal((17, 24)).astype(np.float32)
    b = rng.standard_normal((24, 9)).astype(np.float32)
    assert np.allclose(oracle.gemm(a, b), a.astype(np.float64) @ b.astype(np.float64), rtol=1e-13)
    assert np.allclose(oracle.gemm(a, np.ascontiguousarray(b.T), trans_b=True), a.astype(np.float64) @ b.astype(np.float64), rtol=1e-13)
    # integer-valued operands (the idiom of tests/test_CUDAGraphConstructor.py:88-93) are exact
    ai = rng.integers(-3, 3, (32, 64)).astype(np.float32)
    bi = rng.integers(-3, 3, (64, 16)).astype(np.float32)
    assert np.array_equal(oracle.gemm(ai, bi), (ai.astype(np.int64) @ bi.astype(np.int64)).astype(np.float64))


def test_csr_softmax(oracle):
    rng = np.random.default_rng(13)
    ro = np.array([0, 3, 3, 7, 8])
    v = rng.standard_normal((2, 8))
    out = oracle.csr_softmax(v, ro)
    for z in range(2):
        for r in range(4):
            seg = v[z, ro[r]:ro[r + 1]]
            if len(seg):
                assert np.allclose(out[z, ro[r]:ro[r + 1]], torch.softmax(torch.from_numpy(seg), 0).numpy(), rtol=1e-12)


# ------------------------------------------------- generators feed valid CSRs
def test_workload_generators_are_well_formed():
    a, b, lhs, rhs = W.config1()
    assert a.nnz == 1024 * 102 and b.shape == (1, 1024, 256) and lhs.shape == (1, 1024, 64)
    for csr in (a, W.config2_matrix(0.98, m=512, k=512), W.config2_matrix(0.70, m=256, k=256, even_rows=True)):
        ro, ci = csr.row_offsets, csr.column_indices
        assert ro[0] == 0 and ro[-1] == csr.nnz and (np.diff(ro) >= 0).all()
        for r in range(0, csr.m, 37):
            seg = ci[ro[r]:ro[r + 1]]
            assert (np.diff(seg) > 0).all() and (seg >= 0).all() and (seg < csr.k).all()
        lens = np.diff(ro)
        assert sorted(csr.row_indices.tolist()) == list(range(csr.m))
        assert (np.diff(lens[csr.row_indices]) <= 0).all()
        assert (csr.values != 0).all() and (csr.values.astype(np.float16) != 0).all()
    c2 = W.config2_matrix(0.90, m=512, k=512)
    assert c2.nnz == round(512 * 512 * 0.10)
    even = W.config2_matrix(0.70, m=256, k=256, even_rows=True)
    assert (np.diff(even.row_offsets) % 2 == 0).all()
    # same seed -> same arrays
    again = W.config2_matrix(0.90, m=512, k=512)
    assert np.array_equal(again.column_indices, c2.column_indices) and np.array_equal(again.values, c2.values)
    m24 = W.two_four_mask(np.random.default_rng(0).standard_normal((8, 16)).astype(np.float32))
    assert (m24.reshape(8, 4, 4).sum(-1) == 2).all()
