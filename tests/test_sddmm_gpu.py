"""GPU parity of the CSR SDDMM operators and the CSR softmax against the CPU oracle."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from _util import RTOL, assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops


def _check(oracle, csr, lhs_np, rhs_np, dev, dtype, sum_over_batch, what):
    ri, _, ro, ci = to_dev(csr, dev)
    lhs = torch.from_numpy(lhs_np).to(dev).to(dtype)
    rhs = torch.from_numpy(rhs_np).to(dev).to(dtype)
    if sum_over_batch:
        out = ops.sddmm_sputnik_atomic_upd_weight(lhs, rhs, ri, ro, ci)
        assert out.shape == (csr.nnz,)
    else:
        out = ops.sddmm_sputnik_half(lhs, rhs, ri, ro, ci)
        assert out.shape == (lhs.shape[0], csr.nnz)
    assert out.dtype == dtype
    l_r, r_r = rounded(lhs_np, dtype), rounded(rhs_np, dtype)
    want = oracle.sddmm(l_r, r_r, csr.row_indices, csr.row_offsets, csr.column_indices, sum_over_batch=sum_over_batch)
    scale = oracle.sddmm_abs_scale(l_r, r_r, csr.row_indices, csr.row_offsets, csr.column_indices,
                                   sum_over_batch=sum_over_batch)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], what)
    return out


def test_config1_fp32(oracle, dev):
    a, _, lhs, rhs = W.config1()
    _check(oracle, a, lhs, rhs, dev, torch.float32, True, "C1 fp32 SDDMM")


def test_config3_fp16_per_head_then_spmm(oracle, dev):
    """Sparse attention of config 3: per-head SDDMM(Q, K) on the banded mask, then SpMM with
    the per-head values against V.  4 of the 16 heads are checked against the oracle (the
    kernel treats heads identically; all 16 run in test_full_size_config3_properties)."""
    pattern, q, k, v = W.config3(heads=4)
    out = _check(oracle, pattern, q, k, dev, torch.float16, False, "C3 fp16 SDDMM")
    ri, _, ro, ci = to_dev(pattern, dev)
    vt = torch.from_numpy(v).to(dev).half()
    ctx = ops.spmm_sputnik_batched_values(vt, ri, out, ro, ci, pattern.m)
    vals = out.float().cpu().numpy()
    want = oracle.spmm(rounded(v, torch.float16), pattern.row_indices, vals, pattern.row_offsets,
                       pattern.column_indices, pattern.m)
    scale = oracle.spmm_abs_scale(rounded(v, torch.float16), pattern.row_indices, vals, pattern.row_offsets,
                                  pattern.column_indices, pattern.m)
    assert_close(ctx.float().cpu().numpy(), want, scale, 1e-2, "C3 SpMM against V")


def test_full_size_config3_properties(dev):
    """All 16 heads: (a) every head of the batched launch equals the same head launched alone
    (bit-exact, kernel by kernel: which one the library picks by itself depends on the amount of work),
    (b) the diagonal entries equal the row-wise dot products <q_i, k_i>."""
    from intrasm_engine_amd.pytorch import ops as pyops
    pattern, q, k, _ = W.config3()
    ri, _, ro, ci = to_dev(pattern, dev)
    qt, kt = torch.from_numpy(q).to(dev).half(), torch.from_numpy(k).to(dev).half()
    for variant in (1, 3):
        with pyops.kernel_params(sddmm={"force_variant": variant}):
            out = ops.sddmm_sputnik_half(qt, kt, ri, ro, ci)
            for h in (0, 7, 15):
                assert torch.equal(ops.sddmm_sputnik_half(qt[h:h + 1].contiguous(), kt[h:h + 1].contiguous(), ri, ro, ci)[0], out[h]), (variant, h)
    out = ops.sddmm_sputnik_half(qt, kt, ri, ro, ci)
    rows = torch.repeat_interleave(torch.arange(pattern.m, device=dev), torch.diff(ro.long()))
    diag = (rows == ci.long()).nonzero().squeeze(1)
    assert diag.numel() == pattern.m
    want = (qt.float() * kt.float()).sum(-1)
    got = out[:, diag].float()
    assert torch.allclose(got, want, rtol=1e-2, atol=1e-2 * 1e-2 * 64)


@pytest.mark.parametrize("k", [1, 3, 8, 20, 32, 64, 72, 128, 200, 1024])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_ragged_shapes(oracle, dev, k, dtype):
    rng = np.random.default_rng(k)
    m, n = 131, 97
    lens = rng.integers(0, 30, m)
    lens[[0, 9, 130]] = 0
    lens[5] = n
    ro, ci = W.csr_from_row_lengths(rng, m, n, lens)
    csr = W.CSR(m, n, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    lhs = rng.standard_normal((2, m, k)).astype(np.float32)
    rhs = rng.standard_normal((2, n, k)).astype(np.float32)
    _check(oracle, csr, lhs, rhs, dev, dtype, False, f"ragged per-batch k={k} {dtype}")
    if dtype == torch.float32:
        _check(oracle, csr, lhs, rhs, dev, dtype, True, f"ragged summed k={k}")


def test_long_rows_split_over_waves(oracle, dev):
    rng = np.random.default_rng(77)
    a = W.config2_matrix(0.70, m=512, k=1024)     # mean row length ~307 -> 4 wavefronts per row
    lhs = rng.standard_normal((1, 512, 64)).astype(np.float32)
    rhs = rng.standard_normal((1, 1024, 64)).astype(np.float32)
    _check(oracle, a, lhs, rhs, dev, torch.float32, True, "long rows fp32")
    _check(oracle, a, lhs, rhs, dev, torch.float16, False, "long rows fp16")


def test_integer_inputs_are_exact_and_full_mask_is_gemm(dev):
    rng = np.random.default_rng(3)
    m, n, k = 64, 48, 64
    lhs = torch.from_numpy(rng.integers(-3, 4, (1, m, k)).astype(np.float32)).to(dev)
    rhs = torch.from_numpy(rng.integers(-3, 4, (1, n, k)).astype(np.float32)).to(dev)
    ro = torch.arange(0, m * n + 1, n, dtype=torch.int32, device=dev)
    ci = torch.arange(n, dtype=torch.int32, device=dev).repeat(m)
    ri = torch.arange(m, dtype=torch.int32, device=dev)
    want = (lhs[0].double() @ rhs[0].double().T).reshape(-1)
    assert torch.equal(ops.sddmm_sputnik_atomic_upd_weight(lhs, rhs, ri, ro, ci).double(), want)
    assert torch.equal(ops.sddmm_sputnik_half(lhs.half(), rhs.half(), ri, ro, ci)[0].double(), want)


def test_reference_launcher_name_through_c_abi(oracle, dev):
    from intrasm_engine_amd import _lib
    a, _, lhs_np, rhs_np = W.config1()
    ri, _, ro, ci = to_dev(a, dev)
    lhs, rhs = torch.from_numpy(lhs_np).to(dev), torch.from_numpy(rhs_np).to(dev)
    out = torch.full((a.nnz,), float("nan"), device=dev)   # written, not accumulated
    rc = _lib.load().iex_CudaSddmm2(a.m, 64, a.k, a.nnz, ri.data_ptr(), ro.data_ptr(), ci.data_ptr(), lhs.data_ptr(),
                                    rhs.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert rc == 0, _lib.last_error()
    want = oracle.sddmm(lhs_np, rhs_np, a.row_indices, a.row_offsets, a.column_indices)
    scale = oracle.sddmm_abs_scale(lhs_np, rhs_np, a.row_indices, a.row_offsets, a.column_indices)
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "iex_CudaSddmm2")


def test_empty_pattern(dev):
    m, n, k = 9, 7, 16
    z = torch.zeros(m + 1, dtype=torch.int32, device=dev)
    out = ops.sddmm_sputnik_atomic_upd_weight(torch.randn(1, m, k, device=dev), torch.randn(1, n, k, device=dev),
                                              torch.arange(m, dtype=torch.int32, device=dev), z,
                                              torch.zeros(0, dtype=torch.int32, device=dev))
    assert out.shape == (0,)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_csr_softmax(oracle, dev, dtype):
    pattern, q, k, _ = W.config3(tokens=512, heads=2, band=64, extra=8)
    rng = np.random.default_rng(4)
    vals = rng.standard_normal((2, pattern.nnz)).astype(np.float32) * 3
    ri, _, ro, _ = to_dev(pattern, dev)
    v = torch.from_numpy(vals).to(dev).to(dtype)
    ops.csr_softmax_(v, ri, ro, 0.125)
    want = oracle.csr_softmax(rounded(vals, dtype).astype(np.float64) * 0.125, pattern.row_offsets)
    tol = 2e-6 if dtype == torch.float32 else 2e-3
    assert np.abs(v.float().cpu().numpy() - want).max() <= tol
    sums = np.add.reduceat(v.float().cpu().numpy(), pattern.row_offsets[:-1], axis=1)
    assert np.allclose(sums, 1.0, atol=1e-2 if dtype == torch.float16 else 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_csr_softmax_long_short_and_empty_rows(oracle, dev, dtype):
    """Rows of 0, 1, 64, 65, 512 (the longest that stays in registers), 513 and 2000 entries."""
    lens = np.array([0, 1, 64, 65, 512, 513, 2000, 0, 7, 300])
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    rng = np.random.default_rng(11)
    vals = rng.standard_normal((3, int(ro[-1]))).astype(np.float32) * 4
    ri = torch.from_numpy(W.swizzle_from_offsets(ro)).to(dev)
    v = torch.from_numpy(vals).to(dev).to(dtype)
    ops.csr_softmax_(v, ri, torch.from_numpy(ro).to(dev), 0.5)
    want = oracle.csr_softmax(rounded(vals, dtype).astype(np.float64) * 0.5, ro)
    got = v.float().cpu().numpy()
    assert np.abs(got - want).max() <= (2e-6 if dtype == torch.float32 else 8e-3)
    for r in np.nonzero(lens)[0]:
        assert np.allclose(got[:, ro[r]:ro[r + 1]].sum(axis=1), 1.0, atol=1e-5 if dtype == torch.float32 else 2e-2), r


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tail", [1, 2, 129, 385])
def test_csr_softmax_pairs_of_16_bit_entries(oracle, dev, dtype, tail):
    """16-bit entries are read and written two at a time: row lengths on both sides of every slot boundary of that
    path (128, 384, 512 entries), rows that start at odd positions, and a last row of `tail` entries whose final
    pair ends exactly at (or one entry before) the end of the tensor; one and three batch entries."""
    lens = np.array([2, 3, 127, 128, 129, 0, 383, 384, 385, 511, 512, 5, tail])
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    rng = np.random.default_rng(tail)
    ri = torch.from_numpy(W.swizzle_from_offsets(ro)).to(dev)
    for batch in (1, 3):
        vals = rng.standard_normal((batch, int(ro[-1]))).astype(np.float32) * 4
        v = torch.from_numpy(vals).to(dev).to(dtype)
        ops.csr_softmax_(v, ri, torch.from_numpy(ro).to(dev), 0.5)
        want = oracle.csr_softmax(rounded(vals, dtype).astype(np.float64) * 0.5, ro)
        got = v.float().cpu().numpy()
        assert np.abs(got - want).max() <= (2e-3 if dtype == torch.float16 else 8e-3), batch


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_csr_softmax_four_rows_of_16_bit_entries_per_wavefront(oracle, dev, dtype):
    """16-bit tensors whose rows average 512 entries or fewer run four rows per wavefront, 16 lanes per row, as many pairs
    per lane as the longest of the four needs: row lengths on both sides of every pair count (32 p - 1, 32 p, 32 p + 1 for
    p = 1 .. 16), in the order of the swizzle and in a shuffled order (rows of very different length in one wavefront, a
    long row of 900 among them: that wavefront takes its rows one by one), a number of rows that is no multiple of 16, a
    negative scale and an average above 512 (both: the kernel with a wavefront per row)."""
    lens = np.array([x for p in range(1, 17) for x in (32 * p - 1, 32 * p, 32 * p + 1)] + [0, 900, 1, 0, 6])
    ro = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    rng = np.random.default_rng(5)
    vals = rng.standard_normal((2, int(ro[-1]))).astype(np.float32) * 4
    tol = 2e-3 if dtype == torch.float16 else 8e-3
    for order in (W.swizzle_from_offsets(ro), rng.permutation(len(lens)).astype(np.int32)):
        for scale in (0.5, -0.5):
            v = torch.from_numpy(vals).to(dev).to(dtype)
            ops.csr_softmax_(v, torch.from_numpy(order).to(dev), torch.from_numpy(ro).to(dev), scale)
            want = oracle.csr_softmax(rounded(vals, dtype).astype(np.float64) * scale, ro)
            assert np.abs(v.float().cpu().numpy() - want).max() <= tol, scale
    long_lens = np.array([600, 700, 513, 520])
    ro2 = np.concatenate([[0], np.cumsum(long_lens)]).astype(np.int32)
    vals2 = rng.standard_normal((1, int(ro2[-1]))).astype(np.float32)
    v2 = torch.from_numpy(vals2).to(dev).to(dtype)
    ops.csr_softmax_(v2, torch.arange(4, dtype=torch.int32, device=dev), torch.from_numpy(ro2).to(dev), 1.0)
    assert np.abs(v2.float().cpu().numpy() - oracle.csr_softmax(rounded(vals2, dtype).astype(np.float64), ro2)).max() <= tol


def test_operator_argument_checks(dev):
    a, _, lhs_np, rhs_np = W.config1()
    ri, _, ro, ci = to_dev(a, dev)
    lhs, rhs = torch.from_numpy(lhs_np).to(dev), torch.from_numpy(rhs_np).to(dev)
    with pytest.raises(RuntimeError, match="a must be a CUDA tensor"):
        ops.sddmm_sputnik_atomic_upd_weight(lhs.cpu(), rhs, ri, ro, ci)
    with pytest.raises(RuntimeError):
        ops.sddmm_sputnik_atomic_upd_weight(lhs, rhs[:, :, :32].contiguous(), ri, ro, ci)   # k mismatch
    with pytest.raises(RuntimeError, match="b must be a contiguous tensor"):
        ops.sddmm_sputnik_atomic_upd_weight(lhs, rhs.transpose(1, 2).contiguous().transpose(1, 2), ri, ro, ci)


def _dense_product_case(rng, m, k, n, sparsity, batch, dtype, dev):
    lens = rng.binomial(n, 1 - sparsity, m)
    lens[0] = 0
    lens[min(3, m - 1)] = n
    ro, ci = W.csr_from_row_lengths(rng, m, n, lens)
    csr = W.CSR(m, n, np.zeros(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    lhs_np = (rng.standard_normal((batch, m, k)) * 0.25).astype(np.float32)
    rhs_np = rng.standard_normal((batch, n, k)).astype(np.float32)
    t = lambda x: torch.from_numpy(x).to(dev).to(dtype)
    return csr, lhs_np, rhs_np, t(lhs_np), t(rhs_np), to_dev(csr, dev)


@pytest.mark.parametrize("dtype,m,k,n,batch", [(torch.float16, 203, 160, 256, 2), (torch.bfloat16, 75, 304, 264, 1),
                                               (torch.float16, 130, 8, 8, 3), (torch.float16, 33, 1032, 520, 1)])
def test_dense_product_path(oracle, dev, dtype, m, k, n, batch):
    """The whole product lhs * rhs^T by the dense GEMM into a workspace, then the nonzeros' entries
    picked: on request on small ragged shapes (an empty row, a full row, a batch), against the oracle."""
    from intrasm_engine_amd.pytorch import ops as pyops
    csr, lhs_np, rhs_np, lhs, rhs, (ri, _, ro, ci) = _dense_product_case(np.random.default_rng(m + k), m, k, n, 0.8, batch, dtype, dev)
    out = pyops._sddmm(lhs, rhs, ri, ro, ci, sum_over_batch=False, dtypes=(dtype,), force_variant=7)
    assert out.shape == (batch, csr.nnz) and out.dtype == dtype
    l_r, r_r = rounded(lhs_np, dtype), rounded(rhs_np, dtype)
    want = oracle.sddmm(l_r, r_r, csr.row_indices, csr.row_offsets, csr.column_indices, sum_over_batch=False)
    scale = oracle.sddmm_abs_scale(l_r, r_r, csr.row_indices, csr.row_offsets, csr.column_indices, sum_over_batch=False)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"dense product {dtype} {m}x{k}x{n}")


def test_dense_product_path_is_chosen_with_a_workspace_and_only_then(oracle, dev):
    """1024 x 1024 mask at 70 % sparsity, k = 4096, fp16: the time model prefers the dense product.
    The operator asks for the workspace size, allocates it and gets that result; without a workspace,
    with a short one, and for calls the path does not serve (fp32, batch-summed output of a batch,
    accumulate, a short k with a sparse mask) the gather kernel runs."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    lib = _lib.load()
    m = n = 1024
    k = 4096
    dtype = torch.float16
    csr, lhs_np, rhs_np, lhs, rhs, (ri, _, ro, ci) = _dense_product_case(np.random.default_rng(8), m, k, n, 0.7, 1, dtype, dev)
    nnz = csr.nnz
    need = lib.iex_sddmm_workspace_bytes(_lib.F16, 0, m, k, n, nnz, 1)
    assert need == m * n * 2
    assert lib.iex_sddmm_workspace_bytes(_lib.F32, 0, m, k, n, nnz, 1) == 0
    assert lib.iex_sddmm_workspace_bytes(_lib.F16, _lib.SDDMM_SUM_OVER_BATCH, m, k, n, nnz, 2) == 0
    assert lib.iex_sddmm_workspace_bytes(_lib.F16, _lib.SDDMM_SUM_OVER_BATCH, m, k, n, nnz, 1) == need
    assert lib.iex_sddmm_workspace_bytes(_lib.F16, _lib.SDDMM_ACCUMULATE, m, k, n, nnz, 1) == 0
    # config 3: not the dense product; the tables of the kernel that samples score tiles inside the workgroup
    assert lib.iex_sddmm_workspace_bytes(_lib.F16, 0, 4096, 64, 4096, 1150000, 16) == ((6 * 32 + 1) * 4096 + 64 + 2 * 1150000 + 4096 + 32 * (32 + 2) // 2) * 4   # tables + lists
    assert lib.iex_sddmm_workspace_bytes(_lib.F16, 0, 4096, 64, 4096, 1150000 // 4, 16) == 0   # a mask this thin: the gather kernel
    assert lib.iex_sddmm_workspace_bytes(_lib.F16, 7 << 16, 4096, 64, 4096, 1150000, 16) == 4096 * 4096 * 2  # on request
    kw = dict(sum_over_batch=False, dtypes=(dtype,))
    auto = pyops._sddmm(lhs, rhs, ri, ro, ci, **kw)
    assert torch.equal(auto, pyops._sddmm(lhs, rhs, ri, ro, ci, force_variant=7, **kw))
    l_r, r_r = rounded(lhs_np, dtype), rounded(rhs_np, dtype)
    want = oracle.sddmm(l_r, r_r, csr.row_indices, csr.row_offsets, csr.column_indices, sum_over_batch=False)
    scale = oracle.sddmm_abs_scale(l_r, r_r, csr.row_indices, csr.row_offsets, csr.column_indices, sum_over_batch=False)
    assert_close(auto.float().cpu().numpy(), want, scale, RTOL[dtype], "dense product, chosen")
    gather = pyops._sddmm(lhs, rhs, ri, ro, ci, force_variant=1, **kw)
    assert torch.equal(pyops._sddmm(lhs, rhs, ri, ro, ci, no_workspace=True, **kw), gather)
    assert not torch.equal(auto, gather)    # (another order of summation)
    short = torch.empty(need - 16, dtype=torch.uint8, device=dev)
    out = torch.empty_like(gather)
    args = (_lib.F16, 0, m, k, n, nnz, ri.data_ptr(), ro.data_ptr(), ci.data_ptr(), lhs.data_ptr(), rhs.data_ptr(),
            out.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert lib.iex_sddmm_ws(*args, short.data_ptr(), need - 16) == 0, _lib.last_error()
    assert torch.equal(out, gather)
    forced = (_lib.F16, 7 << 16) + args[2:]
    assert lib.iex_sddmm_ex(*forced) != 0 and "workspace" in _lib.last_error()
    torch.cuda.synchronize()
