"""CSR arrays whose columns are not ascending inside a row, or repeat: the reference's kernels take them as they come
(Sputnik reads values and indices in storage order, sputnik_spmm.cu.inc:229-243, sputnik_sddmm.cu.inc:137), so the
reference-named entry points must too -- at sizes where, for canonical CSR, the library would pick a family that relies
on ascending columns (matrix cores, LDS-staged gather, dense form, the kernels for masks with structure)."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import _lib, workloads as W
from intrasm_engine_amd.pytorch import ops as pyops
from _util import FP16_SUBNORMAL_HALF_STEP, assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops


def _shuffled(csr, seed, duplicate=False):
    """A matrix with the nonzeros of every row in random order.  With ``duplicate`` the first nonzero of every row with
    at least two is stored as two entries of the same column, half of its value each, in the slot of the row's last
    nonzero, which is dropped: row lengths, offsets and swizzle stay what they were, and the expected results are
    computed from the arrays returned here."""
    rng = np.random.default_rng(seed)
    cols, vals = csr.column_indices.copy(), csr.values.astype(np.float32).copy()
    ro = csr.row_offsets
    for r in range(csr.m):
        a, b = int(ro[r]), int(ro[r + 1])
        if duplicate and b - a >= 2:
            # entry a becomes two halves of itself (exact in binary); entry b-1 disappears: its value is dropped
            # from the matrix, which the expected result below is computed from, so nothing needs to add up elsewhere
            cols[b - 1] = cols[a]
            vals[a] = vals[a] * 0.5
            vals[b - 1] = vals[a]
        perm = rng.permutation(b - a)
        cols[a:b], vals[a:b] = cols[a:b][perm], vals[a:b][perm]
    return W.CSR(csr.m, csr.k, vals.astype(csr.values.dtype), csr.row_indices, ro, cols)


def _spmm_want(oracle, c, b_np, dtype):
    v = rounded(c.values, dtype)
    b_r = rounded(b_np, dtype)
    want = oracle.spmm(b_r, c.row_indices, v, c.row_offsets, c.column_indices, c.m)
    scale = oracle.spmm_abs_scale(b_r, c.row_indices, v, c.row_offsets, c.column_indices, c.m)
    return want, scale


@pytest.mark.parametrize("duplicate", [False, True])
def test_fp32_drop_in_and_operator(oracle, dev, duplicate):
    """4096 x 4096 at 70 % sparsity, n = 256: canonical input runs on the fp32 matrix-core kernel (family 5)."""
    canon = W.config2_matrix(0.70)
    rng = np.random.default_rng(5)
    b_np = rng.standard_normal((1, canon.k, 256)).astype(np.float32)
    bt = torch.from_numpy(b_np).to(dev)
    ri, v, ro, ci = to_dev(canon, dev)
    ops.spmm_sputnik_reuse_weight(bt, ri, v, ro, ci, canon.m)
    assert "mfma_f32" in _lib.last_kernels()      # what the shuffled input must not reach

    c = _shuffled(canon, 11, duplicate)
    ri, v, ro, ci = to_dev(c, dev)
    assert pyops.csr_check(ro, ci, c.k) == _lib.CSR_NOT_ASCENDING
    want, scale = _spmm_want(oracle, c, b_np, torch.float32)
    out = ops.spmm_sputnik_reuse_weight(bt, ri, v, ro, ci, c.m)
    assert _lib.last_kernels().startswith("spmm_kernel<"), _lib.last_kernels()
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "operator, shuffled columns")
    raw = torch.full((1, c.m, 256), float("nan"), device=dev)
    rc = _lib.load().iex_CudaSpmm3(c.m, c.k, 256, c.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                                   bt.data_ptr(), raw.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert rc == 0, _lib.last_error()
    assert _lib.last_kernels().startswith("spmm_kernel<"), _lib.last_kernels()
    assert_close(raw.cpu().numpy(), want, scale, 1e-5, "iex_CudaSpmm3, shuffled columns")
    # the atomic drop-in: accumulates into what is there
    acc = torch.ones((1, c.m, 256), device=dev)
    rc = _lib.load().iex_CudaSpmm2(c.m, c.k, 256, c.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                                   bt.data_ptr(), acc.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert rc == 0, _lib.last_error()
    assert_close(acc.cpu().numpy(), want + 1.0, scale + 1.0, 1e-5, "iex_CudaSpmm2, shuffled columns")


@pytest.mark.parametrize("duplicate", [False, True])
def test_fp16_drop_in_and_operator(oracle, dev, duplicate):
    """2048 x 2048 at 80 % sparsity, n = 1024, int16 indices: canonical input goes to the matrix cores (family 4 without
    a workspace, the dense form + GEMM with the operator's workspace)."""
    canon = W.config2_matrix(0.80, m=2048, k=2048, seed=3)
    rng = np.random.default_rng(6)
    b_np = rng.standard_normal((1, canon.k, 1024)).astype(np.float32)
    bt = torch.from_numpy(b_np).to(dev).half()
    ri, v, ro, ci = to_dev(canon, dev, torch.float16, torch.int16)
    ops.spmm_sputnik_reuse_weight_half(bt, ri, v, ro, ci, canon.m)
    assert "gemm" in _lib.last_kernels() or "mfma" in _lib.last_kernels(), _lib.last_kernels()

    c = _shuffled(canon, 12, duplicate)
    ri, v, ro, ci = to_dev(c, dev, torch.float16, torch.int16)
    want, scale = _spmm_want(oracle, c, b_np, torch.float16)
    out = ops.spmm_sputnik_reuse_weight_half(bt, ri, v, ro, ci, c.m)
    assert _lib.last_kernels().startswith("spmm_kernel<"), _lib.last_kernels()
    assert_close(out.float().cpu().numpy(), want, scale, 1e-2, "operator (half), shuffled columns", atol=FP16_SUBNORMAL_HALF_STEP)
    raw = torch.full((1, c.m, 1024), float("nan"), device=dev, dtype=torch.float16)
    rc = _lib.load().iex_CudaSpmm5(c.m, c.k, 1024, c.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                                   bt.data_ptr(), raw.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert rc == 0, _lib.last_error()
    assert _lib.last_kernels().startswith("spmm_kernel<"), _lib.last_kernels()
    assert_close(raw.float().cpu().numpy(), want, scale, 1e-2, "iex_CudaSpmm5, shuffled columns", atol=FP16_SUBNORMAL_HALF_STEP)
    # a caller of the general entry point who says so gets the same; one who does not is on his own (documented)
    out2 = torch.empty_like(raw)
    rc = _lib.load().iex_spmm_ex(_lib.F16, _lib.I16, _lib.SPMM_ANY_COLUMN_ORDER, c.m, c.k, 1024, c.nnz, ri.data_ptr(), v.data_ptr(),
                                 ro.data_ptr(), ci.data_ptr(), bt.data_ptr(), None, out2.data_ptr(),
                                 torch.cuda.current_stream().cuda_stream, 1)
    assert rc == 0 and torch.equal(out2, raw)


def test_canonical_drop_in_still_matches_oracle(oracle, dev):
    """The drop-ins now keep to the row kernel whatever the input: same result as the operator's choice, within tolerance."""
    c = W.config2_matrix(0.70)
    rng = np.random.default_rng(7)
    b_np = rng.standard_normal((1, c.k, 128)).astype(np.float32)
    bt = torch.from_numpy(b_np).to(dev)
    ri, v, ro, ci = to_dev(c, dev)
    want, scale = _spmm_want(oracle, c, b_np, torch.float32)
    raw = torch.empty((1, c.m, 128), device=dev)
    rc = _lib.load().iex_CudaSpmm3(c.m, c.k, 128, c.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                                   bt.data_ptr(), raw.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert rc == 0, _lib.last_error()
    assert_close(raw.cpu().numpy(), want, scale, 1e-5, "iex_CudaSpmm3, canonical")


@pytest.mark.parametrize("duplicate", [False, True])
def test_per_entry_sddmm_and_spmm_for_attention_masks(oracle, dev, duplicate):
    """8 heads of 2048 x 2048 with a band mask, 7 % dense: canonical input takes the kernels for masks with structure
    (SDDMM variant 3, SpMM family 10), whose tables assume ascending, distinct columns."""
    heads, t, d = 8, 2048, 64
    canon, q, kk, _ = W.config3(tokens=t, head_dim=d, heads=heads)
    rng = np.random.default_rng(8)
    qt, kt = torch.from_numpy(q).to(dev).half(), torch.from_numpy(kk).to(dev).half()
    ri, _, ro, ci = to_dev(canon, dev)
    ops.sddmm_sputnik_half(qt, kt, ri, ro, ci)
    assert "sddmm_mfma_kernel" in _lib.last_kernels(), _lib.last_kernels()

    c = _shuffled(canon, 13, duplicate)
    ri, _, ro, ci = to_dev(c, dev)
    out = ops.sddmm_sputnik_half(qt, kt, ri, ro, ci)
    assert "sddmm_mfma_kernel" not in _lib.last_kernels(), _lib.last_kernels()
    qr, kr = rounded(q, torch.float16), rounded(kk, torch.float16)
    for z in (0, heads - 1):
        want = oracle.sddmm(qr[z:z + 1], kr[z:z + 1], c.row_indices, c.row_offsets, c.column_indices)
        scale = oracle.sddmm_abs_scale(qr[z:z + 1], kr[z:z + 1], c.row_indices, c.row_offsets, c.column_indices)
        assert_close(out[z].float().cpu().numpy(), want, scale, 1e-2, f"sddmm head {z}, shuffled columns", atol=FP16_SUBNORMAL_HALF_STEP)
    # second product: probabilities (any values) times V
    vals = torch.from_numpy(rng.standard_normal((heads, c.nnz)).astype(np.float32)).to(dev).half()
    vv = rng.standard_normal((heads, t, d)).astype(np.float32)
    vt = torch.from_numpy(vv).to(dev).half()
    got = ops.spmm_sputnik_batched_values(vt, ri, vals, ro, ci, t)
    assert "spmm_blocks_kernel" not in _lib.last_kernels(), _lib.last_kernels()
    for z in (0, heads - 1):
        vz = vals[z].float().cpu().numpy()
        want = oracle.spmm(rounded(vv[z:z + 1], torch.float16), c.row_indices, vz, c.row_offsets, c.column_indices, t)
        scale = oracle.spmm_abs_scale(rounded(vv[z:z + 1], torch.float16), c.row_indices, vz, c.row_offsets, c.column_indices, t)
        assert_close(got[z:z + 1].float().cpu().numpy(), want, scale, 1e-2, f"spmm head {z}, shuffled columns", atol=FP16_SUBNORMAL_HALF_STEP)


def test_offsets_or_columns_that_point_outside_are_refused(dev):
    m, k, n = 8, 16, 64
    ri = torch.arange(m, dtype=torch.int32, device=dev)
    ro = torch.arange(0, 2 * m + 1, 2, dtype=torch.int32, device=dev)
    b = torch.randn(1, k, n, device=dev)
    v = torch.randn(2 * m, device=dev)
    ci = torch.arange(2 * m, dtype=torch.int32, device=dev) % k
    ci_bad = ci.clone()
    ci_bad[3] = k
    with pytest.raises(RuntimeError, match="column index"):
        ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci_bad, m)
    ro_bad = ro.clone()
    ro_bad[-1] = 2 * m + 5
    with pytest.raises(RuntimeError, match="row_offsets"):
        ops.spmm_sputnik_reuse_weight(b, ri, v, ro_bad, ci, m)


def test_an_unseen_pattern_under_capture_keeps_to_the_any_order_kernels(oracle, dev):
    """Nothing can be looked at while a stream is being captured (the check ends in a synchronising read): a pattern that
    no operator has seen before is then taken for what the reference would accept -- columns in any order."""
    from intrasm_engine_amd import interleaving as IL
    canon = W.config2_matrix(0.70)
    c = _shuffled(canon, 14)
    rng = np.random.default_rng(9)
    b_np = rng.standard_normal((1, c.k, 256)).astype(np.float32)
    bt = torch.from_numpy(b_np).to(dev)
    ri, v, ro, ci = (torch.from_numpy(x).to(dev) for x in (c.row_indices, c.values, c.row_offsets, c.column_indices))   # (nobody has looked at it)
    constructor, keep = IL.capture_serialized([lambda: ops.spmm_sputnik_reuse_weight(bt, ri, v, ro, ci, c.m)])
    constructor.instantiate_graph_exec()
    constructor.execute_graph()
    constructor.synchronize()
    constructor.destroy_graph_exec()
    want, scale = _spmm_want(oracle, c, b_np, torch.float32)
    assert_close(keep[0].cpu().numpy(), want, scale, 1e-5, "captured, unseen shuffled pattern")


def test_a_pattern_made_under_capture_can_be_vouched_for(oracle, dev):
    """A mask that changes from step to step is made on the device inside the captured region; nobody can look at it
    there.  A caller whose construction guarantees canonical CSR says so with mark_canonical(..., measure=False), which
    launches nothing and reads nothing back: the call then takes the kernel families for canonical CSR (here: the fp32
    matrix cores, which the any-order path never takes)."""
    from intrasm_engine_amd import _lib, interleaving as IL
    from intrasm_engine_amd.pytorch import ops as pyops
    c = W.config2_matrix(0.70)
    rng = np.random.default_rng(10)
    b_np = rng.standard_normal((1, c.k, 256)).astype(np.float32)
    bt = torch.from_numpy(b_np).to(dev)
    ri, v, ro, src = (torch.from_numpy(x).to(dev) for x in (c.row_indices, c.values, c.row_offsets, c.column_indices))
    trail = []

    def step():
        ci = src.clone()                                    # (stands for: the mask of this step, computed on the device)
        pyops.mark_canonical(ro, ci, c.k, measure=False)
        out = ops.spmm_sputnik_reuse_weight(bt, ri, v, ro, ci, c.m)
        trail.append(_lib.last_kernels())
        return out
    constructor, keep = IL.capture_serialized([step])
    constructor.instantiate_graph_exec()
    constructor.execute_graph()
    constructor.synchronize()
    constructor.destroy_graph_exec()
    assert "spmm_mfma_f32_kernel" in trail[0], trail
    want, scale = _spmm_want(oracle, c, b_np, torch.float32)
    assert_close(keep[0].cpu().numpy(), want, scale, 1e-5, "captured, pattern vouched for")


def test_sparse_attention_under_inference_mode(dev):
    """Tensors made under torch.inference_mode() keep no version counter; the plan's key must not ask for one."""
    from intrasm_engine_amd.pytorch.sparse_attention import sparse_attention
    heads, t, d = 8, 2048, 64
    mask = W.config3(tokens=t, heads=1)[0]
    with torch.inference_mode():
        ri, _, ro, ci = to_dev(mask, dev)
        q, k, v = (torch.randn(heads, t, d, device=dev).half() for _ in range(3))
        out = sparse_attention(q, k, v, ri, ro, ci)
        again = sparse_attention(q, k, v, ri, ro, ci)
    assert out.shape == (heads, t, d) and torch.isfinite(out.float()).all() and torch.equal(out, again)
