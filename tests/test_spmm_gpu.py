"""GPU parity of the CSR SpMM operators against the CPU oracle (through torch.ops.iex_ops
and, for the launcher drop-ins, straight through the C ABI)."""
import ctypes

import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from _util import FP16_SUBNORMAL_HALF_STEP, RTOL, assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops


def _check(oracle, csr, b_np, dev, dtype=torch.float32, idtype=torch.int32, op=None, what=""):
    ri, v, ro, ci = to_dev(csr, dev, dtype, idtype)
    b = torch.from_numpy(b_np).to(dev).to(dtype)
    if op is None:
        op = ops.spmm_sputnik_reuse_weight if dtype == torch.float32 else ops.spmm_sputnik_reuse_weight_half
    out = op(b, ri, v, ro, ci, csr.m)
    torch.cuda.synchronize()
    assert out.shape == (b.shape[0], csr.m, b.shape[2]) and out.dtype == dtype
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, csr.m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, csr.m)
    return assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], what)


def test_config1_fp32(oracle, dev):
    a, b, _, _ = W.config1()
    _check(oracle, a, b, dev, what="C1 fp32 SpMM")


@pytest.mark.parametrize("sparsity", W.C2_SPARSITIES)
def test_config2_sweep_fp32(oracle, dev, sparsity):
    a = W.config2_matrix(sparsity)
    for n in W.C2_NS:
        _check(oracle, a, W.config2_dense(n), dev, what=f"C2 fp32 s={sparsity} n={n}")


@pytest.mark.parametrize("sparsity", W.C2_SPARSITIES)
def test_config2_sweep_fp16(oracle, dev, sparsity):
    a = W.config2_matrix(sparsity, even_rows=True)
    for n, idt in ((64, torch.int16), (128, torch.int32), (256, torch.int16)):
        _check(oracle, a, W.config2_dense(n), dev, torch.float16, idt, what=f"C2 fp16 s={sparsity} n={n} {idt}")


def test_bf16(oracle, dev):
    a = W.config2_matrix(0.95, m=512, k=512)
    _check(oracle, a, W.config2_dense(128, k=512), dev, torch.bfloat16, what="bf16 SpMM")


@pytest.mark.parametrize("n", [1, 3, 33, 64, 70, 130, 200, 512])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_ragged_shapes(oracle, dev, n, dtype):
    """m not a multiple of the rows per workgroup, empty rows, every vector width and the
    scalar tail path."""
    rng = np.random.default_rng(n)
    m, k = 203, 157
    lens = rng.integers(0, 40, m)
    lens[[0, 5, 202]] = 0
    lens[7] = k
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b = rng.standard_normal((2, k, n)).astype(np.float32)
    _check(oracle, csr, b, dev, dtype, what=f"ragged n={n} {dtype}")


@pytest.mark.parametrize("wpr", [1, 4, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_every_row_split_variant(oracle, dev, wpr, dtype):
    """The three work decompositions (1, 4, 8 wavefronts per row) on one skewed matrix."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(99)
    m, k, n = 301, 2048, 192
    lens = np.clip(rng.geometric(1 / 150.0, m), 0, k)
    lens[3] = k
    lens[4] = 0
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((1, k, n)).astype(np.float32)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    b = torch.from_numpy(b_np).to(dev).to(dtype)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=False,
                      dtypes=(dtype,), allow_i16=False, force_wpr=wpr)
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"wpr={wpr}")


def test_all_empty_matrix_and_empty_shapes(dev):
    m, k, n = 17, 9, 64
    z32 = lambda *s: torch.zeros(*s, dtype=torch.int32, device=dev)
    b = torch.randn(1, k, n, device=dev)
    out = ops.spmm_sputnik_reuse_weight(b, torch.arange(m, dtype=torch.int32, device=dev),
                                        torch.zeros(0, device=dev), z32(m + 1), z32(0), m)
    assert out.shape == (1, m, n) and (out == 0).all()
    out = ops.spmm_sputnik_reuse_weight(torch.zeros(1, k, 0, device=dev), torch.arange(m, dtype=torch.int32, device=dev),
                                        torch.zeros(0, device=dev), z32(m + 1), z32(0), m)
    assert out.shape == (1, m, 0)


def test_integer_inputs_are_exact(dev):
    """Small-integer operands make every partial sum exactly representable, so the device
    result must EQUAL the integer product (the exactness idiom of the reference's
    tests/test_CUDAGraphConstructor.py:88-93), in fp32 and in fp16."""
    rng = np.random.default_rng(1)
    a = W.config2_matrix(0.95, m=1024, k=1024)
    a.values = rng.integers(1, 4, a.nnz).astype(np.float32) * rng.choice([-1, 1], a.nnz).astype(np.float32)
    b_np = rng.integers(-3, 4, (1, 1024, 128)).astype(np.float32)
    dense = torch.zeros(1024, 1024, dtype=torch.float64)
    rows = np.repeat(np.arange(1024), np.diff(a.row_offsets))
    dense[rows, a.column_indices.astype(np.int64)] = torch.from_numpy(a.values).double()
    want = (dense @ torch.from_numpy(b_np[0]).double()).numpy()
    for dtype in (torch.float32, torch.float16):
        ri, v, ro, ci = to_dev(a, dev, dtype)
        op = ops.spmm_sputnik_reuse_weight if dtype == torch.float32 else ops.spmm_sputnik_reuse_weight_half
        out = op(torch.from_numpy(b_np).to(dev).to(dtype), ri, v, ro, ci, 1024)
        assert np.array_equal(out[0].double().cpu().numpy(), want), dtype


def test_swizzle_is_scheduling_only(dev):
    a = W.config2_matrix(0.90, m=1024, k=1024)
    b = torch.from_numpy(W.config2_dense(64, k=1024)).to(dev)
    ri, v, ro, ci = to_dev(a, dev)
    base = ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, a.m)
    perm = torch.randperm(a.m, device=dev, generator=torch.Generator(dev).manual_seed(0)).to(torch.int32)
    assert torch.equal(ops.spmm_sputnik_reuse_weight(b, perm, v, ro, ci, a.m), base)
    ident = torch.arange(a.m, device=dev, dtype=torch.int32)
    assert torch.equal(ops.spmm_sputnik_reuse_weight(b, ident, v, ro, ci, a.m), base)


def test_batch_and_per_batch_values(oracle, dev):
    rng = np.random.default_rng(5)
    a = W.config2_matrix(0.875, m=256, k=512)     # nnz = 16384, a multiple of 4
    assert a.nnz % 4 == 0
    batch = 3
    b_np = rng.standard_normal((batch, 512, 96)).astype(np.float32)
    vb = rng.standard_normal((batch, a.nnz)).astype(np.float32)
    ri, v, ro, ci = to_dev(a, dev)
    b = torch.from_numpy(b_np).to(dev)
    # shared values over a batch
    out = ops.spmm_sputnik_reuse_weight(b, ri, v, ro, ci, a.m)
    want = oracle.spmm(b_np, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m)
    scale = oracle.spmm_abs_scale(b_np, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m)
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "batched reuse-weight")
    # per-batch values: the "atomic" operator = zero, then accumulate
    out = ops.spmm_sputnik_atomic(b, ri, torch.from_numpy(vb).to(dev), ro, ci, a.m)
    want = oracle.spmm(b_np, a.row_indices, vb, a.row_offsets, a.column_indices, a.m)
    scale = oracle.spmm_abs_scale(b_np, a.row_indices, vb, a.row_offsets, a.column_indices, a.m)
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "spmm_sputnik_atomic")
    # written (not accumulated) per-batch variant in fp16
    out = ops.spmm_sputnik_batched_values(b.half(), ri, torch.from_numpy(vb).to(dev).half(), ro, ci, a.m)
    want = oracle.spmm(rounded(b_np, torch.float16), a.row_indices, rounded(vb, torch.float16), a.row_offsets,
                       a.column_indices, a.m)
    scale = oracle.spmm_abs_scale(rounded(b_np, torch.float16), a.row_indices, rounded(vb, torch.float16),
                                  a.row_offsets, a.column_indices, a.m)
    assert_close(out.float().cpu().numpy(), want, scale, 1e-2, "batched values fp16")


def test_accumulate_bias_relu_through_c_abi(oracle, dev):
    """iex_spmm_ex with the accumulate flag adds to a pre-filled output; bias + ReLU epilogue."""
    from intrasm_engine_amd import _lib
    rng = np.random.default_rng(6)
    a = W.config2_matrix(0.90, m=128, k=256)
    b_np = rng.standard_normal((1, 256, 64)).astype(np.float32)
    init = rng.standard_normal((1, 128, 64)).astype(np.float32)
    bias = rng.standard_normal(128).astype(np.float32)
    ri, v, ro, ci = to_dev(a, dev)
    b, out, bias_t = torch.from_numpy(b_np).to(dev), torch.from_numpy(init).to(dev), torch.from_numpy(bias).to(dev)
    s = torch.cuda.current_stream().cuda_stream
    rc = _lib.load().iex_spmm_ex(_lib.F32, _lib.I32, _lib.SPMM_ACCUMULATE, a.m, a.k, 64, a.nnz, ri.data_ptr(),
                                 v.data_ptr(), ro.data_ptr(), ci.data_ptr(), b.data_ptr(), None, out.data_ptr(), s, 1)
    assert rc == 0, _lib.last_error()
    want = oracle.spmm(b_np, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m, out_init=init)
    scale = oracle.spmm_abs_scale(b_np, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m) + np.abs(init)
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "accumulate")
    out2 = torch.empty_like(out)
    rc = _lib.load().iex_spmm_ex(_lib.F32, _lib.I32, _lib.SPMM_RELU, a.m, a.k, 64, a.nnz, ri.data_ptr(), v.data_ptr(),
                                 ro.data_ptr(), ci.data_ptr(), b.data_ptr(), bias_t.data_ptr(), out2.data_ptr(), s, 1)
    assert rc == 0, _lib.last_error()
    want = oracle.spmm(b_np, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m, bias=bias, relu=True)
    assert_close(out2.cpu().numpy(), want, scale + np.abs(bias)[None, :, None], 1e-5, "bias+relu")


def test_reference_launcher_names_through_c_abi(oracle, dev):
    """iex_CudaSpmm3 / iex_CudaSpmm2 / iex_CudaSpmm5 called with raw pointers, the way a
    binding of csrc/extensions.h:28-30 would."""
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    a, b_np, _, _ = W.config1()
    ri, v, ro, ci = to_dev(a, dev)
    b = torch.from_numpy(b_np).to(dev)
    s = torch.cuda.current_stream().cuda_stream
    want = oracle.spmm(b_np, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m)
    scale = oracle.spmm_abs_scale(b_np, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m)
    out = torch.empty(1, a.m, 256, device=dev)
    assert lib.iex_CudaSpmm3(a.m, a.k, 256, a.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                             b.data_ptr(), out.data_ptr(), s, 1) == 0
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "iex_CudaSpmm3")
    out.zero_()
    assert lib.iex_CudaSpmm2(a.m, a.k, 256, a.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                             b.data_ptr(), out.data_ptr(), s, 1) == 0
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "iex_CudaSpmm2")
    outh = torch.empty(1, a.m, 256, device=dev, dtype=torch.float16)
    assert lib.iex_CudaSpmm5(a.m, a.k, 256, a.nnz, ri.data_ptr(), v.half().data_ptr(), ro.data_ptr(),
                             ci.to(torch.int16).data_ptr(), b.half().data_ptr(), outh.data_ptr(), s, 1) == 0
    wanth = oracle.spmm(rounded(b_np, torch.float16), a.row_indices, rounded(a.values, torch.float16), a.row_offsets,
                        a.column_indices, a.m)
    assert_close(outh.float().cpu().numpy(), wanth, scale, 1e-2, "iex_CudaSpmm5")


def test_unreferenced_nan_rows_do_not_leak(dev):
    """Row 0 of the dense operand holds NaN but no nonzero points at column 0: the result
    must stay finite (padding slots never touch memory they were not asked to read)."""
    rng = np.random.default_rng(8)
    m, k, n = 130, 300, 64
    lens = rng.integers(1, 70, m)
    ro, ci = W.csr_from_row_lengths(rng, m, k - 1, lens)
    ci = ci + 1  # shift: column 0 never used
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b = torch.randn(1, k, n, device=dev)
    b[0, 0] = float("nan")
    ri, v, ro_t, ci_t = to_dev(csr, dev)
    assert torch.isfinite(ops.spmm_sputnik_reuse_weight(b, ri, v, ro_t, ci_t, m)).all()
    assert torch.isfinite(ops.spmm_sputnik_reuse_weight_half(b.half(), ri, v.half(), ro_t, ci_t, m)).all()


def test_misaligned_operands_take_the_scalar_path(oracle, dev):
    rng = np.random.default_rng(9)
    a = W.config2_matrix(0.90, m=128, k=128)
    n = 64
    b_np = rng.standard_normal((1, 128, n)).astype(np.float32)
    store = torch.empty(128 * n + 1, device=dev, dtype=torch.float16)
    b = store[1:].view(1, 128, n)      # 2-byte aligned only
    b.copy_(torch.from_numpy(b_np))
    ri, v, ro, ci = to_dev(a, dev, torch.float16)
    out = ops.spmm_sputnik_reuse_weight_half(b, ri, v, ro, ci, a.m)
    want = oracle.spmm(rounded(b_np, torch.float16), a.row_indices, rounded(a.values, torch.float16), a.row_offsets,
                       a.column_indices, a.m)
    scale = oracle.spmm_abs_scale(b_np, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m)
    assert_close(out.float().cpu().numpy(), want, scale, 1e-2, "misaligned")


def test_full_size_config4_integer_exact(dev):
    """Config-4 shape (11008x4096 @ 90 %, 2048 tokens) with small-integer operands: the fp16
    result must equal the exact product, computed densely in float64 on the device."""
    rng = np.random.default_rng(20)
    w = W.pruned_weight(20, 11008, 4096, 0.90)
    w.values = (rng.integers(1, 3, w.nnz) * rng.choice([-1, 1], w.nnz)).astype(np.float32)
    x = torch.from_numpy(rng.integers(-2, 3, (1, 4096, 2048)).astype(np.float32)).to(dev)
    ri, v, ro, ci = to_dev(w, dev, torch.float16, torch.int16)
    out = ops.spmm_sputnik_reuse_weight_half(x.half(), ri, v, ro, ci, w.m)
    from intrasm_engine_amd.pytorch.utils import sparse_to_dense
    dense = sparse_to_dense(w.m, w.k, v.double(), ro, ci.to(torch.int32))
    want = dense @ x[0].double()
    assert want.abs().max() < 2048  # exactly representable in fp16
    assert torch.equal(out[0].double(), want)


@pytest.mark.parametrize("shape", ["config4", "q_2to4"])
def test_full_size_dense_form_agrees_with_the_other_families(dev, shape):
    """At the full sizes of config 4 (11008 x 4096 at 90 %, 2048 tokens) and of a 2:4 projection of the
    decoder layer (4096 x 4096, 8192 tokens), random fp16 operands: the operator's result (dense form + GEMM)
    equals the matrix-core SpMM kernel's bit for bit -- two independent ways to the same MFMA sequence
    over k -- and the gather kernel's to the fp16 tolerance, on a strided sample of rows."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(21)
    if shape == "config4":
        w, n = W.pruned_weight(21, 11008, 4096, 0.90), 2048
    else:
        m = k = 4096
        keep = np.argsort(rng.random((m, k // 4, 4)), axis=2)[:, :, :2] + 4 * np.arange(k // 4)[None, :, None]
        ci = np.sort(keep.reshape(m, k // 2), axis=1).reshape(-1).astype(np.int32)
        ro = (np.arange(m + 1) * (k // 2)).astype(np.int32)
        w, n = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci), 8192
    ri, v, ro_t, ci_t = to_dev(w, dev, torch.float16, torch.int16)
    x = torch.randn(1, w.k, n, device=dev, generator=torch.Generator(dev).manual_seed(5)).half()
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float16,), allow_i16=True)
    auto = pyops._spmm(x, ri, v, ro_t, ci_t, w.m, **kw)
    assert torch.equal(auto, pyops._spmm(x, ri, v, ro_t, ci_t, w.m, force_variant=7, **kw))     # the dense form is what ran
    assert torch.equal(auto, pyops._spmm(x, ri, v, ro_t, ci_t, w.m, force_variant=4, **kw))
    rows = slice(0, w.m, 37)
    gather = pyops._spmm(x, ri, v, ro_t, ci_t, w.m, force_variant=1, **kw)[0, rows].float()
    scale = float(gather.abs().max())
    assert torch.allclose(auto[0, rows].float(), gather, rtol=1e-2, atol=1e-2 * scale)


def test_operator_argument_checks(dev):
    a, b_np, _, _ = W.config1()
    ri, v, ro, ci = to_dev(a, dev)
    b = torch.from_numpy(b_np).to(dev)
    with pytest.raises(RuntimeError, match="b must be a CUDA tensor"):
        ops.spmm_sputnik_reuse_weight(b.cpu(), ri, v, ro, ci, a.m)
    with pytest.raises(RuntimeError, match="b must be a contiguous tensor"):
        ops.spmm_sputnik_reuse_weight(b.transpose(1, 2), ri, v, ro, ci, a.m)
    with pytest.raises(RuntimeError):
        ops.spmm_sputnik_reuse_weight(b[0], ri, v, ro, ci, a.m)              # b.dim() != 3
    with pytest.raises(RuntimeError):
        ops.spmm_sputnik_reuse_weight(b, ri, v[:-1], ro, ci, a.m)            # values vs column_indices
    with pytest.raises(RuntimeError, match="multiple of 4"):
        ops.spmm_sputnik_atomic(b.repeat(2, 1, 1), ri, v[:-2].repeat(2, 1), ro, ci[:-2], a.m)


@pytest.mark.parametrize("rpw", [2, 4, 8])
@pytest.mark.parametrize("dtype,n", [(torch.float32, 256), (torch.float32, 384), (torch.float32, 128),
                                     (torch.float16, 512), (torch.float16, 256), (torch.bfloat16, 512)])
def test_lds_staged_variant(oracle, dev, rpw, dtype, n):
    """The LDS-staged kernel (forced) on a skewed matrix with empty rows, a dense row, a
    k that is not a multiple of the stage height and an m that leaves idle row slots."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(7 * rpw + n)
    m, k = 333, 1000
    lens = np.clip(rng.geometric(1 / 120.0, m), 0, k)
    lens[[0, 17, 332]] = 0
    lens[5] = k
    lens[6] = 1
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((2, k, n)).astype(np.float32)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    b = torch.from_numpy(b_np).to(dev).to(dtype)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=False, dtypes=(dtype,),
                      allow_i16=False, force_variant=2, force_rpw=rpw)
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"lds rpw={rpw} {dtype} n={n}")
    # both kernel families agree on integer-valued data exactly
    csr.values = rng.integers(-2, 3, csr.nnz).astype(np.float32)
    bi = torch.from_numpy(rng.integers(-2, 3, (1, k, n)).astype(np.float32)).to(dev).to(dtype)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(dtype,), allow_i16=False)
    assert torch.equal(pyops._spmm(bi, ri, v, ro_t, ci_t, m, force_variant=2, force_rpw=rpw, **kw),
                       pyops._spmm(bi, ri, v, ro_t, ci_t, m, force_variant=1, **kw))


@pytest.mark.parametrize("family,knob", [(3, 8), (3, 16), (4, 1), (4, 2), (4, 4), (4, 5), (6, 1), (6, 2), (6, 4)])
@pytest.mark.parametrize("dtype,n,itype", [(torch.float16, 264, torch.int16), (torch.float16, 512, torch.int32),
                                           (torch.bfloat16, 776, torch.int32), (torch.float16, 8, torch.int16)])
def test_matrix_core_variants(oracle, dev, family, knob, dtype, n, itype):
    """The kernels that expand A to dense tiles in LDS and multiply on the matrix cores
    (forced): skewed matrix with empty rows, a completely dense row (runs longer than the
    register windows), k not a multiple of the 32- and 128-column steps, m that leaves idle
    row slots, n that leaves a partial column tile."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(11 * family + knob + n)
    m, k = 333, 1000
    lens = np.clip(rng.geometric(1 / 120.0, m), 0, k)
    lens[[0, 17, 332]] = 0
    lens[5] = k
    lens[6] = 1
    lens[7] = 700
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((2, k, n)).astype(np.float32)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    ci_t = ci_t.to(itype)
    b = torch.from_numpy(b_np).to(dev).to(dtype)
    force = dict(force_variant=family, force_lpg=knob) if family == 3 else dict(force_variant=family, force_rpw=knob)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(dtype,), allow_i16=True)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, **force, **kw)
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"matrix-core family {family}/{knob} {dtype} n={n}",
                 atol=FP16_SUBNORMAL_HALF_STEP if dtype == torch.float16 else 0.0)
    # integer-valued data: every family is exact, so they agree bit for bit
    csr.values = rng.integers(-2, 3, csr.nnz).astype(np.float32)
    bi = torch.from_numpy(rng.integers(-2, 3, (1, k, n)).astype(np.float32)).to(dev).to(dtype)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    ci_t = ci_t.to(itype)
    assert torch.equal(pyops._spmm(bi, ri, v, ro_t, ci_t, m, **force, **kw),
                       pyops._spmm(bi, ri, v, ro_t, ci_t, m, force_variant=1, **kw))


@pytest.mark.parametrize("arrangement", [1, 2, 4, 5, 6])
@pytest.mark.parametrize("windows", [0, 2, 4, 8])
@pytest.mark.parametrize("n", [260, 128, 64, 4])
def test_matrix_core_fp32(oracle, dev, arrangement, windows, n):
    """The fp32 kernel on v_mfma_f32_32x32x2 / 16x16x4 (forced), every tile arrangement, with
    separate expanding waves (windows = 0) and with waves that do both and hold 2, 4 or 8
    windows, on the same skewed matrix: empty rows, a completely dense row, ragged m, k and n."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(100 * arrangement + windows + n)
    m, k = 333, 1000
    lens = np.clip(rng.geometric(1 / 120.0, m), 0, k)
    lens[[0, 17, 332]] = 0
    lens[5] = k
    lens[6] = 1
    lens[7] = 700
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((2, k, n)).astype(np.float32)
    ri, v, ro_t, ci_t = to_dev(csr, dev)
    b = torch.from_numpy(b_np).to(dev)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float32,), allow_i16=False)
    force = dict(force_variant=5, force_nt=arrangement)
    if windows:
        force.update(force_rpw=windows, force_lpg=8)   # lanes-per-group code 8 = no separate expanding waves
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, **force, **kw)
    want = oracle.spmm(b_np, csr.row_indices, csr.values, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_np, csr.row_indices, csr.values, csr.row_offsets, csr.column_indices, m)
    assert_close(out.cpu().numpy(), want, scale, RTOL[torch.float32], f"fp32 matrix-core {arrangement}/{windows} n={n}")
    csr.values = rng.integers(-2, 3, csr.nnz).astype(np.float32)
    bi = torch.from_numpy(rng.integers(-2, 3, (1, k, n)).astype(np.float32)).to(dev)
    ri, v, ro_t, ci_t = to_dev(csr, dev)
    assert torch.equal(pyops._spmm(bi, ri, v, ro_t, ci_t, m, **force, **kw),
                       pyops._spmm(bi, ri, v, ro_t, ci_t, m, force_variant=1, **kw))


def test_matrix_core_fp32_epilogue_options(oracle, dev):
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(55)
    m, k, n, batch = 200, 300, 132, 3
    csr = W.pruned_weight(45, m, k, 0.6)
    ri, v, ro_t, ci_t = to_dev(csr, dev)
    b_np = rng.standard_normal((batch, k, n)).astype(np.float32)
    b = torch.from_numpy(b_np).to(dev)
    base = oracle.spmm(b_np, csr.row_indices, csr.values, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_np, csr.row_indices, csr.values, csr.row_offsets, csr.column_indices, m)
    kw = dict(dtypes=(torch.float32,), allow_i16=False, force_variant=5)
    bias_np = rng.standard_normal(m).astype(np.float32)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=False,
                      bias=torch.from_numpy(bias_np).to(dev), relu=True, **kw)
    assert_close(out.cpu().numpy(), np.maximum(base + bias_np[None, :, None], 0.0), scale + np.abs(bias_np)[None, :, None],
                 1e-5, "fp32 bias+relu")
    prev_np = rng.standard_normal((batch, m, n)).astype(np.float32)
    prev = torch.from_numpy(prev_np).to(dev)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=True, out=prev, **kw)
    assert_close(out.cpu().numpy(), base + prev_np, scale + np.abs(prev_np), 1e-5, "fp32 accumulate")
    vb_np = rng.standard_normal((batch, csr.nnz)).astype(np.float32)
    out = pyops._spmm(b, ri, torch.from_numpy(vb_np).to(dev), ro_t, ci_t, m, per_batch_values=True, accumulate=False, **kw)
    for z in range(batch):
        want = oracle.spmm(b_np[z:z + 1], csr.row_indices, vb_np[z], csr.row_offsets, csr.column_indices, m)
        sc = oracle.spmm_abs_scale(b_np[z:z + 1], csr.row_indices, vb_np[z], csr.row_offsets, csr.column_indices, m)
        assert_close(out[z:z + 1].cpu().numpy(), want, sc, 1e-5, f"fp32 per-batch values z={z}")


@pytest.mark.parametrize("family", [3, 4])
def test_matrix_core_epilogue_options(oracle, dev, family):
    """bias + ReLU, accumulation into the output and per-batch values on the matrix-core kernels."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(family)
    m, k, n, batch = 200, 300, 128, 3
    csr = W.pruned_weight(40 + family, m, k, 0.8)
    ri, v, ro_t, ci_t = to_dev(csr, dev, torch.float16)
    b_np = rng.standard_normal((batch, k, n)).astype(np.float32)
    b = torch.from_numpy(b_np).to(dev).half()
    b_r, vals_r = rounded(b_np, torch.float16), rounded(csr.values, torch.float16)
    base = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    kw = dict(dtypes=(torch.float16,), allow_i16=True, force_variant=family)
    # bias + ReLU
    bias_np = rng.standard_normal(m).astype(np.float32)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=False,
                      bias=torch.from_numpy(bias_np).to(dev), relu=True, **kw)
    assert_close(out.float().cpu().numpy(), np.maximum(base + bias_np[None, :, None], 0.0), scale + np.abs(bias_np)[None, :, None],
                 RTOL[torch.float16], "bias+relu")
    # accumulate
    prev_np = rounded(rng.standard_normal((batch, m, n)).astype(np.float32), torch.float16)
    prev = torch.from_numpy(prev_np).to(dev).half()
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=True, out=prev, **kw)
    assert out.data_ptr() == prev.data_ptr()
    assert_close(out.float().cpu().numpy(), base + prev_np, scale + np.abs(prev_np), RTOL[torch.float16], "accumulate")
    # per-batch values
    vb_np = rng.standard_normal((batch, csr.nnz)).astype(np.float32)
    vb = torch.from_numpy(vb_np).to(dev).half()
    out = pyops._spmm(b, ri, vb, ro_t, ci_t, m, per_batch_values=True, accumulate=False, **kw)
    vb_r = rounded(vb_np, torch.float16)
    for z in range(batch):
        want = oracle.spmm(b_r[z:z + 1], csr.row_indices, vb_r[z], csr.row_offsets, csr.column_indices, m)
        sc = oracle.spmm_abs_scale(b_r[z:z + 1], csr.row_indices, vb_r[z], csr.row_offsets, csr.column_indices, m)
        assert_close(out[z:z + 1].float().cpu().numpy(), want, sc, RTOL[torch.float16], f"per-batch values z={z}")


@pytest.mark.parametrize("dtype,k,n,density,family", [(torch.float16, 320, 2048, 0.5, 4), (torch.float16, 320, 1024, 0.5, 3),
                                                      (torch.float16, 320, 2048, 0.5, 6), (torch.bfloat16, 512, 4096, 0.5, 6),
                                                      (torch.float32, 320, 1024, 0.5, 5), (torch.float32, 8192, 2048, 0.1, 2)])
def test_automatic_choice_of_kernel_family(oracle, dev, dtype, k, n, density, family):
    """Shapes on which the library leaves the row kernel by itself: 16-bit operands of moderate
    density go to the matrix-core kernels (8 waves when that still fills the chip, else 4; the
    direct-load kernel, family 6, when exactly half of the entries are nonzero, as in 2:4 weights),
    fp32 of high density to the fp32 matrix-core kernel, fp32 of low density with a long k
    (the slice of the dense operand outgrows an L2) to the LDS-staged gather.
    Checked against the oracle, and bit-equal to the forced family, which shows which one ran."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(n)
    m = 4096
    lens = np.full(m, int(density * k))
    if family != 6:
        lens[::97] = 0          # (empty rows; the nonzeros are then no longer exactly half of the matrix)
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((1, k, n)).astype(np.float32)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    b = torch.from_numpy(b_np).to(dev).to(dtype)
    # (no workspace: the choice among the kernels that need none, what iex_spmm_ex does)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(dtype,), allow_i16=False, no_workspace=True)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, **kw)
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"auto staged {dtype} n={n}")
    assert torch.equal(out, pyops._spmm(b, ri, v, ro_t, ci_t, m, force_variant=family, **kw))
    row = pyops._spmm(b, ri, v, ro_t, ci_t, m, force_variant=1, **kw)
    if family >= 3:
        assert not torch.equal(out, row)   # the matrix cores sum in another order
    assert torch.allclose(out.float(), row.float(), rtol=1e-2, atol=1e-2 * float(scale.max()))


@pytest.mark.parametrize("dtype,n", [(torch.float32, 1024), (torch.float32, 1280), (torch.float16, 2048),
                                     (torch.float16, 2560), (torch.bfloat16, 2048)])
def test_two_tiles_per_wave(oracle, dev, dtype, n):
    """Wide outputs: a wave covers two adjacent 64-lane tiles (chosen automatically from four
    tiles upwards); n = 1280 / 2560 leave the second tile of the last block empty."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(n)
    m, k = 150, 600
    lens = np.clip(rng.geometric(1 / 90.0, m), 0, k)
    lens[[0, 149]] = 0
    lens[3] = k
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((1, k, n)).astype(np.float32)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    b = torch.from_numpy(b_np).to(dev).to(dtype)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(dtype,), allow_i16=False)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, **kw)
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"nt auto {dtype} n={n}")
    # one and two tiles per wave sum a row in the same order: bit-equal
    assert torch.equal(out, pyops._spmm(b, ri, v, ro_t, ci_t, m, force_nt=1, force_wpr=4, **kw))
    assert torch.equal(out, pyops._spmm(b, ri, v, ro_t, ci_t, m, force_nt=2, force_wpr=4, **kw))


@pytest.mark.parametrize("wpr", [1, 4, 8])
@pytest.mark.parametrize("dtype,n", [(torch.float32, 785), (torch.float32, 197), (torch.float32, 130), (torch.float32, 257),
                                     (torch.float16, 785), (torch.float16, 263), (torch.bfloat16, 513)])
def test_rows_that_are_not_a_multiple_of_the_vector(oracle, dev, wpr, dtype, n):
    """n = 785 and 197 are the ViT shapes of the reference's xformers sweep: wide rows whose length is no
    multiple of the 128-bit vector run with 128-bit accesses at element alignment; the one lane per row whose
    vector would pass the end of the row reads back-shifted and stores only its own elements.  Checked with a
    batch (row starts at every alignment), accumulate mode and bias + ReLU, against the oracle, and bit for
    bit against the narrow-vector kernel (force_lpg leaves the ragged path), which sums in the same order."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(n + wpr)
    m, k, batch = 75, 300, 3
    lens = np.clip(rng.geometric(1 / 40.0, m), 0, k)
    lens[[0, 74]] = 0
    lens[3] = k
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((batch, k, n)).astype(np.float32)
    bias_np = rng.standard_normal(m).astype(np.float32)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    b = torch.from_numpy(b_np).to(dev).to(dtype)
    kw = dict(per_batch_values=False, dtypes=(dtype,), allow_i16=False, force_wpr=wpr)
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, accumulate=False, **kw)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"ragged rows {dtype} n={n} wpr={wpr}",
                 atol=FP16_SUBNORMAL_HALF_STEP if dtype == torch.float16 else 0.0)
    assert torch.equal(out, pyops._spmm(b, ri, v, ro_t, ci_t, m, accumulate=False, force_lpg=64, **kw))
    # bias + ReLU
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, accumulate=False, bias=torch.from_numpy(bias_np).to(dev), relu=True, **kw)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m, bias=bias_np, relu=True)
    assert_close(out.float().cpu().numpy(), want, scale + np.abs(bias_np)[None, :, None], RTOL[dtype], "ragged rows, bias + ReLU")
    # accumulate into a pre-filled output
    init_np = rng.standard_normal((batch, m, n)).astype(np.float32)
    init = torch.from_numpy(init_np).to(dev).to(dtype)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, accumulate=True, out=init.clone(), **kw)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m, out_init=rounded(init_np, dtype))
    assert_close(out.float().cpu().numpy(), want, scale + np.abs(init_np), RTOL[dtype], "ragged rows, accumulate")


def _dense_form_case(rng, m, k, n, batch, dtype, itype, dev, mean_len=30.0):
    lens = np.clip(rng.geometric(1 / mean_len, m), 0, k)
    lens[0] = 0
    lens[3] = k
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    b_np = rng.standard_normal((batch, k, n)).astype(np.float32)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype)
    return csr, b_np, (ri, v, ro_t, ci_t.to(itype)), torch.from_numpy(b_np).to(dev).to(dtype)


@pytest.mark.parametrize("dtype,itype,m,k,n,batch", [(torch.float16, torch.int16, 203, 160, 256, 2),
                                                     (torch.bfloat16, torch.int32, 75, 304, 264, 1),
                                                     (torch.float16, torch.int16, 130, 64, 8, 3),
                                                     (torch.float16, torch.int32, 16, 16392, 512, 1)])
def test_dense_form_path(oracle, dev, dtype, itype, m, k, n, batch):
    """Family 7: the dense form of A written into a workspace, then the dense GEMM.  Empty rows, a
    full row, a batch, a k beyond one segment of the row assembly (and no multiple of it)."""
    from intrasm_engine_amd.pytorch import ops as pyops
    csr, b_np, (ri, v, ro_t, ci_t), b = _dense_form_case(np.random.default_rng(m + n), m, k, n, batch, dtype, itype, dev)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=False, dtypes=(dtype,),
                      allow_i16=True, force_variant=7)
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"dense form {dtype} {m}x{k}x{n}")


@pytest.mark.parametrize("dtype,itype,batch,m,k,n,sparsity", [
    (torch.float32, torch.int32, 2, 203, 32, 256, 0.9), (torch.float32, torch.int32, 3, 1000, 128, 516, 0.5),
    (torch.float32, torch.int32, 1, 77, 1, 1024, 0.0), (torch.float16, torch.int16, 2, 300, 100, 520, 0.7),
    (torch.bfloat16, torch.int32, 1, 130, 64, 2048, 0.95), (torch.float32, torch.int32, 1, 5000, 16, 260, 0.99),
    (torch.float32, torch.int32, 2, 197, 64, 785, 0.8), (torch.float16, torch.int16, 2, 150, 32, 1003, 0.9),
    (torch.float32, torch.int32, 1, 90, 48, 257, 0.7)])
def test_few_columns_kernel(oracle, dev, dtype, itype, batch, m, k, n, sparsity):
    """Family 8 (A with at most 128 columns, wide output: the dense operand's tile in LDS, rows streamed in
    natural order): per-batch values and shared values with bias + ReLU + accumulate, an empty first row,
    a single column, a last tile that is partly outside the matrix, rows that are no multiple of the 128-bit
    vector (785, 1003, 257: element-aligned accesses, one back-shifted lane per row).  Against the oracle, and bit-equal to
    the row kernel with one wavefront per row (same order of summation)."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(m + k)
    mask = rng.random((m, k)) >= sparsity
    mask[0] = False
    ro, ci, _ = W.csr_from_mask(mask)
    csr = W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    ri, v, ro_t, ci_t = to_dev(csr, dev, dtype, itype)
    b_np = rng.standard_normal((batch, k, n)).astype(np.float32)
    b = torch.from_numpy(b_np).to(dev).to(dtype)
    vb_np = rng.standard_normal((batch, csr.nnz)).astype(np.float32)
    vb = torch.from_numpy(vb_np).to(dev).to(dtype)
    kw = dict(dtypes=(dtype,), allow_i16=True)
    out = pyops._spmm(b, ri, vb, ro_t, ci_t, m, per_batch_values=True, accumulate=False, force_variant=8, **kw)
    assert torch.equal(out, pyops._spmm(b, ri, vb, ro_t, ci_t, m, per_batch_values=True, accumulate=False,
                                        force_variant=1, force_wpr=1, **kw))
    b_r, vb_r = rounded(b_np, dtype), rounded(vb_np, dtype)
    for z in range(batch):
        want = oracle.spmm(b_r[z:z + 1], csr.row_indices, vb_r[z], csr.row_offsets, csr.column_indices, m)
        sc = oracle.spmm_abs_scale(b_r[z:z + 1], csr.row_indices, vb_r[z], csr.row_offsets, csr.column_indices, m)
        assert_close(out[z:z + 1].float().cpu().numpy(), want, sc, RTOL[dtype], f"few columns, per-batch values z={z}",
                     atol=FP16_SUBNORMAL_HALF_STEP if dtype == torch.float16 else 0.0)
    bias = torch.randn(m, device=dev)
    prev = torch.randn(batch, m, n, device=dev).to(dtype)
    kw2 = dict(per_batch_values=False, accumulate=True, bias=bias, relu=True, **kw)
    got = pyops._spmm(b, ri, v, ro_t, ci_t, m, force_variant=8, out=prev.clone(), **kw2)
    assert torch.equal(got, pyops._spmm(b, ri, v, ro_t, ci_t, m, force_variant=1, force_wpr=1, out=prev.clone(), **kw2))


def test_few_columns_kernel_long_runs_of_rows_and_refusals(dev):
    """40000 rows, k = 128: a wavefront walks 64 rows (two groups of row offsets), the nonzeros of a group
    span several 64-entry reads.  The library takes the kernel by itself here (bit-equal to forcing it);
    shapes it cannot serve are refused on request."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(9)
    m, k, n, batch = 40000, 128, 512, 8
    mask = rng.random((m, k)) >= 0.97
    ro, ci, _ = W.csr_from_mask(mask)
    ri = torch.from_numpy(W.swizzle_from_offsets(ro)).to(dev)
    ro_t, ci_t = torch.from_numpy(ro).to(dev), torch.from_numpy(ci).to(dev)
    v = torch.randn(ci.shape[0], device=dev)
    b = torch.randn(batch, k, n, device=dev)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float32,), allow_i16=False)
    row = pyops._spmm(b, ri, v, ro_t, ci_t, m, force_variant=1, force_wpr=1, **kw)
    assert torch.equal(pyops._spmm(b, ri, v, ro_t, ci_t, m, force_variant=8, **kw), row)
    assert torch.equal(pyops._spmm(b, ri, v, ro_t, ci_t, m, **kw), row)
    with pytest.raises(RuntimeError, match="few-columns kernel needs"):
        pyops._spmm(b[:, :, :130].contiguous(), ri, v, ro_t, ci_t, m, force_variant=8, **kw)      # n = 130
    wide = torch.randn(1, 256, 512, device=dev)
    with pytest.raises(RuntimeError, match="few-columns kernel needs"):
        pyops._spmm(wide, ri[:8], v[:1], torch.zeros(9, dtype=torch.int32, device=dev), ci_t[:1], 8, force_variant=8, **kw)  # k = 256


def test_dense_form_path_epilogue_options(oracle, dev):
    """bias + ReLU and accumulation into the output ride in the GEMM's epilogue; per-batch values have
    no single dense form and are refused on request."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(77)
    m, k, n, batch = 200, 304, 136, 3
    csr = W.pruned_weight(47, m, k, 0.8)
    ri, v, ro_t, ci_t = to_dev(csr, dev, torch.bfloat16)
    b_np = rng.standard_normal((batch, k, n)).astype(np.float32)
    b = torch.from_numpy(b_np).to(dev).bfloat16()
    b_r, vals_r = rounded(b_np, torch.bfloat16), rounded(csr.values, torch.bfloat16)
    base = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    kw = dict(dtypes=(torch.bfloat16,), allow_i16=False, force_variant=7)
    bias_np = rng.standard_normal(m).astype(np.float32)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=False,
                      bias=torch.from_numpy(bias_np).to(dev), relu=True, **kw)
    assert_close(out.float().cpu().numpy(), np.maximum(base + bias_np[None, :, None], 0.0), scale + np.abs(bias_np)[None, :, None],
                 RTOL[torch.bfloat16], "bias+relu")
    prev_np = rounded(rng.standard_normal((batch, m, n)).astype(np.float32), torch.bfloat16)
    prev = torch.from_numpy(prev_np).to(dev).bfloat16()
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, per_batch_values=False, accumulate=True, out=prev, **kw)
    assert out.data_ptr() == prev.data_ptr()
    assert_close(out.float().cpu().numpy(), base + prev_np, scale + np.abs(prev_np), RTOL[torch.bfloat16], "accumulate")
    vb = torch.randn(batch, csr.nnz, device=dev).bfloat16()
    with pytest.raises(RuntimeError, match="dense-form path needs"):
        pyops._spmm(b, ri, vb, ro_t, ci_t, m, per_batch_values=True, accumulate=False, **kw)


def test_dense_form_path_is_chosen_with_a_workspace_and_only_then(oracle, dev):
    """2048 x 2048 at 80 % sparsity times 2048 x 1024 in fp16: the time model prefers the dense form
    (measured 34 against 71 us).  The operator asks the library for the workspace size, allocates it
    and gets the dense-form result; the entry point without a workspace, a short workspace, and
    shapes the path does not serve (fp32, per-batch values, a small product) run the other kernels."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    lib = _lib.load()
    m = k = 2048
    n = 1024
    dtype = torch.float16
    rng = np.random.default_rng(12)
    csr, b_np, (ri, v, ro_t, ci_t), b = _dense_form_case(rng, m, k, n, 1, dtype, torch.int16, dev, mean_len=0.2 * k)
    nnz = csr.column_indices.shape[0]
    need = lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, 0, m, k, n, nnz, 1)
    assert need == m * k * 2
    assert lib.iex_spmm_workspace_bytes(_lib.F32, _lib.I32, 0, m, k, n, nnz, 1) == 0
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, _lib.SPMM_PER_BATCH_VALUES, m, k, n, nnz, 1) == 0
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, _lib.SPMM_ACCUMULATE | _lib.SPMM_RELU, m, k, n, nnz, 1) == need
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, 0, 128, 128, 64, 1000, 1) == 0  # too small to pay
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, 0, m, k, n - 4, nnz, 1) == 0    # n no multiple of 8
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, 7 << 16, 128, 128, 64, 1000, 1) == 128 * 128 * 2  # on request
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(dtype,), allow_i16=True)
    auto = pyops._spmm(b, ri, v, ro_t, ci_t, m, **kw)
    assert torch.equal(auto, pyops._spmm(b, ri, v, ro_t, ci_t, m, force_variant=7, **kw))
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(auto.float().cpu().numpy(), want, scale, RTOL[dtype], "dense form, chosen")
    # without a workspace, and with one that is too short, the gather kernel runs: bit-equal to family 1
    row = pyops._spmm(b, ri, v, ro_t, ci_t, m, force_variant=1, **kw)
    assert torch.equal(pyops._spmm(b, ri, v, ro_t, ci_t, m, no_workspace=True, **kw), row)
    assert not torch.equal(auto, row)   # (the matrix cores sum in another order)
    short = torch.empty(need - 16, dtype=torch.uint8, device=dev)
    out = torch.empty_like(row)
    args = (_lib.F16, _lib.I16, 0, m, k, n, nnz, ri.data_ptr(), v.data_ptr(), ro_t.data_ptr(), ci_t.data_ptr(),
            b.data_ptr(), None, out.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert lib.iex_spmm_ws(*args, short.data_ptr(), need - 16) == 0, _lib.last_error()
    assert torch.equal(out, row)
    # the path on request where it cannot run: an error, not another kernel
    forced = (_lib.F16, _lib.I16, 7 << 16) + args[3:]
    assert lib.iex_spmm_ex(*forced) != 0 and "workspace" in _lib.last_error()
    assert lib.iex_spmm_ws(*forced, short.data_ptr(), need - 16) != 0 and "workspace" in _lib.last_error()
    torch.cuda.synchronize()


def test_dense_form_path_splits_k_where_the_product_has_few_tiles(oracle, dev):
    """4096 x 4096 at 70 % sparsity times 4096 x 128 in fp16: the dense form wins, and its product is 64 tiles of 64 x 128
    with k = 4096, which the GEMM runs with k in four parts when it has room for the partial sums.  The size the
    library asks for holds that room behind the dense form; the kernel that writes the dense form zeroes the tile words
    (no launch of its own for that); a workspace of the dense form alone still runs the path, unsplit; both agree with
    the oracle and every repeat gives the same bits."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    lib = _lib.load()
    m = k = 4096
    n = 128
    dtype = torch.float16
    rng = np.random.default_rng(21)
    csr, b_np, (ri, v, ro_t, ci_t), b = _dense_form_case(rng, m, k, n, 1, dtype, torch.int16, dev, mean_len=0.3 * k)
    nnz = csr.column_indices.shape[0]
    need = lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, 0, m, k, n, nnz, 1)
    assert need == m * k * 2 + lib.iex_gemm_workspace_bytes(_lib.F16, 0, m, n, k, 1) and need > m * k * 2
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, _lib.SPMM_ACCUMULATE, m, k, n, nnz, 1) == m * k * 2   # (the split stores plainly)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(dtype,), allow_i16=True)
    out = pyops._spmm(b, ri, v, ro_t, ci_t, m, **kw)
    trail = _lib.last_kernels()
    assert "csr_to_dense_kernel" in trail and "gemm_dma_parts_kernel" in trail and "K in 4 parts" in trail and "fill_zero" not in trail
    for _ in range(3):
        assert torch.equal(out, pyops._spmm(b, ri, v, ro_t, ci_t, m, **kw))
    vals_r, b_r = rounded(csr.values, dtype), rounded(b_np, dtype)
    want = oracle.spmm(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_r, csr.row_indices, vals_r, csr.row_offsets, csr.column_indices, m)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], "dense form, k in parts")
    small = torch.empty(m * k * 2, dtype=torch.uint8, device=dev)
    unsplit = torch.empty_like(out)
    args = (_lib.F16, _lib.I16, 0, m, k, n, nnz, ri.data_ptr(), v.data_ptr(), ro_t.data_ptr(), ci_t.data_ptr(),
            b.data_ptr(), None, unsplit.data_ptr(), torch.cuda.current_stream().cuda_stream, 1)
    assert lib.iex_spmm_ws(*args, small.data_ptr(), m * k * 2) == 0, _lib.last_error()
    trail = _lib.last_kernels()
    assert "csr_to_dense_kernel" in trail and "parts" not in trail
    torch.cuda.synchronize()
    assert_close(unsplit.float().cpu().numpy(), want, scale, RTOL[dtype], "dense form, unsplit")


@pytest.mark.parametrize("idtype", [torch.int32, torch.int16])
def test_csr_check_finds_one_fault_wherever_it_sits(dev, idtype):
    """The check kernel reads 256 columns of a row per step, in four chunks of 64 whose left neighbours come from three
    places (the lane before, the chunk before, the step before): a single swapped pair, a single repeated column and a
    single column outside the matrix are found at every such seam of a long row, in a row of the middle of the matrix
    and in the last one, and a clean pattern reads 0."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(23)
    m, k = 9, 2000
    lens = np.array([700, 0, 1, 64, 256, 257, 700, 65, 700])
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    rot = torch.from_numpy(ro).to(dev)
    assert pyops.csr_check(rot, torch.from_numpy(ci).to(dev).to(idtype), k) == 0
    for r in (0, 6, 8):
        for at in (1, 63, 64, 65, 127, 128, 255, 256, 257, 319, 320, 511, 512, 513, 699):
            j = ro[r] + at
            swapped = ci.copy()
            swapped[j - 1], swapped[j] = ci[j], ci[j - 1]
            assert pyops.csr_check(rot, torch.from_numpy(swapped).to(dev).to(idtype), k) == _lib.CSR_NOT_ASCENDING, (r, at)
            twice = ci.copy()
            twice[j] = ci[j - 1]
            assert pyops.csr_check(rot, torch.from_numpy(twice).to(dev).to(idtype), k) == _lib.CSR_NOT_ASCENDING, (r, at)
            out = ci.copy()
            out[j] = k
            assert pyops.csr_check(rot, torch.from_numpy(out).to(dev).to(idtype), k) & _lib.CSR_COLUMN_OUT_OF_RANGE, (r, at)
    # the first column of a row is compared with nothing: every row starts below the last column of the row before
    low = ci.copy()
    for r in (2, 3, 4, 5, 6, 7, 8):
        low[ro[r]] = 0
    assert pyops.csr_check(rot, torch.from_numpy(low).to(dev).to(idtype), k) == 0


def test_csr_check_names_what_a_pattern_lacks(dev):
    """``iex_csr_check``: 0 for what ``dense_to_sparse`` produces; unsorted or duplicated columns (valid for the row
    kernel and for the reference, not for the other families), a column outside the matrix, offsets that do not run
    from 0 to nnz; int16 columns; an empty pattern.  The unsorted pattern then runs on the row kernel and still
    equals the sorted one's product."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(17)
    m, k, n = 300, 500, 64
    lens = rng.integers(0, 40, m)
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    rot, cit = torch.from_numpy(ro).to(dev), torch.from_numpy(ci).to(dev)
    assert pyops.csr_check(rot, cit, k) == 0
    assert pyops.csr_check(rot, cit.to(torch.int16), k) == 0
    assert pyops.csr_check(torch.zeros(m + 1, dtype=torch.int32, device=dev), cit[:0], k) == 0
    r = int(np.argmax(lens >= 3))
    swapped = ci.copy()
    swapped[ro[r]], swapped[ro[r] + 2] = ci[ro[r] + 2], ci[ro[r]]
    assert pyops.csr_check(rot, torch.from_numpy(swapped).to(dev), k) == _lib.CSR_NOT_ASCENDING
    twice = ci.copy()
    twice[ro[r] + 1] = ci[ro[r]]
    assert pyops.csr_check(rot, torch.from_numpy(twice).to(dev), k) == _lib.CSR_NOT_ASCENDING
    assert pyops.csr_check(rot, cit, int(ci.max())) & _lib.CSR_COLUMN_OUT_OF_RANGE
    short = ro.copy()
    short[-1] -= 1
    assert pyops.csr_check(torch.from_numpy(short).to(dev), cit, k) == _lib.CSR_BAD_OFFSETS
    back = ro.copy()
    back[5] = back[6] + 1
    assert pyops.csr_check(torch.from_numpy(back).to(dev), cit, k) & _lib.CSR_BAD_OFFSETS
    # any order is fine for the row kernel: same product as the sorted pattern with the values moved along
    values = rng.standard_normal(ci.shape[0]).astype(np.float32)
    moved = values.copy()
    moved[ro[r]], moved[ro[r] + 2] = values[ro[r] + 2], values[ro[r]]
    dense = torch.from_numpy(rng.standard_normal((1, k, n)).astype(np.float32)).to(dev)
    ri = torch.from_numpy(W.swizzle_from_offsets(ro)).to(dev)
    kw = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float32,), allow_i16=False, force_variant=1, force_wpr=1)
    a = pyops._spmm(dense, ri, torch.from_numpy(values).to(dev), rot, cit, m, **kw)
    b = pyops._spmm(dense, ri, torch.from_numpy(moved).to(dev), rot, torch.from_numpy(swapped).to(dev), m, **kw)
    rows = np.ones(m, bool)
    rows[r] = False
    assert torch.equal(a[0, torch.from_numpy(rows)], b[0, torch.from_numpy(rows)])
    assert torch.allclose(a[0, r], b[0, r], rtol=1e-5, atol=1e-5)
