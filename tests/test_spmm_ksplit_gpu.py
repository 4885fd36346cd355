"""The fp32 SpMM kernel that keeps a slice of the dense operand in LDS and splits k over workgroups (family 9,
on request only): parity with the CPU oracle and bit-stability, over ragged shapes, every tile width, one to
fifteen k slices, both workgroup sizes, and the epilogue options."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from _util import RTOL, assert_close, to_dev

pytestmark = pytest.mark.gpu
KW = dict(per_batch_values=False, accumulate=False, dtypes=(torch.float32,), allow_i16=False)


def _skewed(rng, m, k, mean):
    lens = np.clip(rng.geometric(1.0 / mean, m), 0, k)
    lens[[0, m // 2, m - 1]] = 0          # empty rows
    lens[5] = k                           # a completely dense row: 64 nonzeros in every stage
    lens[6] = 1
    lens[7] = (3 * k) // 4
    lens[8] = 8 + (-(int(lens.sum()) - int(lens[8]) + 8)) % 4      # nnz a multiple of 4 (the per-batch accumulate rule)
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    return W.CSR(m, k, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)


@pytest.mark.parametrize("slices", [0, 1, 2, 3, 8, 15])
@pytest.mark.parametrize("n,waves16", [(256, False), (256, True), (128, False), (64, False), (320, False), (8, False), (196, True)])
def test_ksplit_kernel_against_the_oracle(oracle, dev, slices, n, waves16):
    """m leaves idle row slots, k is no multiple of the stage height or of the slice count, n = 320 / 196 leave a
    partly filled column tile (n = 8 a nearly empty one); slices = 0 lets the library pick the count."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(100 * slices + n)
    m, k = 333, 1000
    csr = _skewed(rng, m, k, 120.0)
    b_np = rng.standard_normal((2, k, n)).astype(np.float32)
    ri, v, ro, ci = to_dev(csr, dev)
    b = torch.from_numpy(b_np).to(dev)
    force = dict(force_variant=9, force_rpw=slices, force_nt=2 if waves16 else 0)
    out = pyops._spmm(b, ri, v, ro, ci, m, **force, **KW)
    want = oracle.spmm(b_np, csr.row_indices, csr.values, csr.row_offsets, csr.column_indices, m)
    scale = oracle.spmm_abs_scale(b_np, csr.row_indices, csr.values, csr.row_offsets, csr.column_indices, m)
    assert_close(out.cpu().numpy(), want, scale, RTOL[torch.float32], f"k split, {slices} slices, n={n}")
    assert torch.equal(out, pyops._spmm(b, ri, v, ro, ci, m, **force, **KW))          # same call, same bits
    # integer-valued operands: exact in every family, so bit-equal to the row kernel whatever the slicing
    csr.values = rng.integers(-2, 3, csr.nnz).astype(np.float32)
    bi = torch.from_numpy(rng.integers(-2, 3, (1, k, n)).astype(np.float32)).to(dev)
    ri, v, ro, ci = to_dev(csr, dev)
    assert torch.equal(pyops._spmm(bi, ri, v, ro, ci, m, **force, **KW), pyops._spmm(bi, ri, v, ro, ci, m, force_variant=1, **KW))


@pytest.mark.parametrize("slices", [1, 4])
def test_ksplit_epilogue_options_and_per_batch_values(oracle, dev, slices):
    """Bias + ReLU, accumulation into an existing output and per-batch values, with and without the second
    (partial-sum) kernel."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(slices)
    m, k, n, batch = 200, 520, 128, 3
    csr = _skewed(rng, m, k, 60.0)
    b_np = rng.standard_normal((batch, k, n)).astype(np.float32)
    ri, v, ro, ci = to_dev(csr, dev)
    b = torch.from_numpy(b_np).to(dev)
    bias_np = rng.standard_normal(m).astype(np.float32)
    bias = torch.from_numpy(bias_np).to(dev)
    force = dict(force_variant=9, force_rpw=slices)
    got = pyops._spmm(b, ri, v, ro, ci, m, bias=bias, relu=True, **force, **KW)
    want = oracle.spmm(b_np, csr.row_indices, csr.values, csr.row_offsets, csr.column_indices, m, bias=bias_np, relu=True)
    scale = oracle.spmm_abs_scale(b_np, csr.row_indices, csr.values, csr.row_offsets, csr.column_indices, m) + np.abs(bias_np)[None, :, None]
    assert_close(got.cpu().numpy(), want, scale, 1e-5, "bias + relu")

    init_np = rng.standard_normal((batch, m, n)).astype(np.float32)
    vals2 = rng.standard_normal((batch, csr.nnz)).astype(np.float32)
    out = torch.from_numpy(init_np).to(dev)
    pyops._spmm(b, ri, torch.from_numpy(vals2).to(dev), ro, ci, m, per_batch_values=True, accumulate=True, dtypes=(torch.float32,),
                allow_i16=False, out=out, **force)
    want = oracle.spmm(b_np, csr.row_indices, vals2, csr.row_offsets, csr.column_indices, m, out_init=init_np)
    scale = oracle.spmm_abs_scale(b_np, csr.row_indices, vals2, csr.row_offsets, csr.column_indices, m) + np.abs(init_np)
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "accumulate, per-batch values")


def test_ksplit_on_a_headline_cell_and_refusals(oracle, dev):
    """One cell of the 4096 x 4096 sweep (90 % sparse, n = 256, the library's own slice count) against the oracle;
    shapes the kernel cannot take are refused, and so is a missing workspace through the C ABI."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    c = W.config2_matrix(0.90)
    b_np = W.config2_dense(256)
    ri, v, ro, ci = to_dev(c, dev)
    b = torch.from_numpy(b_np).to(dev)
    out = pyops._spmm(b, ri, v, ro, ci, c.m, force_variant=9, **KW)
    want = oracle.spmm(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
    scale = oracle.spmm_abs_scale(b_np, c.row_indices, c.values, c.row_offsets, c.column_indices, c.m)
    assert_close(out.cpu().numpy(), want, scale, 1e-5, "4096 x 4096 at 90 %, n = 256")

    lib = _lib.load()
    need = lib.iex_spmm_workspace_bytes(_lib.F32, _lib.I32, 9 << 16, c.m, c.k, 256, c.nnz, 1)
    assert need > 0 and need % (c.m * 256 * 4) == 0                    # whole fp32 copies of the output, one per slice
    rc = lib.iex_spmm_ex(_lib.F32, _lib.I32, 9 << 16, c.m, c.k, 256, c.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                         b.data_ptr(), None, out.data_ptr(), torch.cuda.current_stream(dev).cuda_stream, 1)
    assert rc == -1 and "workspace" in _lib.last_error()
    with pytest.raises(RuntimeError, match="k-split kernel needs"):
        pyops._spmm(b[:, :, :250].contiguous(), ri, v, ro, ci, c.m, force_variant=9, **KW)     # n % 4 != 0
