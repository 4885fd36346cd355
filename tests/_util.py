"""Shared checks of the parity tests."""
import numpy as np
import torch

# Tolerances of the path: fp32 within 1e-5 relative, fp16 / bf16 within 1e-2 relative, per
# element.  A pure relative test is meaningless for outputs that cancel towards zero, so
# the bound is  |got - want| <= rtol * |want| + rtol * FLOOR * scale  where scale is the
# element's condition scale sum_j |a_j| * |b_j|.  FLOOR = 0.1 gives fp32 an absolute slack
# of 1e-6 * scale: fp32 accumulation of L terms carries a rounding error of about
# sqrt(L) * 6e-8 * scale (5e-7 .. 4e-6 for the row lengths used here), which no summation
# order can avoid; one ulp of the scale (1.2e-7) was observed to be too tight by 3 %.
RTOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2,
        np.dtype("float32"): 1e-5, np.dtype("float16"): 1e-2}
FLOOR = 0.1
# An fp16 output below 6.1e-5 is a subnormal with an absolute spacing of 2^-24: half of that
# is the rounding error of storing the result, whatever its relative size.
FP16_SUBNORMAL_HALF_STEP = 2.0 ** -25


def assert_close(got, want, scale, rtol, what="", atol=0.0):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    scale = np.asarray(scale, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + rtol * FLOOR * scale + atol
    bad = err > bound
    if bad.any():
        idx = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {bad.size} elements out of tolerance (rtol={rtol}); worst at "
            f"{idx}: got {got[idx]!r} want {want[idx]!r} scale {scale[idx]!r}")
    # report the plain relative error on well-conditioned elements as well
    return float((err / np.maximum(np.abs(want), 1e-300))[np.abs(want) > 1e-3 * np.maximum(scale, 1e-300)].max(initial=0.0))


def to_dev(csr, dev, vdtype=torch.float32, idtype=torch.int32, tables=True):
    """(row_indices, values, row_offsets, column_indices) tensors of a workloads.CSR.  The pattern is looked at here,
    once (``ops.prepare_pattern``), as set-up code does: operators that meet it under stream capture then know it
    (``tables`` = False: without making the tables that a pattern with structure keeps for its kernels)."""
    t = (torch.from_numpy(csr.row_indices).to(dev),
         torch.from_numpy(csr.values).to(dev).to(vdtype),
         torch.from_numpy(csr.row_offsets).to(dev),
         torch.from_numpy(csr.column_indices).to(dev).to(idtype))
    if t[3].is_cuda and csr.nnz > 0:
        from intrasm_engine_amd.pytorch import ops as pyops
        pyops.prepare_pattern(t[2], t[3], csr.k, tables=tables)
    return t


def rounded(x, dtype):
    """numpy float32 copy of x after rounding to `dtype` (what the device kernel sees)."""
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(dtype).to(torch.float32).numpy()
