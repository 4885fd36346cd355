"""Shared checks of the parity tests."""
import numpy as np
import torch

# Tolerances of the path: fp32 within 1e-5 relative, fp16 / bf16 within 1e-2 relative, per
# element.  A pure relative test is meaningless for outputs that cancel towards zero, so
# the bound is  |got - want| <= rtol * |want| + rtol * FLOOR * scale  where scale is the
# element's condition scale sum_j |a_j| * |b_j| (FLOOR = 1e-2: an absolute slack of
# 1e-7 * scale for fp32, i.e. about one ulp of the largest partial sum).
RTOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2,
        np.dtype("float32"): 1e-5, np.dtype("float16"): 1e-2}
FLOOR = 1e-2


def assert_close(got, want, scale, rtol, what=""):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    scale = np.asarray(scale, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - want)
    bound = rtol * np.abs(want) + rtol * FLOOR * scale
    bad = err > bound
    if bad.any():
        idx = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {bad.size} elements out of tolerance (rtol={rtol}); worst at "
            f"{idx}: got {got[idx]!r} want {want[idx]!r} scale {scale[idx]!r}")
    # report the plain relative error on well-conditioned elements as well
    return float((err / np.maximum(np.abs(want), 1e-300))[np.abs(want) > 1e-3 * np.maximum(scale, 1e-300)].max(initial=0.0))


def to_dev(csr, dev, vdtype=torch.float32, idtype=torch.int32):
    """(row_indices, values, row_offsets, column_indices) tensors of a workloads.CSR."""
    return (torch.from_numpy(csr.row_indices).to(dev),
            torch.from_numpy(csr.values).to(dev).to(vdtype),
            torch.from_numpy(csr.row_offsets).to(dev),
            torch.from_numpy(csr.column_indices).to(dev).to(idtype))


def rounded(x, dtype):
    """numpy float32 copy of x after rounding to `dtype` (what the device kernel sees)."""
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(dtype).to(torch.float32).numpy()
