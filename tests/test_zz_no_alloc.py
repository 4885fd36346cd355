"""iex_spmm_static, the SpMM entry point that allocates nothing (its workspace is an array the library holds on
the GPU), called through the C ABI: its output must equal, bit for bit, what iex_spmm_ws writes with a
caller-owned workspace -- on two calls in a row that share the library's array, the second with a smaller
input -- and what the oracle computes, to the fp16 tolerance.  Sizes beyond the array are refused."""
import ctypes

import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from _util import assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu


def _call(lib, fn, dev, a, x, idtype, ws=None, flags=0):
    from intrasm_engine_amd import _lib
    ri, v, ro, ci = to_dev(a, dev, torch.float16, idtype)
    out = torch.full((x.shape[0], a.m, x.shape[2]), float("nan"), dtype=torch.float16, device=dev)
    it = _lib.I16 if idtype == torch.int16 else _lib.I32
    stream = torch.cuda.current_stream(dev).cuda_stream
    args = [_lib.F16, it, flags, a.m, a.k, x.shape[2], a.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
            x.data_ptr(), None, out.data_ptr(), stream, x.shape[0]]
    if ws is not None:
        args += [ws.data_ptr(), ws.numel()]
    _lib.check(fn(*args), fn.__name__)
    torch.cuda.synchronize()
    return out


def test_static_scratch_equals_caller_workspace_two_calls_in_a_row(dev, oracle):
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    assert lib.iex_spmm_static_scratch_bytes() == 96 << 20
    rng = np.random.default_rng(3)
    cases = [(W.pruned_weight(41, 2048, 1024, 0.80), 1024, torch.int16),     # first call: 4 MB of dense form
             (W.pruned_weight(42, 512, 768, 0.50), 512, torch.int32)]        # second, smaller: 0.75 MB, same array
    for a, n, idtype in cases:
        x_np = rng.standard_normal((1, a.k, n)).astype(np.float32)
        x = torch.from_numpy(x_np).to(dev).half()
        need = lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16 if idtype == torch.int16 else _lib.I32, 0, a.m, a.k, n, a.nnz, 1)
        assert need == a.m * a.k * 2, "the case must be one that uses the workspace"
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
        want_ws = _call(lib, lib.iex_spmm_ws, dev, a, x, idtype, ws=ws)
        got = _call(lib, lib.iex_spmm_static, dev, a, x, idtype)
        assert torch.equal(got, want_ws)
        x16 = rounded(x_np, torch.float16)
        want = oracle.spmm(x16, a.row_indices, rounded(a.values, torch.float16), a.row_offsets, a.column_indices, a.m)
        scale = oracle.spmm_abs_scale(x16, a.row_indices, a.values, a.row_offsets, a.column_indices, a.m)
        assert_close(got.float().cpu().numpy(), want, scale, 1e-2, f"static scratch, {a.m}x{a.k}")


def test_static_scratch_serves_the_kernel_for_patterns_with_structure_between_other_uses(dev):
    """Family 10 keeps tables and lists in the workspace: from the library's array they are written by every call
    (no caller can vouch for what another call left there), also right after a dense-form call has used the same
    bytes.  Bit-equal to iex_spmm_ws with a workspace of the caller's."""
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(8)
    m = 640
    idx = np.arange(m)
    mask = np.abs(idx[:, None] - idx[None, :]) < 70
    mask[np.repeat(idx, 3), rng.integers(0, m, (m, 3)).ravel()] = True
    ro, ci, _ = W.csr_from_mask(mask)
    band = W.CSR(m, m, rng.standard_normal(ci.shape[0]).astype(np.float32), W.swizzle_from_offsets(ro), ro, ci)
    flags = _lib.SPMM_PER_BATCH_VALUES | (10 << 16)
    x = torch.randn(1, m, 64, device=dev).half()
    need = lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I32, flags, m, m, 64, band.nnz, 1)
    assert lib.iex_spmm_workspace_kind(_lib.F16, _lib.I32, flags, m, m, 64, band.nnz, 1) == 10 and 0 < need < (96 << 20)
    want = _call(lib, lib.iex_spmm_ws, dev, band, x, torch.int32, ws=torch.empty(need, dtype=torch.uint8, device=dev), flags=flags)
    assert "spmm_blocks_kernel" in _lib.last_kernels()
    first = _call(lib, lib.iex_spmm_static, dev, band, x, torch.int32, flags=flags)
    other = W.pruned_weight(43, 1024, 1024, 0.70)                             # a dense-form call overwrites the array
    _call(lib, lib.iex_spmm_static, dev, other, torch.randn(1, 1024, 1024, device=dev).half(), torch.int16)
    assert "csr_to_dense_kernel" in _lib.last_kernels()
    again = _call(lib, lib.iex_spmm_static, dev, band, x, torch.int32, flags=flags)
    assert _lib.last_kernels().split(" + ") == ["sddmm_tile_ptr_kernel", "sb_lists_kernel", "spmm_blocks_kernel<false>"]
    assert torch.equal(first, want) and torch.equal(again, want)
    # a caller cannot vouch for what another call left in the shared array: the READY flags are ignored here
    _call(lib, lib.iex_spmm_static, dev, other, torch.randn(1, 1024, 1024, device=dev).half(), torch.int16)
    vouched = _call(lib, lib.iex_spmm_static, dev, band, x, torch.int32, flags=flags | _lib.SPMM_TABLES_READY | _lib.SPMM_LISTS_READY)
    assert _lib.last_kernels().split(" + ") == ["sddmm_tile_ptr_kernel", "sb_lists_kernel", "spmm_blocks_kernel<false>"]
    assert torch.equal(vouched, want)


def test_static_scratch_without_workspace_use_runs_as_the_plain_entry_point(dev):
    """fp32 operands never use the workspace: the call must equal iex_spmm_ex bit for bit."""
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    a = W.config2_matrix(0.9, m=512, k=512)
    ri, v, ro, ci = to_dev(a, dev)
    x = torch.randn(1, 512, 128, device=dev)
    outs = []
    for fn in (lib.iex_spmm_ex, lib.iex_spmm_static):
        out = torch.empty(1, a.m, 128, device=dev)
        _lib.check(fn(_lib.F32, _lib.I32, 0, a.m, a.k, 128, a.nnz, ri.data_ptr(), v.data_ptr(), ro.data_ptr(), ci.data_ptr(),
                      x.data_ptr(), None, out.data_ptr(), torch.cuda.current_stream(dev).cuda_stream, 1))
        outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])


def test_static_scratch_refuses_what_does_not_fit(dev):
    """A forced dense-form call of 8192 x 8192 needs 128 MB: refused before any launch, with the limit in the text."""
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    flags = 7 << 16
    m = k = 8192
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I32, flags, m, k, 256, 1000, 1) == m * k * 2
    one = torch.zeros(16, dtype=torch.int32, device=dev)
    rc = lib.iex_spmm_static(_lib.F16, _lib.I32, flags, m, k, 256, 1000, one.data_ptr(), one.data_ptr(), one.data_ptr(),
                             one.data_ptr(), one.data_ptr(), None, one.data_ptr(), None, 1)
    assert rc == -3 and "100663296" in _lib.last_error() and "134217728" in _lib.last_error()
