"""Horizontally fused sparse + dense launch: both results must be bit-identical to the
separate launches (the SpMM half embeds the row kernel, so that family is forced for the
comparison), for both workgroup-role layouts."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from _util import to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops


def _row_kernel_spmm(x, ri, v, ro, ci, m):
    from intrasm_engine_amd.pytorch import ops as pyops
    return pyops._spmm(x, ri, v, ro, ci, m, per_batch_values=False, accumulate=False, dtypes=(torch.float16,),
                       allow_i16=True, force_variant=1)


@pytest.mark.parametrize("interleave", [0, 1, 4, 7, -1])
@pytest.mark.parametrize("gdtype,trans_b", [(torch.bfloat16, False), (torch.float16, True)])
@pytest.mark.parametrize("n,idtype", [(512, torch.int16), (64, torch.int32), (200, torch.int32)])
def test_fused_equals_separate_launches(dev, interleave, gdtype, trans_b, n, idtype):
    rng = np.random.default_rng(n)
    a = W.config2_matrix(0.90, m=700, k=512)
    ri, v, ro, ci = to_dev(a, dev, torch.float16, idtype)
    x = torch.from_numpy(rng.standard_normal((1, 512, n)).astype(np.float32)).to(dev).half()
    M, N, K = 300, 264, 136
    ga = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dev).to(gdtype)
    gb = torch.from_numpy(rng.standard_normal((N, K) if trans_b else (K, N)).astype(np.float32)).to(dev).to(gdtype)
    out, c = ops.fused_spmm_gemm(x, ri, v, ro, ci, a.m, ga, gb, trans_b, interleave)
    assert torch.equal(out, _row_kernel_spmm(x, ri, v, ro, ci, a.m))
    assert torch.equal(c, ops.gemm_mfma(ga, gb, trans_b))


def test_fused_config4_shape(dev):
    """At this shape the stand-alone SpMM runs on the 8-wave matrix-core kernel, and so does the
    sparse role of the fused launch (512-thread workgroups beside 128 x 256 GEMM tiles): both
    outputs stay bit-identical to the separate launches, for both layouts of B and both
    workgroup-role layouts."""
    w, x, ga, gb = W.config4()
    ri, v, ro, ci = to_dev(w, dev, torch.float16, torch.int16)
    xt = torch.from_numpy(x).to(dev).half()
    gat, gbt = torch.from_numpy(ga).to(dev).bfloat16(), torch.from_numpy(gb).to(dev).bfloat16()
    alone = ops.spmm_sputnik_reuse_weight_half(xt, ri, v, ro, ci, w.m)
    assert not torch.equal(alone, _row_kernel_spmm(xt, ri, v, ro, ci, w.m))     # i.e. not the row kernel
    c_alone = ops.gemm_mfma(gat, gbt, False)
    for interleave in (1, 0, 16, 5, 37, -1):
        out, c = ops.fused_spmm_gemm(xt, ri, v, ro, ci, w.m, gat, gbt, False, interleave)
        assert torch.equal(out, alone) and torch.equal(c, c_alone), interleave
    gbt_t = gbt.t().contiguous()
    out, c = ops.fused_spmm_gemm(xt, ri, v, ro, ci, w.m, gat, gbt_t, True, 0)
    assert torch.equal(out, alone) and torch.equal(c, ops.gemm_mfma(gat, gbt_t, True))


def test_fused_timeline_records_every_workgroup_and_changes_no_result(dev):
    """The diagnostic timeline (iex_fused_timeline): one record per workgroup (both clocks set, end after begin, every
    GEMM tile and every SpMM tile exactly once), the outputs are those of a launch without it, and it is off again after
    iex_fused_timeline(NULL)."""
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    w, x, ga, gb = W.config4()
    ri, v, ro, ci = to_dev(w, dev, torch.float16, torch.int16)
    xt = torch.from_numpy(x).to(dev).half()
    gat, gbt = torch.from_numpy(ga).to(dev).bfloat16(), torch.from_numpy(gb).to(dev).bfloat16()
    out0, c0 = ops.fused_spmm_gemm(xt, ri, v, ro, ci, w.m, gat, gbt, False, -1)
    groups = 344 + 256                                   # 128 x 512 SpMM tiles of 11008 x 2048, 128 x 256 GEMM tiles of 4096 x 2048
    buf = torch.zeros(4 * (groups + 8), dtype=torch.int64, device=dev)
    assert lib.iex_fused_timeline(buf.data_ptr()) == 0
    try:
        out1, c1 = ops.fused_spmm_gemm(xt, ri, v, ro, ci, w.m, gat, gbt, False, -1)
        torch.cuda.synchronize()
    finally:
        assert lib.iex_fused_timeline(None) == 0
    assert torch.equal(out0, out1) and torch.equal(c0, c1)
    t = buf.cpu().numpy().reshape(-1, 4)
    assert (t[groups:] == 0).all()
    t = t[:groups]
    assert (t[:, 0] > 0).all() and (t[:, 1] > t[:, 0]).all()
    is_gemm, index = (t[:, 3] >> 32) != 0, t[:, 3] & 0xffffffff
    assert not is_gemm[:344].any() and is_gemm[344:].all()           # SpMM tiles first
    assert sorted(index[~is_gemm]) == list(range(344)) and sorted(index[is_gemm]) == list(range(256))
    assert 1 < len(set(int(p) >> 8 for p in t[:, 2])) <= 256         # (XCD and CU: bits 8 and up of the place word)
    buf.zero_()
    out2, _ = ops.fused_spmm_gemm(xt, ri, v, ro, ci, w.m, gat, gbt, False, -1)
    torch.cuda.synchronize()
    assert torch.equal(out2, out0) and not buf.any()


def test_fused_matrix_core_batched_gemm(dev):
    """Matrix-core fused launch with a batched, ragged GEMM (the attention products of the
    decoder layer ride along like this) and int32 column indices."""
    rng = np.random.default_rng(9)
    a = W.pruned_weight(77, 2048, 640, 0.8)
    ri, v, ro, ci = to_dev(a, dev, torch.float16, torch.int32)
    x = torch.from_numpy(rng.standard_normal((1, 640, 4096)).astype(np.float32)).to(dev).half()
    q = torch.from_numpy(rng.standard_normal((6, 200, 72)).astype(np.float32)).to(dev).half()
    kmat = torch.from_numpy(rng.standard_normal((6, 136, 72)).astype(np.float32)).to(dev).half()
    out, c = ops.fused_spmm_gemm(x, ri, v, ro, ci, a.m, q, kmat, True, 0)
    assert torch.equal(out, ops.spmm_sputnik_reuse_weight_half(x, ri, v, ro, ci, a.m))
    assert torch.equal(c, ops.gemm_mfma(q, kmat, True))


def test_argument_checks(dev):
    a = W.config2_matrix(0.90, m=64, k=64)
    ri, v, ro, ci = to_dev(a, dev, torch.float16)
    x = torch.randn(1, 64, 64, device=dev).half()
    g = torch.randn(64, 64, device=dev).half()
    with pytest.raises(RuntimeError, match="fp16"):
        ops.fused_spmm_gemm(x.float(), ri, v.float(), ro, ci, a.m, g, g, False, 0)
    with pytest.raises(RuntimeError, match="one batch entry"):
        ops.fused_spmm_gemm(x.repeat(2, 1, 1), ri, v, ro, ci, a.m, g, g, False, 0)
