"""The SDDMM kernel for attention-like masks (variant 3: score tiles of the dense blocks on the matrix cores,
sampled inside the workgroup; the nonzeros of thin blocks one dot product at a time): parity with the CPU oracle on
ragged shapes and on config 3, forced and where the library picks it, with every block treated as dense, every
block as thin, and with the built-in threshold."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from _util import FP16_SUBNORMAL_HALF_STEP, RTOL, assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops


def _run(dev, csr, lhs, rhs, dtype, **force):
    from intrasm_engine_amd.pytorch import ops as pyops
    ri, _, ro, ci = to_dev(csr, dev)
    lt, rt = torch.from_numpy(lhs).to(dev).to(dtype), torch.from_numpy(rhs).to(dev).to(dtype)
    return pyops._sddmm(lt, rt, ri, ro, ci, sum_over_batch=False, dtypes=(dtype,), **force)


def _want(oracle, csr, lhs, rhs, dtype):
    l16, r16 = rounded(lhs, dtype), rounded(rhs, dtype)
    want = oracle.sddmm(l16, r16, csr.row_indices, csr.row_offsets, csr.column_indices, sum_over_batch=False)
    scale = oracle.sddmm_abs_scale(l16, r16, csr.row_indices, csr.row_offsets, csr.column_indices, sum_over_batch=False)
    return want, scale


@pytest.mark.parametrize("k", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,n", [(131, 97), (300, 517), (128, 128)])
@pytest.mark.parametrize("blocks", [0, 1, 255, 2])      # threshold: built-in, all dense, all thin, 128 nonzeros
def test_ragged_shapes_forced(oracle, dev, k, dtype, m, n, blocks):
    """m and n that are no multiples of the 128 x 128 tile, empty rows, a completely dense row (more than 64
    nonzeros in one tile: both sampling steps), rows of 1 to 4 nonzeros per tile (the row's own lane) and of 5 and
    more (the wavefront), two batch entries."""
    rng = np.random.default_rng(k + m)
    lens = rng.integers(0, min(n, 40), m)
    lens[[0, 9, m - 1]] = 0
    lens[5] = n
    lens[6] = min(n, 70)
    ro, ci = W.csr_from_row_lengths(rng, m, n, lens)
    csr = W.CSR(m, n, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    lhs = rng.standard_normal((2, m, k)).astype(np.float32)
    rhs = rng.standard_normal((2, n, k)).astype(np.float32)
    out = _run(dev, csr, lhs, rhs, dtype, force_variant=3, force_wpr=blocks)
    want, scale = _want(oracle, csr, lhs, rhs, dtype)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"matrix-core SDDMM {m}x{n} k={k} {dtype} blocks={blocks}",
                 atol=FP16_SUBNORMAL_HALF_STEP if dtype == torch.float16 else 0.0)
    assert torch.equal(out, _run(dev, csr, lhs, rhs, dtype, force_variant=3, force_wpr=blocks))         # same call, same bits


def test_integer_operands_agree_with_the_gather_kernel_exactly(dev):
    rng = np.random.default_rng(8)
    m, n, k = 260, 390, 64
    lens = rng.integers(0, 200, m)
    ro, ci = W.csr_from_row_lengths(rng, m, n, lens)
    csr = W.CSR(m, n, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    lhs = rng.integers(-3, 4, (3, m, k)).astype(np.float32)
    rhs = rng.integers(-3, 4, (3, n, k)).astype(np.float32)
    want = _run(dev, csr, lhs, rhs, torch.float16, force_variant=1)
    for blocks in (0, 1, 255, 3):
        assert torch.equal(_run(dev, csr, lhs, rhs, torch.float16, force_variant=3, force_wpr=blocks), want), blocks


def test_band_plus_scattered_mask_mixes_both_kinds_of_block(oracle, dev):
    """A 640 x 1100 mask with a band of 96 columns and 3 scattered entries per row: band blocks go to the matrix
    cores, the others are sampled entry by entry, within one workgroup; bf16 and fp16, three batch entries."""
    rng = np.random.default_rng(77)
    m, n, k = 640, 1100, 64
    idx = np.arange(m)
    mask = np.abs(idx[:, None] * n // m - np.arange(n)[None, :]) < 48
    mask[np.repeat(idx, 3), rng.integers(0, n, (m, 3)).ravel()] = True
    ro, ci, _ = W.csr_from_mask(mask)
    csr = W.CSR(m, n, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    lhs = rng.standard_normal((3, m, k)).astype(np.float32)
    rhs = rng.standard_normal((3, n, k)).astype(np.float32)
    for dtype in (torch.float16, torch.bfloat16):
        out = _run(dev, csr, lhs, rhs, dtype, force_variant=3)
        want, scale = _want(oracle, csr, lhs, rhs, dtype)
        assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"band + scattered {dtype}",
                     atol=FP16_SUBNORMAL_HALF_STEP if dtype == torch.float16 else 0.0)


def test_config3_four_heads_against_the_oracle_and_sixteen_against_the_gather_kernel(oracle, dev):
    from intrasm_engine_amd import _lib
    pattern, q, k, _ = W.config3(heads=4)
    out = _run(dev, pattern, q, k, torch.float16, force_variant=3)
    want, scale = _want(oracle, pattern, q, k, torch.float16)
    assert_close(out.float().cpu().numpy(), want, scale, 1e-2, "config 3, 4 heads, matrix cores", atol=FP16_SUBNORMAL_HALF_STEP)
    # all 16 heads: what the operator picks by itself for this shape is this kernel, each head equals the head alone,
    # and the gather kernel agrees to the tolerance
    pattern, q, k, _ = W.config3()
    ri, _, ro, ci = to_dev(pattern, dev)
    qt, kt = torch.from_numpy(q).to(dev).half(), torch.from_numpy(k).to(dev).half()
    auto = ops.sddmm_sputnik_half(qt, kt, ri, ro, ci)
    assert "sddmm_mfma_kernel" in _lib.last_kernels()
    assert torch.equal(auto, _run(dev, pattern, q, k, torch.float16, force_variant=3))
    for h in (0, 15):           # (a single head alone is too little work for this kernel to be picked: forced)
        alone = _run(dev, pattern, q[h:h + 1], k[h:h + 1], torch.float16, force_variant=3)
        assert torch.equal(alone[0], auto[h])
    gather = _run(dev, pattern, q, k, torch.float16, force_variant=1).float()
    assert torch.allclose(auto.float(), gather, rtol=1e-2, atol=1e-2 * 8.0 * 0.1)


@pytest.mark.parametrize("n", [9000, 20100, 65536])
@pytest.mark.parametrize("blocks", [0, 1, 255])
def test_many_column_blocks(oracle, dev, n, blocks):
    """More than 64 (and more than 128) blocks of 128 columns per row: the setup kernel, the workgroup's list of dense
    and thin blocks and the runs of thin blocks between dense ones all work in pieces of 64 blocks.  A band that
    wanders through the columns plus scattered entries, 260 rows, two batch entries; n = 65536 is the largest the
    kernel takes (one more column is refused)."""
    rng = np.random.default_rng(n)
    m, k = 260, 64
    idx = np.arange(m)
    centre = (idx * (n - 200) // m) + 100
    cols = [np.unique(np.concatenate([np.arange(c - 40, c + 40), rng.integers(0, n, 12)])) for c in centre]
    cols[7] = np.array([], dtype=np.int64)
    cols[100] = np.arange(0, n, 97)                       # a long row that touches every block
    lens = np.array([len(c) for c in cols])
    ro = np.zeros(m + 1, dtype=np.int32)
    np.cumsum(lens, out=ro[1:])
    ci = np.concatenate(cols).astype(np.int32)
    csr = W.CSR(m, n, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    lhs = rng.standard_normal((2, m, k)).astype(np.float32)
    rhs = rng.standard_normal((2, n, k)).astype(np.float32)
    out = _run(dev, csr, lhs, rhs, torch.float16, force_variant=3, force_wpr=blocks)
    want, scale = _want(oracle, csr, lhs, rhs, torch.float16)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[torch.float16], f"n={n} blocks={blocks}", atol=FP16_SUBNORMAL_HALF_STEP)
    if n == 65536 and blocks == 0:
        with pytest.raises(RuntimeError, match="matrix-core kernel needs"):
            _run(dev, csr, lhs, np.concatenate([rhs, rhs[:, :1]], axis=1), torch.float16, force_variant=3)


def test_tables_kept_between_calls_of_one_mask(oracle, dev):
    """A caller with a fixed mask keeps a plan: the second call skips the setup kernel and gives the same bits; another
    mask (or the same index tensor changed in place) makes the plan write the tables again; the attention block takes
    a plan too."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    from intrasm_engine_amd.pytorch.sparse_attention import sparse_attention
    pattern, q, k, v = W.config3(heads=8)
    ri, _, ro, ci = to_dev(pattern, dev)
    qt, kt, vt = (torch.from_numpy(x).to(dev).half() for x in (q, k, v))
    # (the operator itself keeps the tables of a pattern it has looked at: no setup kernel in its calls either)
    want = ops.sddmm_sputnik_half(qt, kt, ri, ro, ci)
    assert _lib.last_kernels().startswith("sddmm_mfma_kernel")
    plan = pyops.SddmmPlan()
    first = pyops.sddmm_half_planned(qt, kt, ri, ro, ci, plan)
    assert "sddmm_tile_ptr_kernel" in _lib.last_kernels() and torch.equal(first, want)
    second = pyops.sddmm_half_planned(qt, kt, ri, ro, ci, plan)
    assert _lib.last_kernels().startswith("sddmm_mfma_kernel") and torch.equal(second, want)
    # other operands, same mask: still no setup
    third = pyops.sddmm_half_planned(kt, qt, ri, ro, ci, plan)
    assert _lib.last_kernels().startswith("sddmm_mfma_kernel") and torch.equal(third, ops.sddmm_sputnik_half(kt, qt, ri, ro, ci))
    # another mask through the same plan: tables written again, results those of the new mask
    p2, *_ = W.config3(seed=11, heads=1, band=128, extra=16)
    ri2, _, ro2, ci2 = to_dev(p2, dev)
    other = pyops.sddmm_half_planned(qt, kt, ri2, ro2, ci2, plan)
    assert "sddmm_tile_ptr_kernel" in _lib.last_kernels()
    assert torch.equal(other, ops.sddmm_sputnik_half(qt, kt, ri2, ro2, ci2))
    # the first mask again, then changed in place (one scattered column moved): noticed through the version counter
    assert torch.equal(pyops.sddmm_half_planned(qt, kt, ri, ro, ci, plan), want)
    ci.add_(0)
    pyops.sddmm_half_planned(qt, kt, ri, ro, ci, plan)
    assert "sddmm_tile_ptr_kernel" in _lib.last_kernels()
    # the attention block
    plan2 = pyops.SddmmPlan()
    a0 = sparse_attention(qt, kt, vt, ri, ro, ci)
    a1 = sparse_attention(qt, kt, vt, ri, ro, ci, plan=plan2)
    a2 = sparse_attention(qt, kt, vt, ri, ro, ci, plan=plan2)
    assert torch.equal(a0, a1) and torch.equal(a0, a2)


def test_structure_settles_the_kernel(dev):
    """Two masks of the same density: a band (its nonzeros sit in dense 128 x 128 blocks) and columns at random.  The
    library's own rule, asked through the C interface with nothing known about the pattern, goes by density and names
    the kernel for masks with structure for both.  The operator has looked at the pattern (the share of its nonzeros
    in dense blocks is part of that look) and takes that kernel for the band and the gather kernel for the random one;
    so does a plan.  Same results either way, and the band's tables are made once: later calls run no setup kernel."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    lib = _lib.load()
    rng = np.random.default_rng(5)
    tokens, heads = 2048, 16
    q = rng.standard_normal((heads, tokens, 64)).astype(np.float32)
    k = rng.standard_normal((heads, tokens, 64)).astype(np.float32)
    qt, kt = torch.from_numpy(q).to(dev).half(), torch.from_numpy(k).to(dev).half()
    band, *_ = W.config3(tokens=tokens, heads=1, band=160, extra=4)
    per_row = band.nnz // tokens
    ro, ci = W.csr_from_row_lengths(rng, tokens, tokens, np.full(tokens, per_row))
    rand = W.CSR(tokens, tokens, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    for csr, variant, kernel in ((band, 3, "sddmm_mfma_kernel"), (rand, 1, "sddmm_kernel")):
        assert lib.iex_sddmm_workspace_kind(_lib.F16, 0, tokens, 64, tokens, csr.nnz, heads) == 3
        ri, _, ro_t, ci_t = to_dev(csr, dev)
        share = pyops._known_dense_share(ro_t, ci_t, tokens)
        assert (share >= 0.5) == (variant == 3), share
        forced = pyops._sddmm(qt, kt, ri, ro_t, ci_t, sum_over_batch=False, dtypes=(torch.float16,), force_variant=3)
        assert "sddmm_mfma_kernel" in _lib.last_kernels()
        auto = ops.sddmm_sputnik_half(qt, kt, ri, ro_t, ci_t)
        assert kernel in _lib.last_kernels()
        assert torch.allclose(forced.float(), auto.float(), rtol=1e-2, atol=1e-2 * 8.0 * 0.1)
        if variant == 3:
            assert torch.equal(forced, auto)
            again = ops.sddmm_sputnik_half(qt, kt, ri, ro_t, ci_t)
            assert _lib.last_kernels().startswith("sddmm_mfma_kernel") and torch.equal(again, auto)
        plan = pyops.SddmmPlan()
        assert plan.analyze(ro_t, ci_t, tokens) == variant, plan.dense_share
        assert abs(plan.dense_share - share) < 1e-6
        planned = pyops.sddmm_half_planned(qt, kt, ri, ro_t, ci_t, plan)
        assert kernel in _lib.last_kernels()
        assert torch.equal(planned, auto)
        # fp32 operands through the same plan: the planned kernel does not serve them, the call runs all the same
        f32 = pyops.sddmm_half_planned(qt.float(), kt.float(), ri, ro_t, ci_t, plan)
        assert torch.allclose(f32, auto.float(), rtol=1e-2, atol=1e-2 * 8.0 * 0.1)


@pytest.mark.parametrize("idtype", [torch.int32, torch.int16])
def test_dense_share_kernel_counts_like_numpy(dev, idtype):
    """iex_csr_dense_share against a numpy count, for several thresholds, on a band with scattered entries, a random
    mask, a ragged shape (m and k no multiples of 128) and an empty pattern."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    lib = _lib.load()
    rng = np.random.default_rng(3)
    band, *_ = W.config3(tokens=1024, heads=1, band=96, extra=6)
    ro, ci = W.csr_from_row_lengths(rng, 700, 1000, rng.integers(0, 300, 700))
    ragged = W.CSR(700, 1000, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    for csr in (band, ragged):
        rows = np.repeat(np.arange(csr.m), np.diff(csr.row_offsets))
        tiles_n = (csr.k + 127) // 128
        counts = np.bincount((rows // 128) * tiles_n + csr.column_indices // 128, minlength=((csr.m + 127) // 128) * tiles_n)
        ro_t = torch.from_numpy(csr.row_offsets).to(dev)
        ci_t = torch.from_numpy(csr.column_indices).to(dev).to(idtype)
        for dense_min in (1, 1536, 2048, 5000, 16384, 16385):
            want = counts[counts >= dense_min].sum() / csr.nnz
            assert abs(pyops._dense_share_host(ro_t, ci_t, csr.k, dense_min) - want) < 1e-9, dense_min
            # the entry point itself: one workgroup per block of rows (no scratch memory, or too little), several (zeroed scratch)
            need = lib.iex_csr_dense_share_scratch_bytes(csr.m, csr.k)
            assert need == ((csr.m + 127) // 128) * (tiles_n + 1) * 4
            for scratch in (None, torch.zeros(need - 4, dtype=torch.uint8, device=dev), torch.zeros(need, dtype=torch.uint8, device=dev)):
                got = torch.zeros(1, dtype=torch.int32, device=dev)
                rc = lib.iex_csr_dense_share(1 if idtype == torch.int16 else 0, csr.m, csr.k, csr.nnz, ro_t.data_ptr(), ci_t.data_ptr(), dense_min,
                                             got.data_ptr(), scratch.data_ptr() if scratch is not None else None,
                                             scratch.numel() if scratch is not None else 0, torch.cuda.current_stream().cuda_stream)
                assert rc == 0, _lib.last_error()
                assert int(got.item()) == int(counts[counts >= dense_min].sum()), (dense_min, None if scratch is None else scratch.numel())
    assert lib.iex_csr_dense_share_scratch_bytes(128 * 512, 4096) == 0   # 512 blocks of rows fill the chip by themselves
    empty = torch.zeros(65, dtype=torch.int32, device=dev)
    assert pyops._dense_share_host(empty, torch.zeros(0, dtype=idtype, device=dev), 64) is None


def test_refusals(dev):
    from intrasm_engine_amd import _lib
    rng = np.random.default_rng(1)
    ro, ci = W.csr_from_row_lengths(rng, 64, 64, np.full(64, 8))
    csr = W.CSR(64, 64, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    with pytest.raises(RuntimeError, match="k = 32, 64 or 128"):
        _run(dev, csr, rng.standard_normal((1, 64, 48)).astype(np.float32), rng.standard_normal((1, 64, 48)).astype(np.float32),
             torch.float16, force_variant=3)
    lib = _lib.load()
    assert lib.iex_sddmm_workspace_bytes(_lib.F16, 3 << 16, 4096, 64, 4096, 1000, 16) == ((6 * 32 + 1) * 4096 + 64 + 2 * 1000 + 4096 + 32 * (32 + 2) // 2) * 4   # tables + lists
    assert lib.iex_sddmm_workspace_bytes(_lib.F32, 3 << 16, 4096, 64, 4096, 1000, 16) == 0
    assert lib.iex_sddmm_workspace_kind(_lib.F16, 3 << 16, 4096, 64, 4096, 1000, 16) == 3
    assert lib.iex_sddmm_workspace_kind(_lib.F16, 0, 4096, 64, 4096, 1150000, 16) == 3
    assert lib.iex_sddmm_workspace_kind(_lib.F16, 0, 1024, 4096, 1024, 300000, 1) == 7
    assert lib.iex_sddmm_workspace_kind(_lib.F32, 0, 4096, 64, 4096, 1150000, 16) == 0


def test_plan_keeps_the_index_tensors_of_its_tables_alive(dev):
    """The plan names a pattern by the addresses and versions of its index tensors.  If the caller drops them, the
    allocator may hand the same addresses to another pattern of the same size: the plan holds the tensors, so that
    cannot happen, and the other pattern gets tables of its own."""
    import gc
    from intrasm_engine_amd.pytorch import ops as pyops
    m = 512
    idx = np.arange(m)

    def pattern(shift):
        mask = np.abs(idx[:, None] - ((idx[None, :] + shift) % m)) < 40
        ro, ci, _ = W.csr_from_mask(mask)
        return W.CSR(m, m, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)

    first, second = pattern(0), pattern(100)
    assert first.nnz == second.nnz                                   # same sizes: the allocator would reuse the blocks
    q = torch.randn(2, m, 64, device=dev).half()
    k = torch.randn(2, m, 64, device=dev).half()
    plan = pyops.SddmmPlan()
    plan.variant = 3
    ri, _, ro, ci = to_dev(first, dev)
    pyops.sddmm_half_planned(q, k, ri, ro, ci, plan)
    addresses = (ro.data_ptr(), ci.data_ptr())
    del ro, ci
    gc.collect()
    ri2, _, ro2, ci2 = to_dev(second, dev)
    assert (ro2.data_ptr(), ci2.data_ptr()) != addresses             # the plan still holds the first pattern's tensors
    got = pyops.sddmm_half_planned(q, k, ri2, ro2, ci2, plan)
    want = pyops._sddmm(q, k, ri2, ro2, ci2, sum_over_batch=False, dtypes=(torch.float16,), force_variant=3)
    assert torch.equal(got, want)
