"""The SpMM kernel for attention-like sparse operands (family 10: the dense 128 x 128 blocks of A laid out in LDS and
multiplied on the matrix cores, the nonzeros elsewhere gathered row by row): parity with the CPU oracle on ragged
shapes and on config 3's product with V, with every block treated as dense, every block as thin, and with the
built-in threshold; values per batch entry and shared; tables kept between calls and shared with the SDDMM."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from _util import FP16_SUBNORMAL_HALF_STEP, RTOL, assert_close, rounded, to_dev

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops


def _run(dev, csr, values, dense, dtype, **force):
    from intrasm_engine_amd.pytorch import ops as pyops
    ri, _, ro, ci = to_dev(csr, dev)
    vt, dt = torch.from_numpy(values).to(dev).to(dtype), torch.from_numpy(dense).to(dev).to(dtype)
    return pyops._spmm(dt, ri, vt, ro, ci, csr.m, per_batch_values=values.ndim == 2, accumulate=False, dtypes=(dtype,),
                       allow_i16=False, **force)


def _want(oracle, csr, values, dense, dtype):
    v16, d16 = rounded(values, dtype), rounded(dense, dtype)
    want = oracle.spmm(d16, csr.row_indices, v16, csr.row_offsets, csr.column_indices, csr.m)
    scale = oracle.spmm_abs_scale(d16, csr.row_indices, v16, csr.row_offsets, csr.column_indices, csr.m)
    return want, scale


def _pattern(rng, m, k, lens):
    ro, ci = W.csr_from_row_lengths(rng, m, k, lens)
    return W.CSR(m, k, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k", [(131, 97), (300, 517), (128, 128), (64, 1000)])
@pytest.mark.parametrize("blocks", [0, 1, 255, 2])      # threshold: built-in, all dense, all thin, 128 nonzeros
def test_ragged_shapes_forced(oracle, dev, dtype, m, k, blocks):
    """m and k that are no multiples of the 128 x 128 tile, empty rows, a completely dense row, rows of 1 to 4
    nonzeros per tile (the row's own lane) and of 5 and more (the wavefront), two batch entries with values of
    their own."""
    rng = np.random.default_rng(k + m)
    lens = rng.integers(0, min(k, 40), m)
    lens[[0, 9, m - 1]] = 0
    lens[5] = k
    lens[6] = min(k, 70)
    csr = _pattern(rng, m, k, lens)
    values = rng.standard_normal((2, csr.nnz)).astype(np.float32)
    dense = rng.standard_normal((2, k, 64)).astype(np.float32)
    out = _run(dev, csr, values, dense, dtype, force_variant=10, force_wpr=blocks)
    want, scale = _want(oracle, csr, values, dense, dtype)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"dense-blocks SpMM {m}x{k} {dtype} blocks={blocks}",
                 atol=FP16_SUBNORMAL_HALF_STEP if dtype == torch.float16 else 0.0)
    assert torch.equal(out, _run(dev, csr, values, dense, dtype, force_variant=10, force_wpr=blocks))   # same call, same bits


@pytest.mark.parametrize("last_row", [[3, 4, 5, 6, 7, 8], [1, 2, 9, 17, 18, 40, 41], [120, 121, 122, 123, 124, 125, 126, 127],
                                      [0, 1, 2, 3, 4, 5, 6, 7, 8]])
def test_rows_at_the_end_of_the_values(oracle, dev, last_row):
    """The kernel reads a long row's values 16 bytes at a time; the reads of the last rows are moved back so that none
    passes the end of the values: last rows of neighbouring columns, of scattered columns, of exactly 8 and of 9, with
    a few rows before them, every block on the matrix cores, two batch entries."""
    rng = np.random.default_rng(len(last_row))
    m, k = 40, 128
    mask = np.zeros((m, k), bool)
    for r in range(m - 3):
        mask[r, rng.choice(k, int(rng.integers(0, 12)), replace=False)] = True
    mask[m - 3, 5:11] = True
    mask[m - 2, [0, 64, 65, 66, 100, 127]] = True
    mask[m - 1, last_row] = True
    ro, ci, _ = W.csr_from_mask(mask)
    csr = W.CSR(m, k, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    values = rng.integers(-4, 5, (2, csr.nnz)).astype(np.float32)
    dense = rng.integers(-4, 5, (2, k, 64)).astype(np.float32)
    out = _run(dev, csr, values, dense, torch.float16, force_variant=10, force_wpr=1)
    want, _ = _want(oracle, csr, values, dense, torch.float16)
    assert np.array_equal(out.float().cpu().numpy(), want)          # small integers: exact


@pytest.mark.parametrize("k", [9000, 20100, 65536])
@pytest.mark.parametrize("blocks", [0, 2])
def test_many_column_blocks(oracle, dev, k, blocks):
    """More than 64 (and more than 128) blocks of 128 columns per row: the setup kernels and the kernel's walk over
    the dense blocks all work on lists of up to 512 blocks.  A band that wanders through the columns plus scattered
    entries, 260 rows, two batch entries; k = 65536 is the largest the kernel takes (one more column is refused)."""
    rng = np.random.default_rng(k)
    m = 260
    idx = np.arange(m)
    centre = (idx * (k - 200) // m) + 100
    cols = [np.unique(np.concatenate([np.arange(c - 40, c + 40), rng.integers(0, k, 12)])) for c in centre]
    cols[7] = np.array([], dtype=np.int64)
    cols[100] = np.arange(0, k, 97)                       # a long row that touches every block
    lens = np.array([len(c) for c in cols])
    ro = np.zeros(m + 1, dtype=np.int32)
    np.cumsum(lens, out=ro[1:])
    ci = np.concatenate(cols).astype(np.int32)
    csr = W.CSR(m, k, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    values = rng.standard_normal((2, csr.nnz)).astype(np.float32)
    dense = rng.standard_normal((2, k, 64)).astype(np.float32)
    out = _run(dev, csr, values, dense, torch.float16, force_variant=10, force_wpr=blocks)
    want, scale = _want(oracle, csr, values, dense, torch.float16)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[torch.float16], f"k={k} blocks={blocks}", atol=FP16_SUBNORMAL_HALF_STEP)
    if k == 65536 and blocks == 0:
        with pytest.raises(RuntimeError, match="dense-blocks kernel needs fp16"):
            wide = W.CSR(m, k + 1, csr.values, csr.row_indices, csr.row_offsets, csr.column_indices)
            _run(dev, wide, values, rng.standard_normal((2, k + 1, 64)).astype(np.float32), torch.float16, force_variant=10)


@pytest.mark.parametrize("n", [128, 192])
def test_wider_outputs_in_slices_of_64_columns(oracle, dev, n):
    rng = np.random.default_rng(n)
    m, k = 300, 517
    lens = rng.integers(0, 60, m)
    lens[5] = k
    csr = _pattern(rng, m, k, lens)
    values = rng.standard_normal((3, csr.nnz)).astype(np.float32)
    dense = rng.standard_normal((3, k, n)).astype(np.float32)
    for blocks in (0, 1):
        out = _run(dev, csr, values, dense, torch.bfloat16, force_variant=10, force_wpr=blocks)
        want, scale = _want(oracle, csr, values, dense, torch.bfloat16)
        assert_close(out.float().cpu().numpy(), want, scale, RTOL[torch.bfloat16], f"n={n} blocks={blocks}")


@pytest.mark.parametrize("blocks", [0, 2, 255])
def test_fewer_than_eight_nonzeros_go_to_the_row_kernel(oracle, dev, blocks):
    """The kernel reads values eight at a time; a product with fewer nonzeros than that is handed to the row kernel,
    whatever threshold for dense blocks came with the request."""
    rng = np.random.default_rng(blocks)
    mask = np.zeros((70, 90), bool)
    mask[[3, 3, 40, 69, 69], [0, 89, 17, 5, 6]] = True
    ro, ci, _ = W.csr_from_mask(mask)
    csr = W.CSR(70, 90, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    values = rng.standard_normal((2, csr.nnz)).astype(np.float32)
    dense = rng.standard_normal((2, 90, 64)).astype(np.float32)
    out = _run(dev, csr, values, dense, torch.float16, force_variant=10, force_wpr=blocks)
    want, scale = _want(oracle, csr, values, dense, torch.float16)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[torch.float16], f"5 nonzeros, blocks={blocks}", atol=FP16_SUBNORMAL_HALF_STEP)


def test_integer_operands_agree_with_the_row_kernel_exactly(dev):
    rng = np.random.default_rng(8)
    m, k = 260, 390
    csr = _pattern(rng, m, k, rng.integers(0, 200, m))
    values = rng.integers(-3, 4, (3, csr.nnz)).astype(np.float32)
    dense = rng.integers(-3, 4, (3, k, 64)).astype(np.float32)
    want = _run(dev, csr, values, dense, torch.float16, force_variant=1)
    for blocks in (0, 1, 255, 3):
        assert torch.equal(_run(dev, csr, values, dense, torch.float16, force_variant=10, force_wpr=blocks), want), blocks
    shared = values[0]
    want = _run(dev, csr, shared, dense, torch.float16, force_variant=1)
    assert torch.equal(_run(dev, csr, shared, dense, torch.float16, force_variant=10), want)


def test_band_plus_scattered_mask_mixes_both_kinds_of_block(oracle, dev):
    rng = np.random.default_rng(77)
    m, k = 640, 1100
    idx = np.arange(m)
    mask = np.abs(idx[:, None] * k // m - np.arange(k)[None, :]) < 48
    mask[np.repeat(idx, 3), rng.integers(0, k, (m, 3)).ravel()] = True
    ro, ci, _ = W.csr_from_mask(mask)
    csr = W.CSR(m, k, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    values = rng.standard_normal((3, csr.nnz)).astype(np.float32)
    dense = rng.standard_normal((3, k, 64)).astype(np.float32)
    for dtype in (torch.float16, torch.bfloat16):
        out = _run(dev, csr, values, dense, dtype, force_variant=10)
        want, scale = _want(oracle, csr, values, dense, dtype)
        assert_close(out.float().cpu().numpy(), want, scale, RTOL[dtype], f"band + scattered {dtype}",
                     atol=FP16_SUBNORMAL_HALF_STEP if dtype == torch.float16 else 0.0)


def test_config3_probabilities_times_v(oracle, dev):
    """Config 3's second product at full size: 4 heads against the oracle, 16 heads against the row kernel head by
    head (same fp32 sums up to their order: compared at the 16-bit tolerance)."""
    pat, _, _, v = W.config3()
    rng = np.random.default_rng(3)
    probs = (rng.random((16, pat.nnz)) / 280.0).astype(np.float32)
    out = _run(dev, pat, probs[:4], v[:4], torch.float16, force_variant=10)
    want, scale = _want(oracle, pat, probs[:4], v[:4], torch.float16)
    assert_close(out.float().cpu().numpy(), want, scale, RTOL[torch.float16], "config 3, 4 heads", atol=FP16_SUBNORMAL_HALF_STEP)
    full = _run(dev, pat, probs, v, torch.float16, force_variant=10)
    assert torch.equal(full[:4], out)
    rows = _run(dev, pat, probs, v, torch.float16, force_variant=1)
    assert torch.allclose(full.float(), rows.float(), rtol=1e-2, atol=2e-3)


def test_tables_kept_between_calls_and_shared_with_the_sddmm(dev):
    """One plan serves the SDDMM for masks with structure and this kernel on the same pattern: whichever runs first
    writes the tables and lists, the other finds them; another threshold for dense blocks makes the lists, another
    pattern makes everything be written again."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(5)
    m = 512
    idx = np.arange(m)
    mask = np.abs(idx[:, None] - idx[None, :]) < 40
    mask[np.repeat(idx, 2), rng.integers(0, m, (m, 2)).ravel()] = True
    ro, ci, _ = W.csr_from_mask(mask)
    csr = W.CSR(m, m, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    ri, _, rot, cit = to_dev(csr, dev)
    q = torch.randn(2, m, 64, device=dev, dtype=torch.float16)
    kk = torch.randn(2, m, 64, device=dev, dtype=torch.float16)
    v = torch.randn(2, m, 64, device=dev, dtype=torch.float16)
    plan = pyops.SddmmPlan()
    plan.variant = 3
    scores = pyops.sddmm_half_planned(q, kk, ri, rot, cit, plan)
    assert plan.key is not None
    kw = dict(per_batch_values=True, accumulate=False, dtypes=(torch.float16,), allow_i16=False, force_variant=10)
    fresh = pyops._spmm(v, ri, scores, rot.clone(), cit.clone(), m, **kw)    # (copies: nothing kept with them, the call sets up its own tables)
    assert _lib.last_kernels().split(" + ") == ["sddmm_tile_ptr_kernel", "sb_lists_kernel", "spmm_blocks_kernel<false>"]
    first = pyops._spmm(v, ri, scores, rot, cit, m, plan=plan, **kw)      # tables and lists are the SDDMM's: nothing to write
    assert _lib.last_kernels() == "spmm_blocks_kernel<false>"
    kept = pyops._spmm(v, ri, scores, rot, cit, m, plan=plan, **kw)
    assert _lib.last_kernels() == "spmm_blocks_kernel<false>"
    assert torch.equal(kept, fresh) and torch.equal(first, fresh)
    again_scores = pyops.sddmm_half_planned(q, kk, ri, rot, cit, plan)
    assert _lib.last_kernels() == "sddmm_mfma_kernel<false, 4>" and torch.equal(again_scores, scores)
    other_threshold = pyops._spmm(v, ri, scores, rot, cit, m, plan=plan, force_wpr=1, **kw)    # tables kept, lists not
    assert _lib.last_kernels().split(" + ") == ["sb_lists_kernel", "spmm_blocks_kernel<false>"]
    assert torch.allclose(other_threshold.float(), fresh.float(), rtol=1e-2, atol=1e-2)
    mask2 = np.abs(idx[:, None] - idx[None, :]) < 90
    ro2, ci2, _ = W.csr_from_mask(mask2)
    csr2 = W.CSR(m, m, np.ones(ci2.shape[0], np.float32), W.swizzle_from_offsets(ro2), ro2, ci2)
    ri2, _, rot2, cit2 = to_dev(csr2, dev)
    vals2 = torch.randn(2, csr2.nnz, device=dev, dtype=torch.float16)
    again = pyops._spmm(v, ri2, vals2, rot2, cit2, m, plan=plan, **kw)
    assert _lib.last_kernels().split(" + ")[0] == "sddmm_tile_ptr_kernel" and "spmm_blocks_kernel" in _lib.last_kernels()
    assert torch.equal(again, pyops._spmm(v, ri2, vals2, rot2, cit2, m, **kw))


def test_rows_past_the_last_one_do_not_count_towards_dense_blocks(dev):
    """The last block of 128 rows may hold fewer: its nonzeros per column block are those of the rows that exist (the
    cursors of the last row once stood in for the missing ones, which made a long last row count up to 128 times).
    130 rows, the last one with 43 nonzeros in each column block: none of its blocks reaches the threshold, so the
    row's list of nonzeros outside dense blocks holds all of them and the block's list of dense blocks is empty (read
    from the plan's workspace: the tables, 64 words of zeros, 2 words per nonzero, the rows' counts, the lists of
    dense blocks as 16-bit entries, tiles + 2 per block of rows)."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(3)
    m, k = 130, 700
    rows = [np.unique(np.concatenate([np.arange(max(0, r - 60), min(k, r + 60)), rng.integers(0, k, 3)])) for r in range(m)]
    rows[m - 1] = np.arange(0, k, 3)
    ro = np.zeros(m + 1, dtype=np.int32)
    np.cumsum([len(c) for c in rows], out=ro[1:])
    ci = np.concatenate(rows).astype(np.int32)
    csr = W.CSR(m, k, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
    ri, _, rot, cit = to_dev(csr, dev)
    vals = torch.from_numpy(rng.integers(-3, 4, (2, csr.nnz)).astype(np.float32)).to(dev).half()
    dense = torch.from_numpy(rng.integers(-3, 4, (2, k, 64)).astype(np.float32)).to(dev).half()
    kw = dict(per_batch_values=True, accumulate=False, dtypes=(torch.float16,), allow_i16=False)
    plan = pyops.SddmmPlan()
    got = pyops._spmm(dense, ri, vals, rot, cit, m, plan=plan, force_variant=10, **kw)
    assert torch.equal(got, pyops._spmm(dense, ri, vals, rot, cit, m, force_variant=1, **kw))
    tiles = (k + 127) // 128
    words = plan.workspace.view(torch.int32).cpu().numpy()
    lists_at = (m * (6 * tiles + 1) + 3) & ~3
    counts_at = lists_at + 64 + 2 * csr.nnz
    assert words[counts_at + m - 1] == len(rows[m - 1])
    dense_lists = words[counts_at + m:].view(np.uint16)
    assert dense_lists[0] >= 1 and dense_lists[tiles + 2] == 0      # the band in the first 128 rows; nothing in the last 2


def test_picked_for_attention_sized_products_with_values_per_head(dev):
    """Nothing forced: 16 heads of config 3's mask take this kernel when the values differ per head, the row kernel
    when they are shared or the product is small; a plan whose analysis found no structure keeps the row kernel."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    pat, _, _, v = W.config3()
    ri, _, ro, ci = to_dev(pat, dev)
    vt = torch.from_numpy(v).to(dev).half()
    probs = (torch.rand(16, pat.nnz, device=dev) / 280).half()
    got = ops.spmm_sputnik_batched_values(vt, ri, probs, ro, ci, pat.m)
    assert "spmm_blocks_kernel" in _lib.last_kernels()
    with pyops.kernel_params(spmm={"force_variant": 1}):
        rows = ops.spmm_sputnik_batched_values(vt, ri, probs, ro, ci, pat.m)
    assert "spmm_blocks_kernel" not in _lib.last_kernels()
    assert torch.allclose(got.float(), rows.float(), rtol=1e-2, atol=2e-3)
    ops.spmm_sputnik_reuse_weight_half(vt, ri, probs[0].contiguous(), ro, ci, pat.m)
    assert "spmm_blocks_kernel" not in _lib.last_kernels()
    ops.spmm_sputnik_batched_values(vt[:1], ri, probs[:1], ro, ci, pat.m)
    assert "spmm_blocks_kernel" not in _lib.last_kernels()
    plan = pyops.SddmmPlan()
    assert plan.analyze(ro, ci, pat.k) == 3
    planned = pyops.spmm_batched_values_planned(vt, ri, probs, ro, ci, pat.m, plan)
    assert "spmm_blocks_kernel" in _lib.last_kernels() and torch.equal(planned, got)
    pyops.spmm_batched_values_planned(vt, ri, probs, ro, ci, pat.m, plan)
    assert _lib.last_kernels() == "spmm_blocks_kernel<false>"
    fp32 = pyops.spmm_batched_values_planned(vt.float(), ri, probs.float(), ro, ci, pat.m, plan)     # the planned kernel does not serve fp32
    assert "spmm_blocks_kernel" not in _lib.last_kernels() and torch.allclose(fp32, rows.float(), rtol=1e-2, atol=2e-3)
    flat = pyops.SddmmPlan()
    flat.variant = 1
    pyops.spmm_batched_values_planned(vt, ri, probs, ro, ci, pat.m, flat)
    assert "spmm_blocks_kernel" not in _lib.last_kernels()


def test_refusals_and_workspace_size(dev):
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    flags = (10 << 16) | _lib.SPMM_PER_BATCH_VALUES
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I32, flags, 4096, 4096, 64, 1000, 16) == ((6 * 32 + 1) * 4096 + 64 + 2 * 1000 + 4096 + 32 * (32 + 2) // 2) * 4
    assert lib.iex_spmm_workspace_kind(_lib.F16, _lib.I32, flags, 4096, 4096, 64, 1000, 16) == 10
    assert lib.iex_spmm_workspace_kind(_lib.F16, _lib.I32, _lib.SPMM_PER_BATCH_VALUES, 4096, 4096, 64, 1000, 16) == 0        # too sparse for the rule
    assert lib.iex_spmm_workspace_kind(_lib.F16, _lib.I32, _lib.SPMM_PER_BATCH_VALUES, 4096, 4096, 64, 1 << 20, 16) == 10
    assert lib.iex_spmm_workspace_kind(_lib.F16, _lib.I32, 0, 4096, 4096, 64, 1 << 20, 16) != 10                              # shared values
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I32, flags, 4096, 4096, 128, 1000, 16) != 0      # two slices of 64 columns
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I32, flags, 4096, 4096, 96, 1000, 16) == 0       # n no multiple of 64
    assert lib.iex_spmm_workspace_bytes(_lib.F32, _lib.I32, flags, 4096, 4096, 64, 1000, 16) == 0
    assert lib.iex_spmm_workspace_bytes(_lib.F16, _lib.I16, flags, 4096, 4096, 64, 1000, 16) == 0
    rng = np.random.default_rng(1)
    csr = _pattern(rng, 64, 64, rng.integers(0, 20, 64))
    values = rng.standard_normal((1, csr.nnz)).astype(np.float32)
    with pytest.raises(RuntimeError, match="dense-blocks kernel needs fp16"):
        _run(dev, csr, values, rng.standard_normal((1, 64, 32)).astype(np.float32), torch.float16, force_variant=10)
    with pytest.raises(RuntimeError, match="workspace"):
        _run(dev, csr, values, rng.standard_normal((1, 64, 64)).astype(np.float32), torch.float16, force_variant=10, no_workspace=True)
