"""The two kernels for patterns with structure (SDDMM variant 3, SpMM family 10) on seeded random cases, bit for bit
against the gather / row kernels: operands are small integers, so every fp32 sum is exact and the kernels must agree
whatever the order of their additions.  Shapes that are no multiples of any tile, four kinds of pattern (random,
band + scattered, runs that start and end anywhere, blocks), every way of choosing the dense blocks, both 16-bit
types, 1 to 3 batch entries, 64 or 128 dense columns, k = 32, 64 or 128 for the SDDMM."""
import numpy as np
import pytest
import torch

from intrasm_engine_amd import workloads as W
from _util import to_dev

pytestmark = pytest.mark.gpu


def _random_mask(rng, m, k):
    kind = int(rng.integers(0, 4))
    mask = np.zeros((m, k), bool)
    if kind == 0:
        mask = rng.random((m, k)) < rng.choice([0.01, 0.05, 0.2, 0.6])
    elif kind == 1:
        width = int(rng.integers(1, 200))
        idx = np.arange(m)
        centre = idx * k // max(m, 1)
        mask = np.abs(centre[:, None] - np.arange(k)[None, :]) < width
        extra = int(rng.integers(0, 5))
        if extra:
            mask[np.repeat(idx, extra), rng.integers(0, k, (m, extra)).ravel()] = True
    elif kind == 2:
        for r in range(m):
            for _ in range(int(rng.integers(0, 4))):
                a = int(rng.integers(0, k))
                mask[r, a:min(k, a + int(rng.integers(1, 150)))] = True
    else:
        size = int(rng.choice([16, 64, 128, 256]))
        mask = (np.arange(m)[:, None] // size) == (np.arange(k)[None, :] // size)
        mask &= rng.random((m, k)) < rng.choice([0.5, 1.0])
    return mask


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_patterns_agree_exactly_with_the_gather_kernels(dev, seed):
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(seed)
    done = 0
    while done < 15:
        wide = done % 5 == 4                                   # every fifth case: many column blocks
        m = int(rng.integers(1, 260 if wide else 700))
        k = int(rng.integers(8, 30000 if wide else 900))
        ro, ci, _ = W.csr_from_mask(_random_mask(rng, m, k))
        if ci.shape[0] == 0:
            continue
        done += 1
        csr = W.CSR(m, k, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
        ri, _, rot, cit = to_dev(csr, dev)
        batch = int(rng.integers(1, 4))
        dtype = [torch.float16, torch.bfloat16][int(rng.integers(0, 2))]
        code = int(rng.choice([0, 1, 2, 3, 8, 255]))
        what = f"seed {seed} case {done}: {m} x {k}, {csr.nnz} nonzeros, {batch} entries, {dtype}, threshold code {code}"
        small = lambda *shape: torch.from_numpy(rng.integers(-3, 4, shape).astype(np.float32)).to(dev).to(dtype)

        n = int(rng.choice([64, 128]))
        values, dense = small(batch, csr.nnz), small(batch, k, n)
        kw = dict(per_batch_values=True, accumulate=False, dtypes=(dtype,), allow_i16=False)
        want = pyops._spmm(dense, ri, values, rot, cit, m, force_variant=1, **kw)
        got = pyops._spmm(dense, ri, values, rot, cit, m, force_variant=10, force_wpr=code, **kw)
        assert torch.equal(got, want), "SpMM, " + what

        depth = int(rng.choice([32, 64, 128]))
        lhs, rhs = small(batch, m, depth), small(batch, k, depth)
        kw = dict(sum_over_batch=False, dtypes=(dtype,))
        want = pyops._sddmm(lhs, rhs, ri, rot, cit, force_variant=1, **kw)
        got = pyops._sddmm(lhs, rhs, ri, rot, cit, force_variant=3, force_wpr=code, **kw)
        assert torch.equal(got, want), "SDDMM, " + what


def test_calls_that_share_a_plan_in_any_order(dev):
    """Random sequences of the two operators on three patterns with one plan between them (tables and lists are written,
    kept or written again as pattern and threshold change): every result equals that of the gather / row kernel."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(5)
    for trial in range(4):
        m = int(rng.integers(100, 700))
        patterns = []
        for _ in range(3):
            idx = np.arange(m)
            mask = np.abs(idx[:, None] - idx[None, :]) < int(rng.integers(8, 120))
            extra = int(rng.integers(0, 4))
            if extra:
                mask[np.repeat(idx, extra), rng.integers(0, m, (m, extra)).ravel()] = True
            ro, ci, _ = W.csr_from_mask(mask)
            csr = W.CSR(m, m, np.ones(ci.shape[0], np.float32), W.swizzle_from_offsets(ro), ro, ci)
            patterns.append((csr, to_dev(csr, dev)))
        plan = pyops.SddmmPlan()
        heads = int(rng.integers(1, 4))
        small = lambda *shape: torch.from_numpy(rng.integers(-3, 4, shape).astype(np.float32)).to(dev).half()
        for step in range(20):
            csr, (ri, _, ro, ci) = patterns[int(rng.integers(0, 3))]
            code = int(rng.choice([0, 0, 0, 1, 3, 255]))
            if rng.integers(0, 2):
                a, b = small(heads, m, 64), small(heads, m, 64)
                kw = dict(sum_over_batch=False, dtypes=(torch.float16,))
                got = pyops._sddmm(a, b, ri, ro, ci, plan=plan, force_variant=3, force_wpr=code, **kw)
                want = pyops._sddmm(a, b, ri, ro, ci, force_variant=1, **kw)
            else:
                v, d = small(heads, csr.nnz), small(heads, m, 64)
                kw = dict(per_batch_values=True, accumulate=False, dtypes=(torch.float16,), allow_i16=False)
                got = pyops._spmm(d, ri, v, ro, ci, m, plan=plan, force_variant=10, force_wpr=code, **kw)
                want = pyops._spmm(d, ri, v, ro, ci, m, force_variant=1, **kw)
            assert torch.equal(got, want), (trial, step, code)
