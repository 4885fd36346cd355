"""GPU parity of the MFMA companion GEMM against the CPU oracle."""
import numpy as np
import pytest
import torch

from _util import assert_close, rounded

pytestmark = pytest.mark.gpu
ops = torch.ops.iex_ops


def _check(oracle, dev, M, N, K, dtype, trans_b, seed=0):
    rng = np.random.default_rng(seed)
    a_np = rng.standard_normal((M, K)).astype(np.float32)
    b_np = rng.standard_normal((N, K) if trans_b else (K, N)).astype(np.float32)
    a, b = torch.from_numpy(a_np).to(dev).to(dtype), torch.from_numpy(b_np).to(dev).to(dtype)
    out = ops.gemm_mfma(a, b, trans_b)
    assert out.shape == (M, N) and out.dtype == dtype
    a_r, b_r = rounded(a_np, dtype), rounded(b_np, dtype)
    want = oracle.gemm(a_r, b_r, trans_b=trans_b)
    scale = oracle.gemm(np.abs(a_r), np.abs(b_r), trans_b=trans_b)
    assert_close(out.float().cpu().numpy(), want, scale, 1e-2, f"gemm {M}x{N}x{K} {dtype} trans_b={trans_b}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("shape", [(128, 128, 32), (256, 128, 64), (512, 384, 256), (100, 64, 72), (33, 264, 8),
                                   (1, 8, 8), (300, 136, 1000), (257, 520, 200)])
def test_gemm_shapes(oracle, dev, dtype, trans_b, shape):
    _check(oracle, dev, *shape, dtype, trans_b)


@pytest.mark.parametrize("shape", [(100, 60, 72), (33, 260, 8), (1, 4, 8), (300, 131, 1000)])
def test_gemm_ragged_n_with_transposed_b(oracle, dev, shape):
    """B given as (N, K) has no constraint on N (B as (K, N) needs N % 8 == 0)."""
    _check(oracle, dev, *shape, torch.bfloat16, True)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ops.gemm_mfma(torch.zeros(8, 8, device=dev).half(), torch.zeros(8, shape[1] | 1, device=dev).half(), False)


@pytest.mark.parametrize("shape_code", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 13])
@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mnk", [(300, 520, 200), (129, 136, 8), (260, 264, 1000)])
def test_every_tile_shape(oracle, dev, shape_code, trans_b, dtype, mnk):
    """Every kernel of the GEMM entry point forced through the C ABI (register-staged 128x128, 128x256, 256x256 tiles
    and 128x128 with K steps of 64; 128x128, 128x256, 256x256, 128x128 and 64x128 by eight waves with K steps of 64, and 128x256 by eight waves with K steps of 32 and 64, operands loaded straight
    into LDS) on ragged
    problems: m, n and k leave partial tiles and a partial last K step; k = 8 is a single, mostly empty step;
    k = 1000 runs the load pipeline through many steps and ends on a partial one."""
    from intrasm_engine_amd import _lib
    rng = np.random.default_rng(shape_code)
    M, N, K = mnk
    a_np = rng.standard_normal((M, K)).astype(np.float32)
    b_np = rng.standard_normal((N, K) if trans_b else (K, N)).astype(np.float32)
    a, b = torch.from_numpy(a_np).to(dev).to(dtype), torch.from_numpy(b_np).to(dev).to(dtype)
    out = torch.empty(M, N, device=dev, dtype=dtype)
    rc = _lib.load().iex_gemm(2 if dtype == torch.bfloat16 else 1, int(trans_b) | (shape_code << 4), M, N, K,
                              a.data_ptr(), b.data_ptr(), out.data_ptr(), 1, 0, 0, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, _lib.load().iex_last_error()
    a_r, b_r = rounded(a_np, dtype), rounded(b_np, dtype)
    want = oracle.gemm(a_r, b_r, trans_b=trans_b)
    scale = oracle.gemm(np.abs(a_r), np.abs(b_r), trans_b=trans_b)
    assert_close(out.float().cpu().numpy(), want, scale, 1e-2, f"tile shape {shape_code} {dtype} trans_b={trans_b}")


def test_large_tiles(oracle, dev):
    """Enough 128x256 tiles (and a long enough K) to select the wide-tile kernel; a corner is
    checked against the oracle and the whole result against the transposed-B layout of the
    same kernel."""
    rng = np.random.default_rng(3)
    M, N, K = 4096, 8192, 256
    a_np = rng.standard_normal((M, K)).astype(np.float32)
    b_np = rng.standard_normal((K, N)).astype(np.float32)
    a, b = torch.from_numpy(a_np).to(dev).half(), torch.from_numpy(b_np).to(dev).half()
    out = ops.gemm_mfma(a, b, False)
    want = oracle.gemm(rounded(a_np[-300:], torch.float16), rounded(b_np[:, -520:], torch.float16))
    scale = oracle.gemm(np.abs(a_np[-300:]), np.abs(b_np[:, -520:]))
    assert_close(out[-300:, -520:].float().cpu().numpy(), want, scale, 1e-2, "large tiles corner")
    assert torch.equal(ops.gemm_mfma(a, b.t().contiguous(), True), out)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_integer_inputs_are_exact(dev, dtype):
    """randint(-3, 3) operands (the idiom of the reference's tests/test_CUDAGraphConstructor.py:88-93)
    make the product exact: the result must equal the integer matmul, for both tile shapes."""
    g = torch.Generator().manual_seed(2023)
    for (M, N, K) in ((512, 512, 128), (4096, 2048, 256), (1024, 256, 512)):
        a = torch.randint(-3, 3, (M, K), generator=g).to(dev)
        b = torch.randint(-3, 3, (K, N), generator=g).to(dev)
        want = (a.double() @ b.double())
        assert want.abs().max() <= 256 * 9
        out = ops.gemm_mfma(a.to(dtype), b.to(dtype), False)
        # products of small integers are exact in fp32; bf16 output rounding needs |C| < 256
        if dtype == torch.float16 or want.abs().max() < 256:
            assert torch.equal(out.double(), want)
        else:
            assert torch.allclose(out.double(), want, rtol=2 ** -8)
        out_t = ops.gemm_mfma(a.to(dtype), b.t().contiguous().to(dtype), True)
        assert torch.equal(out_t, out)


def test_config4_dense_branch(oracle, dev):
    """bf16 (4096x4096)(4096x2048): a 256-row x 512-column corner is checked against the
    oracle, the whole product against the same kernel fed the transposed-B layout."""
    rng = np.random.default_rng(21)
    a_np = rng.standard_normal((4096, 4096)).astype(np.float32)
    b_np = rng.standard_normal((4096, 2048)).astype(np.float32)
    a, b = torch.from_numpy(a_np).to(dev).bfloat16(), torch.from_numpy(b_np).to(dev).bfloat16()
    out = ops.gemm_mfma(a, b, False)
    a_r, b_r = rounded(a_np[:256], torch.bfloat16), rounded(b_np[:, :512], torch.bfloat16)
    want = oracle.gemm(a_r, b_r)
    scale = oracle.gemm(np.abs(a_r), np.abs(b_r))
    assert_close(out[:256, :512].float().cpu().numpy(), want, scale, 1e-2, "C4 GEMM corner")
    assert torch.equal(ops.gemm_mfma(a, b.t().contiguous(), True), out)


def test_batched(oracle, dev):
    rng = np.random.default_rng(5)
    a_np = rng.standard_normal((6, 96, 64)).astype(np.float32)
    b_np = rng.standard_normal((6, 64, 40)).astype(np.float32)
    a, b = torch.from_numpy(a_np).to(dev).half(), torch.from_numpy(b_np).to(dev).half()
    out = ops.gemm_mfma(a, b, False)
    assert out.shape == (6, 96, 40)
    for z in range(6):
        want = oracle.gemm(rounded(a_np[z], torch.float16), rounded(b_np[z], torch.float16))
        scale = oracle.gemm(np.abs(a_np[z]), np.abs(b_np[z]))
        assert_close(out[z].float().cpu().numpy(), want, scale, 1e-2, f"batched z={z}")
    # shared B
    out2 = ops.gemm_mfma(a, b[0].contiguous(), False)
    assert torch.equal(out2[0], out[0])


def test_argument_checks(dev):
    a = torch.randn(16, 12, device=dev).half()
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ops.gemm_mfma(a, torch.randn(12, 16, device=dev).half(), False)
    with pytest.raises(RuntimeError, match="fp16 or bf16"):
        ops.gemm_mfma(a.float(), a.float(), True)
    with pytest.raises(RuntimeError, match="inner dimensions"):
        ops.gemm_mfma(torch.randn(16, 16, device=dev).half(), torch.randn(8, 16, device=dev).half(), False)


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mnk,batch", [((300, 520, 200), 1), ((260, 264, 1000), 3), ((512, 256, 64), 2), ((129, 136, 2048), 1), ((70, 136, 8200), 1)])
@pytest.mark.parametrize("split,whole", [(12, 7), (14, 9)])
def test_k_split_over_two_workgroups(oracle, dev, trans_b, dtype, mnk, batch, split, whole):
    """256 x 256 tiles with K in two halves (code 12) and 64 x 128 tiles with K in two to eight parts (code 14: partial
    sums meet in a workspace, the last workgroup to arrive adds them up in the order of the parts and stores), on
    request: ragged m, n, a K whose halves are 96 + 104 (128 + 72 with steps of 64), 512 + 488 (a partial last step),
    32 + 32, a K of 2048 in two parts; batches; against the oracle, twice with the same bits, and on integer operands
    exactly equal to the unsplit kernel of the same tile."""
    from intrasm_engine_amd.pytorch import ops as pyops
    rng = np.random.default_rng(batch)
    M, N, K = mnk
    if split == 14 and K < 128:
        with pytest.raises(RuntimeError, match="K step of 64 for every part"), pyops.kernel_params(gemm={"tile": 14}):
            ops.gemm_mfma(torch.zeros(M, K, device=dev, dtype=dtype), torch.zeros(K, N, device=dev, dtype=dtype), False)
        return
    a_np = rng.standard_normal((batch, M, K)).astype(np.float32)
    b_np = rng.standard_normal((batch, N, K) if trans_b else (batch, K, N)).astype(np.float32)
    a, b = torch.from_numpy(a_np).to(dev).to(dtype), torch.from_numpy(b_np).to(dev).to(dtype)
    with pyops.kernel_params(gemm={"tile": split}):
        out = ops.gemm_mfma(a, b, trans_b)
        again = ops.gemm_mfma(a, b, trans_b)
    assert torch.equal(out, again)
    for z in range(batch):
        a_r, b_r = rounded(a_np[z], dtype), rounded(b_np[z], dtype)
        want = oracle.gemm(a_r, b_r, trans_b=trans_b)
        scale = oracle.gemm(np.abs(a_r), np.abs(b_r), trans_b=trans_b)
        assert_close(out[z].float().cpu().numpy(), want, scale, 1e-2, f"split-K gemm {M}x{N}x{K} {dtype} trans_b={trans_b} entry {z}")
    ai = torch.from_numpy(rng.integers(-3, 4, a_np.shape).astype(np.float32)).to(dev).to(dtype)
    bi = torch.from_numpy(rng.integers(-3, 4, b_np.shape).astype(np.float32)).to(dev).to(dtype)
    with pyops.kernel_params(gemm={"tile": split}):
        in_halves = ops.gemm_mfma(ai, bi, trans_b)
    with pyops.kernel_params(gemm={"tile": whole}):
        at_once = ops.gemm_mfma(ai, bi, trans_b)
    assert torch.equal(in_halves, at_once)


def test_k_split_is_picked_for_few_tiles_and_a_long_k(oracle, dev):
    """4096 x 128 x 4096 (64 tiles of 64 x 128 on 256 CUs: K in four parts): the operator asks the library how much room the split wants,
    gets a number, passes the room and the split kernel runs; the entry point without a workspace runs the unsplit tile.
    Shapes with more tiles or a shorter K ask for nothing.  Twice the same bits; against the oracle on sampled rows."""
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    M, N, K = 4096, 128, 4096
    assert lib.iex_gemm_workspace_bytes(_lib.F16, 0, M, N, K, 1) == 64 * 4 * 64 * 128 * 4 + 256      # 64 tiles in 4 parts, a ticket per tile
    assert lib.iex_gemm_workspace_bytes(_lib.F16, 14 << 4, M, N, K, 1) == 64 * 8 * 64 * 128 * 4 + 256  # on request: room for 8 parts
    assert lib.iex_gemm_workspace_bytes(_lib.F16, 0, M, 256, K, 1) == 128 * 2 * 64 * 128 * 4 + 512    # 128 tiles in 2 parts
    assert lib.iex_gemm_workspace_bytes(_lib.F16, 0, M, 256, 2048, 1) == 0        # 128 tiles and K < 4096
    assert lib.iex_gemm_workspace_bytes(_lib.F16, 0, M, N, 2048, 1) == 64 * 2 * 64 * 128 * 4 + 256   # 64 tiles: two parts of 1024
    assert lib.iex_gemm_workspace_bytes(_lib.F16, 0, M, N, 1024, 1) == 0
    assert lib.iex_gemm_workspace_bytes(_lib.F16, 0, M, N, K, 4) == 0            # four times the tiles
    assert lib.iex_gemm_workspace_bytes(_lib.F16, 9 << 4, M, N, K, 1) == 0       # another kernel on request
    rng = np.random.default_rng(9)
    a_np = rng.standard_normal((M, K)).astype(np.float32)
    b_np = rng.standard_normal((K, N)).astype(np.float32)
    a, b = torch.from_numpy(a_np).to(dev).half(), torch.from_numpy(b_np).to(dev).half()
    out = ops.gemm_mfma(a, b, False)
    assert "gemm_dma_parts_kernel" in _lib.last_kernels() and "64 x 128 tiles, K in 4 parts" in _lib.last_kernels()
    assert torch.equal(out, ops.gemm_mfma(a, b, False))
    rows = np.arange(0, M, 61)
    a_r, b_r = rounded(a_np[rows], torch.float16), rounded(b_np, torch.float16)
    scale = np.abs(a_r).astype(np.float64) @ np.abs(b_r).astype(np.float64)
    assert_close(out[torch.from_numpy(rows).to(dev)].float().cpu().numpy(), oracle.gemm(a_r, b_r), scale, 1e-2, "few tiles, K split")
    c = torch.empty_like(out)
    rc = lib.iex_gemm(_lib.F16, 0, M, N, K, a.data_ptr(), b.data_ptr(), c.data_ptr(), 1, 0, 0, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and "parts" not in _lib.last_kernels()
    torch.cuda.synchronize()
    assert torch.allclose(c.float(), out.float(), rtol=2e-2, atol=0.5)


def test_k_split_on_config4s_product_and_refused_without_workspace(oracle, dev):
    """The product the kernel was built for (4096 x 2048 x 4096: 128 tiles of 256 x 256), on request; the library never
    picks it by itself (it measured slower than 128 x 256 tiles by eight waves)."""
    from intrasm_engine_amd import _lib
    from intrasm_engine_amd.pytorch import ops as pyops
    lib = _lib.load()
    assert lib.iex_gemm_workspace_bytes(_lib.BF16, 12 << 4, 4096, 2048, 4096, 1) == 128 * 256 * 256 * 4 + 1024
    assert lib.iex_gemm_workspace_bytes(_lib.BF16, 0, 4096, 2048, 4096, 1) == 0
    rng = np.random.default_rng(4)
    a_np = rng.standard_normal((4096, 4096)).astype(np.float32)
    b_np = rng.standard_normal((4096, 2048)).astype(np.float32)
    a, b = torch.from_numpy(a_np).to(dev).bfloat16(), torch.from_numpy(b_np).to(dev).bfloat16()
    plain = ops.gemm_mfma(a, b, False)
    assert "splitk" not in _lib.last_kernels()
    with pyops.kernel_params(gemm={"tile": 12}):
        out = ops.gemm_mfma(a, b, False)
    assert "gemm_dma_splitk_kernel" in _lib.last_kernels()
    rows = np.arange(0, 4096, 67)
    a_r, b_r = rounded(a_np[rows], torch.bfloat16), rounded(b_np, torch.bfloat16)
    want = oracle.gemm(a_r, b_r)
    scale = np.abs(a_r).astype(np.float64) @ np.abs(b_r).astype(np.float64)
    assert_close(out[torch.from_numpy(rows).to(dev)].float().cpu().numpy(), want, scale, 1e-2, "config 4's product, K split")
    assert torch.allclose(plain.float(), out.float(), rtol=2e-2, atol=1.0)
    c = torch.empty_like(out)
    rc = lib.iex_gemm(_lib.BF16, 12 << 4, 4096, 2048, 4096, a.data_ptr(), b.data_ptr(), c.data_ptr(), 1, 0, 0, 0,
                      torch.cuda.current_stream().cuda_stream)
    assert rc != 0 and "workspace" in _lib.last_error()
    torch.cuda.synchronize()
