// Host side of the dense companion GEMM: kernel wrapper, tile-shape choice, XCD-aware
// tile order, argument checks and the C entry point.  Device code: gemm_device.cuh.
#include "gemm_device.cuh"

namespace iex {
namespace {

constexpr int kXcds = 8;

// Workgroup ids are dealt round-robin to the 8 XCDs (each with its own L2).  Give every
// XCD a contiguous band of C tiles (row-major over tiles) so that the A row panels a
// band needs are fetched into one L2 instead of eight.
__device__ __forceinline__ bool xcd_tile(int block, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int linear = (block % kXcds) * per_xcd + block / kXcds;
  if (linear >= total) return false;
  tile_m = linear / tiles_n;
  tile_n = linear % tiles_n;
  return true;
}

template <bool BF16, bool TRANS_B, int WM, int WN, int BK>
__global__ __launch_bounds__(256, (WM * WN <= 8 ? 2 : 1)) void gemm_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  int tile_m, tile_n;
  if (!xcd_tile(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n)) return;  // uniform per block
  // 128 x 256 tiles: 128 accumulators per lane leave room for two register sets in flight, not three
  gemm_tile<BF16, TRANS_B, WM, WN, (WM * WN == 8 || (BK == 64 && !TRANS_B) ? 2 : kGemmSets), 2, BK>(p, tile_m, tile_n, blockIdx.y, smem);
}

template <bool BF16, bool TRANS_B, int WM, int WN, int BK = kGemmBK>
int launch(GemmParams p, int batch, hipStream_t stream) {
  constexpr int BM = 2 * WM * 32, BN = 2 * WN * 32;
  p.tiles_m = ceil_div(p.M, BM);
  p.tiles_n = ceil_div(p.N, BN);
  const int total = p.tiles_m * p.tiles_n;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  constexpr int lds = gemm_lds_bytes<TRANS_B, WM, WN, 2, BK>();
  auto kern = gemm_kernel<BF16, TRANS_B, WM, WN, BK>;
  if (lds > 64 * 1024) {
    static thread_local bool raised = false;  // per instantiation
    if (!raised) {
      if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                             "hipFuncSetAttribute(LDS size)"))
        return rc;
      raised = true;
    }
  }
  hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds, batch), dim3(256), lds, stream, p);
  return check_hip(hipGetLastError(), "gemm launch");
}

template <bool BF16, bool TRANS_B>
int launch_shape(const GemmParams& p, int batch, int force, hipStream_t stream) {
  if (force == 1) return launch<BF16, TRANS_B, 2, 2>(p, batch, stream);
  if (force == 2) return launch<BF16, TRANS_B, 2, 4>(p, batch, stream);
  if (force == 3) return launch<BF16, TRANS_B, 4, 4>(p, batch, stream);
  if (force == 4) return launch<BF16, TRANS_B, 2, 2, 64>(p, batch, stream);
  // The larger the tile of a wave, the fewer LDS bytes each MFMA needs (128x128 per wave: half of
  // what 64x64 needs), and LDS bandwidth is what the main loop runs against; the smaller the tile,
  // the more workgroups there are to fill 256 CUs.  Measured at 4096..11008 x 8192 x 4096..8192:
  // 256x256 tiles (one wave per SIMD, 504 registers) 830-960 TFLOP/s, 128x256 770-890, 128x128
  // 715-770; at config 4's 4096 x 2048 x 4096 the order reverses (450-470, 620-690, 720-750).
  // Two tiles per CU is where the larger shape starts to win.
  const long long huge_tiles = (long long)ceil_div(p.M, 256) * ceil_div(p.N, 256) * batch;
  if (huge_tiles >= 512 && p.K >= 256) return launch<BF16, TRANS_B, 4, 4>(p, batch, stream);
  const long long wide_tiles = (long long)ceil_div(p.M, 128) * ceil_div(p.N, 256) * batch;
  if (wide_tiles >= 512 && p.K >= 256) return launch<BF16, TRANS_B, 2, 4>(p, batch, stream);
  // 128x128 tiles: K steps of 64 halve the barriers and double the distance between a global load
  // and its use (720-830 TFLOP/s against 660-770 with steps of 32 on the same shapes)
  if (p.K >= 128) return launch<BF16, TRANS_B, 2, 2, 64>(p, batch, stream);
  return launch<BF16, TRANS_B, 2, 2>(p, batch, stream);
}

}  // namespace
}  // namespace iex

// trans_b: bit 0 = B is (N, K); bits 4..7 force the tile shape for tuning (1 = 128x128, 2 = 128x256,
// 3 = 256x256, 4 = 128x128 with K steps of 64; 0 = choose).
extern "C" int iex_gemm(int dtype, int trans_b_and_shape, int M, int N, int K, const void* A, const void* B, void* C, int batch,
                        long long stride_a, long long stride_b, long long stride_c, void* stream) {
  using namespace iex;
  const int trans_b = trans_b_and_shape & 1, force = (trans_b_and_shape >> 4) & 0xf;
  IEX_REQUIRE(M >= 0 && N >= 0 && K >= 0 && batch >= 0, IEX_ERR_BAD_ARGUMENT, "gemm: negative dimension");
  if (M == 0 || N == 0 || batch == 0) return 0;
  IEX_REQUIRE(A && B && C, IEX_ERR_BAD_ARGUMENT, "gemm: null pointer argument");
  IEX_REQUIRE(dtype == IEX_F16 || dtype == IEX_BF16, IEX_ERR_UNSUPPORTED, "gemm: dtype must be fp16 or bf16");
  IEX_REQUIRE(K > 0 && K % 8 == 0, IEX_ERR_UNSUPPORTED, "gemm: K must be a positive multiple of 8 (K=%d)", K);
  IEX_REQUIRE(trans_b || N % 8 == 0, IEX_ERR_UNSUPPORTED, "gemm: N must be a multiple of 8 when B is (K,N) (N=%d)", N);
  IEX_REQUIRE(aligned(A, 16) && aligned(B, 16), IEX_ERR_UNSUPPORTED, "gemm: operands must be 16-byte aligned");
  IEX_REQUIRE(stride_a % 8 == 0 && stride_b % 8 == 0, IEX_ERR_UNSUPPORTED, "gemm: batch strides must be multiples of 8");
  IEX_REQUIRE(batch <= 65535, IEX_ERR_TOO_LARGE, "gemm: batch %d exceeds 65535", batch);
  IEX_REQUIRE((long long)M * K < (1ll << 31) && (long long)N * K < (1ll << 31) && (long long)M * N < (1ll << 31),
              IEX_ERR_TOO_LARGE, "gemm: an operand exceeds 2^31 elements per batch entry");
  GemmParams p{M, N, K, A, B, C, stride_a, stride_b, stride_c, 0, 0};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool bf = dtype == IEX_BF16;
  if (bf && trans_b) return launch_shape<true, true>(p, batch, force, s);
  if (bf && !trans_b) return launch_shape<true, false>(p, batch, force, s);
  if (!bf && trans_b) return launch_shape<false, true>(p, batch, force, s);
  return launch_shape<false, false>(p, batch, force, s);
}
