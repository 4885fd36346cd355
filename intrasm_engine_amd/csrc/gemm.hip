// Host side of the dense companion GEMM: kernel wrapper, tile-shape choice, XCD-aware
// tile order, argument checks and the C entry point.  Device code: gemm_device.cuh.
#include "gemm_pp_device.cuh"

namespace iex {
namespace {

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
  note_kernel("gemm_kernel<%s, %s, %d, %d, %d> (%d x %d tiles, operands staged through registers)", BF16 ? "bf16" : "f16",
              TRANS_B ? "B(N,K)" : "B(K,N)", WM, WN, BK, BM, BN);
  hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds, batch), dim3(256), lds, stream, p);
  return check_hip(hipGetLastError(), "gemm launch");
}

template <bool BF16, bool TRANS_B, int WM, int WN, int BK, int STAGES, int WCN>
__global__ __launch_bounds__(WCN * 128, (WCN == 2 && WM * WN <= 8 && gemm_dma_lds_bytes<WM, WN, WCN, BK, STAGES>() <= 80 * 1024 ? 2 : 1)) void gemm_dma_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  int tile_m, tile_n;
  if (!xcd_tile(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n)) return;  // uniform per block
  gemm_tile_dma<BF16, TRANS_B, WM, WN, WCN, BK, STAGES>(p, tile_m, tile_n, blockIdx.y, smem);
}

template <bool BF16, bool TRANS_B, int WM, int WN, int BK, int STAGES, int WCN = 2>
int launch_dma(GemmParams p, int batch, hipStream_t stream) {
  constexpr int BM = 2 * WM * 32, BN = WCN * WN * 32;
  p.tiles_m = ceil_div(p.M, BM);
  p.tiles_n = ceil_div(p.N, BN);
  const int total = p.tiles_m * p.tiles_n;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  constexpr int lds = gemm_dma_lds_bytes<WM, WN, WCN, BK, STAGES>();
  auto kern = gemm_dma_kernel<BF16, TRANS_B, WM, WN, BK, STAGES, WCN>;
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
  note_kernel("gemm_dma_kernel<%s, %s, %d, %d, %d, %d, %d> (%d x %d tiles, %d waves)", BF16 ? "bf16" : "f16", TRANS_B ? "B(N,K)" : "B(K,N)", WM, WN,
              BK, STAGES, WCN, BM, BN, 2 * WCN);
  hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds, batch), dim3(WCN * 128), lds, stream, p);
  return check_hip(hipGetLastError(), "gemm launch");
}

// Eight wavefronts in two groups that alternate between reading / loading and multiplying (gemm_pp_device.cuh).
template <bool BF16, bool TRANS_B, int WM, int WN, int WCN>
__global__ __launch_bounds__(WCN * 128, 1) void gemm_pp_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  int tile_m, tile_n;
  if (!xcd_tile(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n)) return;  // uniform per block
  gemm_tile_pp<BF16, TRANS_B, WM, WN, WCN>(p, tile_m, tile_n, blockIdx.y, smem);
}

template <bool BF16, bool TRANS_B, int WM, int WN, int WCN>
int launch_pp(GemmParams p, int batch, hipStream_t stream) {
  constexpr int BM = 2 * WM * 32, BN = WCN * WN * 32;
  p.tiles_m = ceil_div(p.M, BM);
  p.tiles_n = ceil_div(p.N, BN);
  const int total = p.tiles_m * p.tiles_n;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  constexpr int lds = gemm_pp_lds_bytes<BF16, TRANS_B, WM, WN, WCN>();
  auto kern = gemm_pp_kernel<BF16, TRANS_B, WM, WN, WCN>;
  static thread_local bool raised = false;  // per instantiation
  if (!raised) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "hipFuncSetAttribute(LDS size)"))
      return rc;
    raised = true;
  }
  note_kernel("gemm_pp_kernel<%s, %s, %d, %d, %d> (%d x %d tiles, two groups of 4 waves in alternating phases)", BF16 ? "bf16" : "f16",
              TRANS_B ? "B(N,K)" : "B(K,N)", WM, WN, WCN, BM, BN);
  hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds, batch), dim3(WCN * 128), lds, stream, p);
  return check_hip(hipGetLastError(), "gemm launch");
}

// K split over two workgroups per 256 x 256 tile, for products with so few tiles that half the CUs would idle
// and a long K.  Workgroups b and b + 8 (same XCD, dispatched one after the other) take the two halves of one tile.
// On request only (shape code 12): built for config 4's 4096 x 2048 x 4096 (128 tiles of 256 x 256), where it takes
// 92 us against 71 for 128 x 256 tiles by eight waves and 107 for the unsplit 256 x 256 tiles: the K loop of half the
// length runs 74 us, not half of 107 (prologue and epilogue of a 256 x 256 tile are 10 us whatever K is), and handing
// 32 MB of fp32 partial sums from one workgroup to the other costs another 18.
__global__ void fill_zero_kernel(int* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

template <bool BF16, bool TRANS_B, int WM, int WN, int WCN, int BK, int STAGES>
__global__ __launch_bounds__(WCN * 128, 1) void gemm_dma_splitk_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int b = blockIdx.x;
  const int part = (b >> 3) & 1, slot = (b >> 4) * kXcds + (b & 7);
  int tile_m, tile_n;
  if (!xcd_tile(slot, p.tiles_m, p.tiles_n, tile_m, tile_n)) return;  // uniform per block
  const int first = ((p.K + BK - 1) / BK / 2) * BK;   // K entries of the first half: whole steps
  GemmParams q = p;
  q.ldk = p.K;
  if (part == 0) {
    q.K = first;
  } else {
    q.K = p.K - first;
    q.A = static_cast<const unsigned short*>(p.A) + first;
    q.B = static_cast<const unsigned short*>(p.B) + (TRANS_B ? (size_t)first : (size_t)first * p.N);
  }
  gemm_tile_dma<BF16, TRANS_B, WM, WN, WCN, BK, STAGES, 1>(q, tile_m, tile_n, blockIdx.y, smem);
}

// Workspace of a K split: the partial sums of one half per tile (fp32), then two words per tile (ticket, "written").
inline size_t gemm_splitk_bytes(int M, int N, int batch, int bm, int bn) {
  const size_t tiles = (size_t)ceil_div(M, bm) * ceil_div(N, bn) * batch;
  return tiles * bm * bn * sizeof(float) + ((tiles * 2 * sizeof(int) + 255) / 256) * 256;
}

// flags_are_zero: the caller has zeroed the tile words on this stream already (they sit behind the partial sums).
template <bool BF16, bool TRANS_B, int WM, int WN, int WCN, int BK, int STAGES>
int launch_dma_splitk(GemmParams p, int batch, void* ws, bool flags_are_zero, hipStream_t stream) {
  constexpr int BM = 2 * WM * 32, BN = WCN * WN * 32;
  p.tiles_m = ceil_div(p.M, BM);
  p.tiles_n = ceil_div(p.N, BN);
  const int total = p.tiles_m * p.tiles_n;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  p.split_ws = static_cast<float*>(ws);
  p.split_flags = reinterpret_cast<int*>(static_cast<unsigned char*>(ws) + (size_t)total * batch * BM * BN * sizeof(float));
  constexpr int lds = gemm_dma_lds_bytes<WM, WN, WCN, BK, STAGES>();
  auto kern = gemm_dma_splitk_kernel<BF16, TRANS_B, WM, WN, WCN, BK, STAGES>;
  static thread_local bool raised = false;  // per instantiation
  if (!raised) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "hipFuncSetAttribute(LDS size)"))
      return rc;
    raised = true;
  }
  if (!flags_are_zero) {
    const int flags = 2 * total * batch;
    note_kernel("fill_zero_kernel");
    hipLaunchKernelGGL(fill_zero_kernel, dim3(ceil_div(flags, 256)), dim3(256), 0, stream, p.split_flags, flags);
  }
  note_kernel("gemm_dma_splitk_kernel<%s, %s> (%d x %d tiles, K in two halves)", BF16 ? "bf16" : "f16", TRANS_B ? "B(N,K)" : "B(K,N)", BM, BN);
  hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds * 2, batch), dim3(WCN * 128), lds, stream, p);
  return check_hip(hipGetLastError(), "gemm (split K) launch");
}

// ---- K split over several workgroups per tile, every part on one XCD, the last to finish adds up (gemm_dma_device.cuh)
template <bool BF16, bool TRANS_B, int WM, int WN, int WCN, int BK, int STAGES>
__global__ __launch_bounds__(WCN * 128, (WCN == 2 && WM * WN <= 8 && gemm_dma_lds_bytes<WM, WN, WCN, BK, STAGES>() <= 80 * 1024 ? 2 : 1)) void gemm_dma_parts_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int b = blockIdx.x, parts = p.split_parts;
  const int part = (b >> 3) % parts, slot = ((b >> 3) / parts) * kXcds + (b & 7);
  int tile_m, tile_n;
  if (!xcd_tile(slot, p.tiles_m, p.tiles_n, tile_m, tile_n)) return;  // uniform per block
  const int steps = (p.K + BK - 1) / BK, per = (steps + parts - 1) / parts * BK;   // K entries per part: whole steps
  const int k0 = part * per;   // (the host has chosen parts so that every part has a step)
  GemmParams q = p;
  q.ldk = p.K;
  q.split_part = part;
  q.K = min(per, p.K - k0);
  q.A = static_cast<const unsigned short*>(p.A) + k0;
  q.B = static_cast<const unsigned short*>(p.B) + (TRANS_B ? (size_t)k0 : (size_t)k0 * p.N);
  gemm_tile_dma<BF16, TRANS_B, WM, WN, WCN, BK, STAGES, 2>(q, tile_m, tile_n, blockIdx.y, smem);
}

// Parts per tile: as many as give every CU a workgroup, at most 8, every part at least 1024 of K, none empty.
inline int split_parts_for(int M, int N, int K, int batch, int bm, int bn, int bk) {
  const long long tiles = (long long)ceil_div(M, bm) * ceil_div(N, bn) * batch;
  const int steps = ceil_div(K, bk);
  int parts = (int)std::min<long long>(8, 256 / std::max<long long>(tiles, 1));
  parts = std::min(parts, K / 1024);
  while (parts > 1 && (parts - 1) * ceil_div(steps, parts) >= steps) --parts;
  return std::max(parts, 1);
}

// Workspace: per tile `parts` sets of partial sums (fp32), then one ticket word per tile.
inline size_t gemm_parts_bytes(int M, int N, int batch, int bm, int bn, int parts) {
  const size_t tiles = (size_t)ceil_div(M, bm) * ceil_div(N, bn) * batch;
  return tiles * parts * bm * bn * sizeof(float) + ((tiles * sizeof(int) + 255) / 256) * 256;
}

template <bool BF16, bool TRANS_B, int WM, int WN, int WCN, int BK, int STAGES>
int launch_dma_parts(GemmParams p, int batch, int parts, void* ws, bool flags_are_zero, hipStream_t stream) {
  constexpr int BM = 2 * WM * 32, BN = WCN * WN * 32;
  p.tiles_m = ceil_div(p.M, BM);
  p.tiles_n = ceil_div(p.N, BN);
  const int total = p.tiles_m * p.tiles_n;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  p.split_parts = parts;
  p.split_ws = static_cast<float*>(ws);
  p.split_flags = reinterpret_cast<int*>(static_cast<unsigned char*>(ws) + (size_t)total * batch * parts * BM * BN * sizeof(float));
  constexpr int lds = gemm_dma_lds_bytes<WM, WN, WCN, BK, STAGES>();
  auto kern = gemm_dma_parts_kernel<BF16, TRANS_B, WM, WN, WCN, BK, STAGES>;
  if (lds > 64 * 1024) {
    static thread_local bool raised = false;  // per instantiation
    if (!raised) {
      if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                             "hipFuncSetAttribute(LDS size)"))
        return rc;
      raised = true;
    }
  }
  if (!flags_are_zero) {
    note_kernel("fill_zero_kernel");
    hipLaunchKernelGGL(fill_zero_kernel, dim3(ceil_div(total * batch, 256)), dim3(256), 0, stream, p.split_flags, total * batch);
  }
  note_kernel("gemm_dma_parts_kernel<%s, %s> (%d x %d tiles, K in %d parts)", BF16 ? "bf16" : "f16", TRANS_B ? "B(N,K)" : "B(K,N)", BM, BN, parts);
  hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds * parts, batch), dim3(WCN * 128), lds, stream, p);
  return check_hip(hipGetLastError(), "gemm (K in parts) launch");
}

// Few 64 x 128 tiles and a long K: the K loop in parts, on as many CUs as there are.  Measured on MI355X (fp16, us, 64 x
// 128 tiles unsplit / in parts, the latter with a launch that zeroes the tickets): 4096 x 128 x 4096 23.8 / 17.1 (4 parts),
// 2048 x 256 x 4096 23.4 / 15.2 (4), 1000 x 200 x 4104 23.6 / 14.1 (8), 512 x 512 x 8192 42.5 / 17.6 (8), 4096 x 256 x 11008
// 57.1 / 45.6 (2), 4096 x 256 x 4096 24.0 / 21.8 (2), 4 x (1024 x 256 x 4096) 24.9 / 23.1 (2); but 4096 x 256 x 2048 13.5 /
// 14.4 and 8192 x 128 x 2048 14.1 / 15.2 (128 tiles in 2 parts: K must be long to pay).  128 x 128 tiles by four
// wavefronts in 4 to 8 parts: 22.7 where 64 x 128 tiles take 16.3.
inline bool auto_split_wanted(int M, int N, int K, int batch) {
  if (K <= 256) return false;
  if ((long long)ceil_div(M, 128) * ceil_div(N, 128) * batch > 256) return false;
  const long long half_tiles = (long long)ceil_div(M, 64) * ceil_div(N, 128) * batch;
  if (half_tiles > 128 || (half_tiles > 64 && K < 4096)) return false;
  return split_parts_for(M, N, K, batch, 64, 128, 64) >= 2;
}

template <bool BF16, bool TRANS_B>
int launch_shape(const GemmParams& p, int batch, int force, hipStream_t stream, void* ws, size_t ws_bytes, bool flags_are_zero) {
  if (force == 12) {
    IEX_REQUIRE(p.K >= 64, IEX_ERR_UNSUPPORTED, "gemm: the K-split kernel needs two K steps (K >= 64; K=%d)", p.K);
    IEX_REQUIRE(ws && aligned(ws, 256) && ws_bytes >= gemm_splitk_bytes(p.M, p.N, batch, 256, 256) && !p.accumulate, IEX_ERR_BAD_ARGUMENT,
                "gemm: the K-split kernel needs a 256-byte aligned workspace of %zu bytes (iex_gemm_ws) and a plain store", gemm_splitk_bytes(p.M, p.N, batch, 256, 256));
    return launch_dma_splitk<BF16, TRANS_B, 4, 4, 2, 32, 4>(p, batch, ws, flags_are_zero, stream);
  }
  if (force == 14) {
    const int parts = std::max(2, split_parts_for(p.M, p.N, p.K, batch, 64, 128, 64)), steps = ceil_div(p.K, 64);
    IEX_REQUIRE(steps >= parts && (parts - 1) * ceil_div(steps, parts) < steps, IEX_ERR_UNSUPPORTED,
                "gemm: K in %d parts needs a K step of 64 for every part (K=%d)", parts, p.K);
    IEX_REQUIRE(ws && aligned(ws, 256) && ws_bytes >= gemm_parts_bytes(p.M, p.N, batch, 64, 128, parts) && !p.accumulate, IEX_ERR_BAD_ARGUMENT,
                "gemm: K in parts needs a 256-byte aligned workspace of %zu bytes (iex_gemm_ws) and a plain store", gemm_parts_bytes(p.M, p.N, batch, 64, 128, parts));
    return launch_dma_parts<BF16, TRANS_B, 1, 1, 4, 64, 4>(p, batch, parts, ws, flags_are_zero, stream);
  }
  if (force == 1) return launch<BF16, TRANS_B, 2, 2>(p, batch, stream);
  if (force == 2) return launch<BF16, TRANS_B, 2, 4>(p, batch, stream);
  if (force == 3) return launch<BF16, TRANS_B, 4, 4>(p, batch, stream);
  if (force == 4) return launch<BF16, TRANS_B, 2, 2, 64>(p, batch, stream);
  if (force == 5) return launch_dma<BF16, TRANS_B, 2, 2, 32, 4>(p, batch, stream);
  if (force == 6) return launch_dma<BF16, TRANS_B, 2, 4, 32, 4>(p, batch, stream);
  if (force == 7) return launch_dma<BF16, TRANS_B, 4, 4, 32, 4>(p, batch, stream);
  if (force == 8) return launch_dma<BF16, TRANS_B, 2, 1, 64, 4, 4>(p, batch, stream);
  if (force == 9) return launch_dma<BF16, TRANS_B, 1, 1, 64, 4, 4>(p, batch, stream);
  if (force == 10) return launch_dma<BF16, TRANS_B, 2, 2, 32, 4, 4>(p, batch, stream);
  if (force == 11) return launch_dma<BF16, TRANS_B, 2, 2, 64, 3, 4>(p, batch, stream);
  if (force == 13) return launch_pp<BF16, TRANS_B, 4, 2, 4>(p, batch, stream);
  // Default: operands straight from global memory into LDS (gemm_dma_device.cuh).  The larger the
  // tile of a wave, the fewer LDS bytes each MFMA needs, and LDS time is what the main loop runs
  // against; the smaller the tile, the more workgroups there are to fill 256 CUs, and a tile wider
  // than what is left of the matrix computes columns nobody stores.  (Register-staged operands, codes 1..4:
  // 8192^3 256x256 980 TFLOP/s against 1200 here.)
  // A short K (at most 8 steps) is prologue and epilogue: small tiles, two workgroups per CU that cover for
  // each other (512 x (512 x 512 x 128), the attention scores of the decoder layer: 229 -> 123 us; 8192 x 8192 x
  // 128: 59 -> 48; from K = 512 the large tiles are ahead again).
  if (p.K <= 256) return launch_dma<BF16, TRANS_B, 2, 2, 32, 4>(p, batch, stream);
  const long long small_tiles = (long long)ceil_div(p.M, 128) * ceil_div(p.N, 128) * batch;
  if (small_tiles > 256) {
    // More 128 x 128 tiles than CUs: the tile shape that finishes first, counting whole rounds of workgroups (a
    // workgroup of the last round takes as long as any other) at the rate each shape reaches with every CU busy.
    // TFLOP/s measured: 256 x 256 (one workgroup per CU, eight waves in two alternating groups) 1250; 128 x 256 by eight waves (64 x 64 each, two per
    // SIMD that cover for each other at the barrier and the waits of every K step; one workgroup per CU) 930,
    // by four waves (64 x 128 each) 790; 128 x 128 (two workgroups per CU) 750.
    //   4096 x 2048 x 4096 (config 4): 627 / 907 / 788 / 750      4096 x 4096 x 4096: 1080 / 985 / 903
    //   11008 x 4096 x 4096: 1093 / 952 / 914                      8192^3: 1208 / 1065 / 1055
    // (128 x 256 by eight waves with five or six stages instead of four: 860 and 850 on config 4's shape.)
    auto cost = [&](int bm, int bn, int slots, double rate) {
      const long long tiles = (long long)ceil_div(p.M, bm) * ceil_div(p.N, bn) * batch;
      return (double)ceil_div(tiles, slots) * slots * bm * bn / rate;
    };
    const double huge = cost(256, 256, 256, 1250.0), wide = cost(128, 256, 256, 930.0), small = cost(128, 128, 512, 750.0);
    // (256 x 256 by two groups of four waves in alternating phases, same-process comparison with the four-wave tile on
    // warmed-up clocks: 8192^3 1250 / 1230, 4096 x 8192 x 4096 1109 / 1076, 11008 x 8192 x 4096 1151 / 1109,
    // 4096^3 1054 / 954; bit-equal results.  11008 x 2048 x 4096, where the two shapes are within 1 % in this count:
    // 218 us in two rounds of 256 x 256 tiles, 221-230 in three of 128 x 256)
    if (huge <= wide && huge <= small) return launch_pp<BF16, TRANS_B, 4, 2, 4>(p, batch, stream);
    if (wide <= small) return launch_dma<BF16, TRANS_B, 2, 2, 32, 4, 4>(p, batch, stream);
    return launch_dma<BF16, TRANS_B, 2, 2, 32, 4>(p, batch, stream);
  }
  // One round of at most one 128 x 128 tile per CU and a long K: eight waves (64 x 32 each) and K steps of 64
  // (4096 x 512 x 4096: 44 -> 34.5 us; eight waves with steps of 32 and eight stages 38.6; 64 x 128 tiles 36.8).
  // Such a product runs on the few CUs that have a tile (128 x 128 x 4096 is 16 us of one CU's matrix cores at
  // their peak and takes 34) while the others idle; only a K split over workgroups (partial sums in a
  // workspace) would change that.
  // Half as tall (64 x 128) where even that leaves at most one tile per CU: twice the CUs at work
  // (4096 x 256 x 4096: 35 -> 27.5 us, 4096 x 512 x 4096: 35 -> 30, 1024 x 2048 x 1024: 13.9 -> 12.4).
  const long long half_tiles = (long long)ceil_div(p.M, 64) * ceil_div(p.N, 128) * batch;
  // ... and with room for the partial sums, K in parts on as many CUs as there are
  if (auto_split_wanted(p.M, p.N, p.K, batch) && !p.accumulate) {
    const int parts = split_parts_for(p.M, p.N, p.K, batch, 64, 128, 64);
    if (ws && aligned(ws, 256) && ws_bytes >= gemm_parts_bytes(p.M, p.N, batch, 64, 128, parts))
      return launch_dma_parts<BF16, TRANS_B, 1, 1, 4, 64, 4>(p, batch, parts, ws, flags_are_zero, stream);
  }
  if (half_tiles <= 256 && p.K >= 512) return launch_dma<BF16, TRANS_B, 1, 1, 64, 4, 4>(p, batch, stream);
  if (p.K >= 2048) return launch_dma<BF16, TRANS_B, 2, 1, 64, 4, 4>(p, batch, stream);
  return launch_dma<BF16, TRANS_B, 2, 2, 32, 4>(p, batch, stream);
}

}  // namespace
}  // namespace iex

// trans_b: bit 0 = B is (N, K); bits 4..7 force the kernel for tuning.  Register-staged operands:
// 1 = 128x128 tiles, 2 = 128x256, 3 = 256x256, 4 = 128x128 with K steps of 64.  Operands loaded
// straight into LDS: 5 = 128x128, 6 = 128x256, 7 = 256x256, 8 = 128x128, 9 = 64x128 by eight waves with K steps of 64,
// 10 = 128x256 by eight waves, 11 = the same with K steps of 64, 12 = 256x256 with K split over two workgroups per tile
// (iex_gemm_ws only; never chosen), 13 = 256x256 by eight waves in two groups that alternate between loading and
// multiplying, 14 = 64x128 by eight waves with K split over two to eight workgroups per tile (iex_gemm_ws only).
// 0 = choose (one of 5, 8, 9, 10, 13, and 14 where iex_gemm_workspace_bytes asked for room and got it).
extern "C" int iex_gemm(int dtype, int trans_b_and_shape, int M, int N, int K, const void* A, const void* B, void* C, int batch,
                        long long stride_a, long long stride_b, long long stride_c, void* stream) {
  iex::trail_reset();
  return iex::gemm_dispatch(dtype, trans_b_and_shape, M, N, K, A, B, C, batch, stride_a, stride_b, stride_c, stream, nullptr, 0, 0);
}

extern "C" int iex_gemm_ws(int dtype, int trans_b_and_shape, int M, int N, int K, const void* A, const void* B, void* C, int batch,
                           long long stride_a, long long stride_b, long long stride_c, void* stream, void* workspace, size_t workspace_bytes) {
  iex::trail_reset();
  return iex::gemm_dispatch(dtype, trans_b_and_shape, M, N, K, A, B, C, batch, stride_a, stride_b, stride_c, stream, nullptr, 0, 0, workspace,
                            workspace_bytes);
}

extern "C" size_t iex_gemm_workspace_bytes(int dtype, int trans_b_and_shape, int M, int N, int K, int batch) {
  if (M <= 0 || N <= 0 || K <= 0 || batch <= 0 || (dtype != IEX_F16 && dtype != IEX_BF16)) return 0;
  const int force = (trans_b_and_shape >> 4) & 0xf;
  if (force == 12) return iex::gemm_splitk_bytes(M, N, batch, 256, 256);
  if (force == 14) return iex::gemm_parts_bytes(M, N, batch, 64, 128, 8);
  return force == 0 ? iex::gemm_auto_split_bytes(M, N, K, batch) : 0;
}

size_t iex::gemm_auto_split_bytes(int M, int N, int K, int batch) {
  return auto_split_wanted(M, N, K, batch) ? gemm_parts_bytes(M, N, batch, 64, 128, split_parts_for(M, N, K, batch, 64, 128, 64)) : 0;
}

int iex::gemm_auto_split_parts(int M, int N, int K, int batch) {
  return auto_split_wanted(M, N, K, batch) ? split_parts_for(M, N, K, batch, 64, 128, 64) : 1;
}

void iex::gemm_auto_split_flags(int M, int N, int K, int batch, size_t* offset_bytes, int* words) {
  const size_t tiles = (size_t)ceil_div(M, 64) * ceil_div(N, 128) * batch;
  *offset_bytes = tiles * split_parts_for(M, N, K, batch, 64, 128, 64) * 64 * 128 * sizeof(float);
  *words = (int)tiles;
}

int iex::gemm_dispatch(int dtype, int trans_b_and_shape, int M, int N, int K, const void* A, const void* B, void* C, int batch,
                       long long stride_a, long long stride_b, long long stride_c, void* stream, const float* row_bias, int relu,
                       int accumulate, void* workspace, size_t workspace_bytes, bool workspace_flags_are_zero) {
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
  GemmParams p{M, N, K, A, B, C, stride_a, stride_b, stride_c, 0, 0, row_bias, relu, accumulate};
  p.stream_out = (double)M * N * batch * 2 >= 128e6;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool bf = dtype == IEX_BF16;
  if (bf && trans_b) return launch_shape<true, true>(p, batch, force, s, workspace, workspace_bytes, workspace_flags_are_zero);
  if (bf && !trans_b) return launch_shape<true, false>(p, batch, force, s, workspace, workspace_bytes, workspace_flags_are_zero);
  if (!bf && trans_b) return launch_shape<false, true>(p, batch, force, s, workspace, workspace_bytes, workspace_flags_are_zero);
  return launch_shape<false, false>(p, batch, force, s, workspace, workspace_bytes, workspace_flags_are_zero);
}
