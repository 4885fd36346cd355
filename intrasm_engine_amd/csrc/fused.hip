// Horizontally fused sparse + dense launch: ONE grid whose workgroups are split between
// tiles of the dense GEMM (matrix cores) and row blocks of the fp16 CSR SpMM (vector ALU
// + memory pipeline), so that both kinds of work are resident on the same compute units
// at the same time without relying on the runtime to overlap two kernels.
//
// Workgroup roles
//   interleave == 0 : ids [0, G) run GEMM tiles, ids [G, G+S) run SpMM blocks;
//   interleave < 0  : ids [0, S) run SpMM blocks, ids [S, S+G) run GEMM tiles: the longer jobs first (a CU takes the
//                     next id whenever it has room), so the short GEMM tiles fill what the SpMM's last round leaves;
//   interleave == g : the G GEMM workgroups are spread through the id range in ceil(G/g) groups of g
//                     consecutive ids, each followed by its even share of the SpMM blocks, so both
//                     kinds are dispatched side by side from start to end while the tiles of a
//                     group still share their operand panels in L2.
// The GEMM may be batched (tiles of all batch entries are enumerated).
// Two kernels, picked by what the stand-alone SpMM of the same shape would run on:
//   gather     256 threads; GEMM tiles of 128 x 128 beside row blocks of the row kernel (at most 4
//              wavefronts per row); LDS of the larger role (the GEMM's 40 KB);
//   matrix     512 threads; GEMM tiles of 128 x 256 (2 x 4 wavefronts) beside 128 x 512 tiles of
//   cores      the 8-wave matrix-core SpMM.  Both roles then want the matrix cores: the launch is
//              a grouped GEMM whose sparse member is expanded in LDS, and what fusing buys is
//              one launch and full tails, not complementary units.
// The device code of both roles is the code of the stand-alone kernels, so results are
// bit-identical to separate launches.
#include "gemm_dma_device.cuh"
#include "spmm_mfma2_device.cuh"

namespace iex {
namespace {

struct FusedParams {
  GemmParams g;
  SpmmParams s;
  int gemm_batch, gemm_blocks, spmm_blocks, spmm_by, interleave;
  unsigned long long* timeline;   // diagnostic (iex_fused_timeline): 4 words per workgroup, or null
};

// Where and when a workgroup ran, for the diagnostic timeline: constant-rate clock (100 MHz), the XCD and the
// hardware id word (compute unit, shader array, shader engine in bits 8..15).
__device__ __forceinline__ unsigned long long fused_clock() { return wall_clock64(); }
__device__ __forceinline__ unsigned fused_where() {
  unsigned hw, xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
  return ((xcc & 0xf) << 16) | (hw & 0xffff);
}

constexpr int kFusedWM = 2, kFusedWN = 2;
// The GEMM role's registers and LDS leave two waves per SIMD; the SpMM role makes up for the
// missing waves by keeping four times as many gathers in flight per wave.
constexpr int kFusedWin = 32;

// Role of workgroup b: GEMM tile `idx` or SpMM block `idx`.  A bijection between the ids [0, G + S) and
// the G tiles plus the S blocks for every G >= 0, S >= 0 and group size g >= 0:
//   g == 0: ids [0, G) are the tiles, [G, G + S) the blocks;
//   g < 0:  ids [0, S) are the blocks, [S, S + G) the tiles;
//   g >= 1: Q = ceil(G / g) groups, each "its tiles, then its share of the blocks"; group q holds the
//           tiles [q g, min(G, (q + 1) g)) and floor(S / Q) blocks, one more in the first S mod Q groups
//           (the last group, the only one that can be short of tiles, never gets the extra block).
// Host and device: the host side is exported as iex_fused_role for the CPU test of this mapping.
__host__ __device__ inline void fused_role_of(int gemm_blocks, int spmm_blocks, int interleave, int b, bool& is_gemm, int& idx) {
  const int G = gemm_blocks, S = spmm_blocks, g = interleave;
  if (g < 0) {
    is_gemm = b >= S;
    idx = is_gemm ? b - S : b;
    return;
  }
  if (g == 0 || G == 0) {
    is_gemm = b < G;
    idx = is_gemm ? b : b - G;
    return;
  }
  const int Q = (G + g - 1) / g;          // groups
  const int s0 = S / Q, r = S % Q;        // blocks per group, groups with one more
  const long long u1 = (long long)g + s0 + 1, u0 = (long long)g + s0;
  const int q = (b < r * u1) ? (int)(b / u1) : r + (int)((b - r * u1) / u0);
  const long long blocks_before = (long long)q * s0 + (q < r ? q : r);
  const int off = (int)(b - ((long long)q * g + blocks_before));
  const int tiles_here = (G - q * g < g) ? G - q * g : g;
  is_gemm = off < tiles_here;
  idx = is_gemm ? q * g + off : (int)(blocks_before + off - tiles_here);
}

__device__ __forceinline__ void fused_role(const FusedParams& p, int b, bool& is_gemm, int& idx) {
  fused_role_of(p.gemm_blocks, p.spmm_blocks, p.interleave, b, is_gemm, idx);
}

template <bool BF16, bool TRANS_B, typename IT, int VEC, int LPG, int WPR>
__global__ __launch_bounds__(256) void fused_kernel(FusedParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  bool is_gemm;
  int idx;
  fused_role(p, blockIdx.x, is_gemm, idx);
  if (is_gemm) {
    const int per_batch = p.g.tiles_m * p.g.tiles_n;
    const int z = idx / per_batch, t = idx % per_batch;
    gemm_tile<BF16, TRANS_B, kFusedWM, kFusedWN>(p.g, t / p.g.tiles_n, t % p.g.tiles_n, z, smem);
  } else {
    spmm_block<__half, IT, VEC, LPG, WPR, kFusedWin>(p.s, idx / p.spmm_by, idx % p.spmm_by, 0, reinterpret_cast<float*>(smem));
  }
}

// ---- both roles on the matrix cores -------------------------------------------------------------
constexpr int kFusedMcWM = 2, kFusedMcWN = 2, kFusedMcWCN = 4;  // GEMM tile 128 x 256 by 2 x 4 wavefronts

template <bool BF16, bool TRANS_B, typename IT, int W>
__global__ __launch_bounds__(kMfma2Threads, 2) void fused_mc_kernel(FusedParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  bool is_gemm;
  int idx;
  fused_role(p, blockIdx.x, is_gemm, idx);
  const unsigned long long began = p.timeline ? fused_clock() : 0ull;
  if (is_gemm) {
    const int per_batch = p.g.tiles_m * p.g.tiles_n;
    const int z = idx / per_batch, t = idx % per_batch;
    gemm_tile_dma<BF16, TRANS_B, kFusedMcWM, kFusedMcWN, kFusedMcWCN, 32, 4>(p.g, t / p.g.tiles_n, t % p.g.tiles_n, z, smem);
  } else {
    // p.spmm_by = row tiles here: consecutive ids walk the row blocks of one column panel
    spmm_mfma2_block<false, IT, W, 128>(p.s, idx % p.spmm_by, idx / p.spmm_by, 0, smem);
  }
  if (p.timeline) {   // (uniform over the grid; the tile routines return to here in every wavefront)
    __syncthreads();
    if (threadIdx.x == 0) {
      unsigned long long* t = p.timeline + 4ull * blockIdx.x;
      t[0] = began;
      t[1] = fused_clock();
      t[2] = fused_where();
      t[3] = (is_gemm ? 1ull << 32 : 0ull) | (unsigned)idx;
    }
  }
}

template <bool BF16, bool TRANS_B, typename IT, int W>
int launch_mc(FusedParams p, hipStream_t stream) {
  constexpr int BM = 2 * kFusedMcWM * 32, BN = kFusedMcWCN * kFusedMcWN * 32;
  p.g.tiles_m = ceil_div(p.g.M, BM);
  p.g.tiles_n = ceil_div(p.g.N, BN);
  IEX_REQUIRE((long long)p.g.tiles_m * p.g.tiles_n * p.gemm_batch < (1ll << 30), IEX_ERR_TOO_LARGE, "fused: too many GEMM tiles");
  p.gemm_blocks = p.g.tiles_m * p.g.tiles_n * p.gemm_batch;
  p.spmm_by = ceil_div(p.s.m, kMfmaBM);
  p.spmm_blocks = p.spmm_by * ceil_div(p.s.n, kMfma2BN);
  constexpr int lds_gemm = gemm_dma_lds_bytes<kFusedMcWM, kFusedMcWN, kFusedMcWCN, 32, 4>();
  constexpr int lds_spmm = spmm_mfma2_lds_bytes<128>();
  constexpr int lds = lds_gemm > lds_spmm ? lds_gemm : lds_spmm;
  auto kernel = fused_mc_kernel<BF16, TRANS_B, IT, W>;
  static thread_local bool raised = false;  // per instantiation: more than 64 KB of dynamic LDS
  if (!raised) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "hipFuncSetAttribute(LDS size)"))
      return rc;
    raised = true;
  }
  trail_reset();
  note_kernel("fused_mc_kernel<%s, %s, %s, %d> (%d GEMM tiles, %d SpMM tiles)", BF16 ? "true" : "false", TRANS_B ? "true" : "false", type_name<IT>(), W,
              p.gemm_blocks, p.spmm_blocks);
  hipLaunchKernelGGL(kernel, dim3(p.gemm_blocks + p.spmm_blocks), dim3(kMfma2Threads), lds, stream, p);
  return check_hip(hipGetLastError(), "fused (matrix-core) launch");
}

template <bool BF16, bool TRANS_B, typename IT>
int launch_mc_w(const FusedParams& p, int windows, hipStream_t stream) {
  switch (windows) {
    case 1: return launch_mc<BF16, TRANS_B, IT, 1>(p, stream);
    case 2: return launch_mc<BF16, TRANS_B, IT, 2>(p, stream);
    case 4: return launch_mc<BF16, TRANS_B, IT, 4>(p, stream);
    case 5: return launch_mc<BF16, TRANS_B, IT, 5>(p, stream);
  }
  return fail(IEX_ERR_BAD_ARGUMENT, "fused: unexpected window count %d", windows);
}

template <typename IT>
int launch_mc_kind(const FusedParams& p, int windows, bool bf16, bool trans_b, hipStream_t stream) {
  if (bf16 && trans_b) return launch_mc_w<true, true, IT>(p, windows, stream);
  if (bf16 && !trans_b) return launch_mc_w<true, false, IT>(p, windows, stream);
  if (!bf16 && trans_b) return launch_mc_w<false, true, IT>(p, windows, stream);
  return launch_mc_w<false, false, IT>(p, windows, stream);
}

template <bool BF16, bool TRANS_B, typename IT, int VEC, int LPG, int WPR>
int launch(FusedParams p, hipStream_t stream) {
  constexpr int BM = 2 * kFusedWM * 32, BN = 2 * kFusedWN * 32;
  p.g.tiles_m = ceil_div(p.g.M, BM);
  p.g.tiles_n = ceil_div(p.g.N, BN);
  IEX_REQUIRE((long long)p.g.tiles_m * p.g.tiles_n * p.gemm_batch < (1ll << 30), IEX_ERR_TOO_LARGE, "fused: too many GEMM tiles");
  p.gemm_blocks = p.g.tiles_m * p.g.tiles_n * p.gemm_batch;
  const int rows_per_block = 4 / WPR;
  p.spmm_by = ceil_div(p.s.n, LPG * VEC);
  const long long sb = (long long)ceil_div(p.s.m, rows_per_block) * p.spmm_by;
  IEX_REQUIRE(sb + p.gemm_blocks < (1ll << 31), IEX_ERR_TOO_LARGE, "fused: grid too large");
  p.spmm_blocks = (int)sb;
  constexpr int lds_gemm = gemm_lds_bytes<TRANS_B, kFusedWM, kFusedWN>();
  constexpr int lds_spmm = spmm_lds_floats<VEC, WPR>() * 4;
  constexpr int lds = lds_gemm > lds_spmm ? lds_gemm : lds_spmm;
  trail_reset();
  note_kernel("fused_kernel<%s, %s, %s, %d, %d, %d> (%d GEMM tiles, %d SpMM blocks)", BF16 ? "true" : "false", TRANS_B ? "true" : "false",
              type_name<IT>(), VEC, LPG, WPR, p.gemm_blocks, p.spmm_blocks);
  hipLaunchKernelGGL((fused_kernel<BF16, TRANS_B, IT, VEC, LPG, WPR>), dim3(p.gemm_blocks + p.spmm_blocks), dim3(256), lds, stream,
                     p);
  return check_hip(hipGetLastError(), "fused launch");
}

// Waves per row as the stand-alone kernel would choose, capped at the 4 wavefronts of a
// 256-thread workgroup (so results equal the stand-alone launch with that choice).
template <bool BF16, bool TRANS_B, typename IT, int VEC, int LPG>
int launch_w(const FusedParams& p, hipStream_t stream) {
  if (spmm_pick_wpr(p.s.m, p.s.nnz) >= 4) return launch<BF16, TRANS_B, IT, VEC, LPG, 4>(p, stream);
  return launch<BF16, TRANS_B, IT, VEC, LPG, 1>(p, stream);
}

template <bool BF16, bool TRANS_B, typename IT>
int launch_vec(const FusedParams& p, SpmmShape sh, hipStream_t stream) {
  if (sh.vec == 8) {
    switch (sh.lpg) {
      case 8: return launch_w<BF16, TRANS_B, IT, 8, 8>(p, stream);
      case 16: return launch_w<BF16, TRANS_B, IT, 8, 16>(p, stream);
      case 32: return launch_w<BF16, TRANS_B, IT, 8, 32>(p, stream);
      default: return launch_w<BF16, TRANS_B, IT, 8, 64>(p, stream);
    }
  }
  switch (sh.vec) {
    case 4: return launch_w<BF16, TRANS_B, IT, 4, 64>(p, stream);
    case 2: return launch_w<BF16, TRANS_B, IT, 2, 64>(p, stream);
    default: return launch_w<BF16, TRANS_B, IT, 1, 64>(p, stream);
  }
}

template <typename IT>
int launch_gemm_kind(const FusedParams& p, SpmmShape vec, bool bf16, bool trans_b, hipStream_t stream) {
  if (bf16 && trans_b) return launch_vec<true, true, IT>(p, vec, stream);
  if (bf16 && !trans_b) return launch_vec<true, false, IT>(p, vec, stream);
  if (!bf16 && trans_b) return launch_vec<false, true, IT>(p, vec, stream);
  return launch_vec<false, false, IT>(p, vec, stream);
}

}  // namespace
}  // namespace iex

extern "C" int iex_fused_role(int gemm_blocks, int spmm_blocks, int interleave, int id, int* is_gemm, int* index) {
  using namespace iex;
  IEX_REQUIRE(gemm_blocks >= 0 && spmm_blocks >= 0 && is_gemm && index, IEX_ERR_BAD_ARGUMENT,
              "fused role: negative count or null pointer");
  IEX_REQUIRE(id >= 0 && (long long)id < (long long)gemm_blocks + spmm_blocks, IEX_ERR_BAD_ARGUMENT,
              "fused role: id %d outside the grid of %lld workgroups", id, (long long)gemm_blocks + spmm_blocks);
  bool ig;
  int idx;
  fused_role_of(gemm_blocks, spmm_blocks, interleave, id, ig, idx);
  *is_gemm = ig ? 1 : 0;
  *index = idx;
  return 0;
}

// The buffer that the next matrix-core fused launches of this thread write their timeline to (null: none).
static thread_local unsigned long long* g_fused_timeline = nullptr;
extern "C" int iex_fused_timeline(void* buffer) {
  g_fused_timeline = static_cast<unsigned long long*>(buffer);
  return 0;
}

extern "C" int iex_fused_spmm_gemm(int spmm_itype, int m, int k, int n, int nonzeros, const int* row_indices,
                                   const void* values, const int* row_offsets, const void* column_indices,
                                   const void* dense, void* spmm_out, int gemm_dtype, int trans_b, int M, int N, int K,
                                   const void* A, const void* B, void* C, int gemm_batch, long long stride_a,
                                   long long stride_b, long long stride_c, int interleave, void* stream) {
  using namespace iex;
  IEX_REQUIRE(m > 0 && k > 0 && n > 0 && nonzeros >= 0, IEX_ERR_BAD_ARGUMENT, "fused: SpMM dimensions must be positive");
  IEX_REQUIRE(M > 0 && N > 0 && K > 0 && gemm_batch > 0, IEX_ERR_BAD_ARGUMENT, "fused: GEMM dimensions must be positive");
  IEX_REQUIRE(stride_a % 8 == 0 && stride_b % 8 == 0, IEX_ERR_UNSUPPORTED, "fused: GEMM batch strides must be multiples of 8");
  IEX_REQUIRE(row_indices && row_offsets && dense && spmm_out && A && B && C, IEX_ERR_BAD_ARGUMENT,
              "fused: null pointer argument");
  IEX_REQUIRE(nonzeros == 0 || (values && column_indices), IEX_ERR_BAD_ARGUMENT, "fused: null values / column_indices");
  IEX_REQUIRE(spmm_itype == IEX_I32 || (spmm_itype == IEX_I16 && k <= 32768), IEX_ERR_BAD_ARGUMENT,
              "fused: int16 column indices need k <= 32768");
  IEX_REQUIRE(gemm_dtype == IEX_F16 || gemm_dtype == IEX_BF16, IEX_ERR_UNSUPPORTED, "fused: GEMM dtype must be fp16 or bf16");
  IEX_REQUIRE(K % 8 == 0, IEX_ERR_UNSUPPORTED, "fused: K must be a multiple of 8 (K=%d)", K);
  IEX_REQUIRE(trans_b || N % 8 == 0, IEX_ERR_UNSUPPORTED, "fused: N must be a multiple of 8 when B is (K,N)");
  IEX_REQUIRE(aligned(A, 16) && aligned(B, 16), IEX_ERR_UNSUPPORTED, "fused: GEMM operands must be 16-byte aligned");
  IEX_REQUIRE((long long)k * n < (1ll << 31) && (long long)m * n < (1ll << 31) && (long long)M * K < (1ll << 31) &&
                  (long long)N * K < (1ll << 31) && (long long)M * N < (1ll << 31),
              IEX_ERR_TOO_LARGE, "fused: an operand exceeds 2^31 elements");
  FusedParams p{};
  p.g = GemmParams{M, N, K, A, B, C, stride_a, stride_b, stride_c, 0, 0};
  p.gemm_batch = gemm_batch;
  p.s = SpmmParams{m, k, n, nonzeros, row_indices, values, row_offsets, column_indices, dense, nullptr, spmm_out, 0, 0, 0};
  p.interleave = interleave;
  p.timeline = nullptr;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (const int windows = spmm_matrix_core_windows(p.s)) {
    p.timeline = g_fused_timeline;  // what the stand-alone SpMM of this shape runs on
    if (spmm_itype == IEX_I16) return launch_mc_kind<short>(p, windows, gemm_dtype == IEX_BF16, trans_b != 0, s);
    return launch_mc_kind<int>(p, windows, gemm_dtype == IEX_BF16, trans_b != 0, s);
  }
  const SpmmShape vec = spmm_pick_shape<__half>(n, dense, spmm_out);
  if (spmm_itype == IEX_I16) return launch_gemm_kind<short>(p, vec, gemm_dtype == IEX_BF16, trans_b != 0, s);
  return launch_gemm_kind<int>(p, vec, gemm_dtype == IEX_BF16, trans_b != 0, s);
}
