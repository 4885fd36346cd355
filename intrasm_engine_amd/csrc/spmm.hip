// Host side of the CSR SpMM: kernel wrappers, variant selection, argument checks and
// the C entry points.  The device code is in spmm_device.cuh.
#include <algorithm>
#include <cmath>
#include <mutex>
#include "spmm_lds_device.cuh"
#include "spmm_mfma2_device.cuh"
#include "spmm_mfma3_device.cuh"
#include "spmm_mfma_f32_device.cuh"
#include "spmm_dense_device.cuh"
#include "spmm_smallk_device.cuh"

namespace iex {
namespace {

template <typename T, typename IT, int VEC, int LPG, int WPR, int NT>
__global__ __launch_bounds__((WPR > 4 ? WPR : 4) * 64) void spmm_kernel(SpmmParams p) {
  __shared__ float red[spmm_lds_floats<VEC, WPR, NT>()];
  spmm_block<T, IT, VEC, LPG, WPR, (NT > 1 ? kSpmmUnroll / 2 : kSpmmUnroll), NT>(p, blockIdx.x, blockIdx.y, blockIdx.z, red);
}

template <typename T, typename IT, int VEC, int LPG, int WPR, int NT = 1>
int launch_one(const SpmmParams& p, int batch, hipStream_t stream) {
  constexpr int kWavesPerBlock = (WPR > 4) ? WPR : 4;
  constexpr int kRowsPerBlock = kWavesPerBlock / WPR;
  dim3 grid(ceil_div(p.m, kRowsPerBlock), ceil_div(p.n, NT * LPG * VEC), batch);
  dim3 block(kWavesPerBlock * kWave);
  note_kernel("spmm_kernel<%s, %s, %d, %d, %d, %d>", type_name<T>(), type_name<IT>(), VEC, LPG, WPR, NT);
  hipLaunchKernelGGL((spmm_kernel<T, IT, VEC, LPG, WPR, NT>), grid, block, 0, stream, p);
  return check_hip(hipGetLastError(), "spmm launch");
}

// n not a multiple of the 128-bit vector: full-width tiles with vectors at element alignment
template <typename T, typename IT, int VEC, int WPR>
__global__ __launch_bounds__((WPR > 4 ? WPR : 4) * 64) void spmm_ragged_kernel(SpmmParams p) {
  __shared__ float red[spmm_lds_floats<VEC, WPR, 1>()];
  spmm_block<T, IT, VEC, kWave, WPR, kSpmmUnroll, 1, true>(p, blockIdx.x, blockIdx.y, blockIdx.z, red);
}

template <typename T, typename IT, int VEC, int WPR>
int launch_ragged_one(const SpmmParams& p, int batch, hipStream_t stream) {
  constexpr int kWavesPerBlock = (WPR > 4) ? WPR : 4;
  constexpr int kRowsPerBlock = kWavesPerBlock / WPR;
  dim3 grid(ceil_div(p.m, kRowsPerBlock), ceil_div(p.n, kWave * VEC), batch);
  note_kernel("spmm_ragged_kernel<%s, %s, %d, %d>", type_name<T>(), type_name<IT>(), VEC, WPR);
  hipLaunchKernelGGL((spmm_ragged_kernel<T, IT, VEC, WPR>), grid, dim3(kWavesPerBlock * kWave), 0, stream, p);
  return check_hip(hipGetLastError(), "spmm (ragged rows) launch");
}

template <typename T, typename IT, int VEC>
int launch_ragged(const SpmmParams& p, int batch, int wpr, hipStream_t stream) {
  switch (wpr) {
    case 1: return launch_ragged_one<T, IT, VEC, 1>(p, batch, stream);
    case 4: return launch_ragged_one<T, IT, VEC, 4>(p, batch, stream);
    case 8: return launch_ragged_one<T, IT, VEC, 8>(p, batch, stream);
  }
  return fail(IEX_ERR_BAD_ARGUMENT, "spmm: waves-per-row must be 1, 4 or 8 (got %d)", wpr);
}

// ---- few columns in A, wide output: the dense operand's tile lives in LDS ---------------------
template <typename T, typename IT, int VEC, bool RAGGED, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void spmm_smallk_kernel(SpmmParams p, int rows_per_wave) {
  extern __shared__ __align__(16) unsigned char smem[];
  spmm_smallk_block<T, IT, VEC, RAGGED, WAVES>(p, rows_per_wave, blockIdx.x, blockIdx.y, blockIdx.z, smem);
}

// full vectors at their natural alignment, or (ragged) any n at element alignment
template <typename T>
bool smallk_aligned(const SpmmParams& p) {
  constexpr int kMax = 16 / (int)sizeof(T);
  return p.n % kMax == 0 && aligned(p.dense, 16) && aligned(p.out, 16);
}

template <typename T>
bool smallk_fits(const SpmmParams& p) {
  constexpr int kMax = 16 / (int)sizeof(T);
  return p.k >= 1 && p.k <= kSmallKMax && p.n >= kWave * kMax && aligned(p.dense, sizeof(T)) && aligned(p.out, sizeof(T));
}

// ... and where the library takes it by itself: up to 64 columns (two workgroups per CU), enough rows for
// the tile load (k KB per workgroup) to be a fraction of what the workgroup writes, and rows that gather:
// from 1.8 nonzeros per row the LDS gather wins (fp32, per-batch values: 192 x 784 x 784 outputs,
// k = 32, 2 per row: 107 against 127 us; 8 x 4096 x 4096, k = 64, 6 per row: 126 / 172, 32 per row: 344 / 535);
// almost empty rows are a plain write, which the row kernel does at 6 TB/s with streaming stores
// (96 x 3136 x 3136, 0.5 per row: 627 against 711).
template <typename T>
bool smallk_wanted(const SpmmParams& p, int batch) {
  (void)batch;
  // (rows that are no multiple of the vector: from 2.5 per row -- 384 x 785 x 785, k = 64: 3.2 per row 377 -> 322 us,
  // 1.9 per row 290 -> 313)
  // k = 65 .. 128 (one workgroup of 16 wavefronts per CU): from 4 per row and 32 k rows -- 8 x 4096 x 4096, k = 128:
  // 6.4 per row 166 -> 137 us, 1.3 per row 102 -> 120.
  if (!smallk_fits<T>(p)) return false;
  if (p.k > 64) return p.m >= 32 * p.k && (double)p.nnz >= 4.0 * p.m;
  return p.m >= 8 * p.k && (double)p.nnz >= (smallk_aligned<T>(p) ? 1.8 : 2.5) * p.m;
}

template <typename T, typename IT>
int launch_smallk(const SpmmParams& p, int batch, hipStream_t stream) {
  constexpr int kMax = 16 / (int)sizeof(T);
  // rows per wavefront: enough for the tile load (k KB per workgroup) to be a fraction of the output
  // (8 * rows KB), as long as that leaves every CU several workgroups
  const long long tiles = (long long)ceil_div(p.n, kWave * kMax) * batch;
  const int waves = smallk_waves(p.k);
  int rows = std::min(64, std::max(16, p.k / 2));
  while (rows > 4 && (long long)ceil_div(p.m, waves * rows) * tiles < 1024) rows >>= 1;
  const int lds = p.k * kWave * 16;
  const bool ragged = !smallk_aligned<T>(p);
  auto kern = waves == 8 ? (ragged ? spmm_smallk_kernel<T, IT, kMax, true, 8> : spmm_smallk_kernel<T, IT, kMax, false, 8>)
                         : (ragged ? spmm_smallk_kernel<T, IT, kMax, true, 16> : spmm_smallk_kernel<T, IT, kMax, false, 16>);
  if (lds > 64 * 1024) {
    static thread_local bool raised[2] = {false, false};  // per instantiation and alignment variant
    if (!raised[ragged]) {
      if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 kSmallKMax * kWave * 16),
                             "hipFuncSetAttribute(LDS size)"))
        return rc;
      raised[ragged] = true;
    }
  }
  dim3 grid(ceil_div(p.m, waves * rows), ceil_div(p.n, kWave * kMax), batch);
  note_kernel("spmm_smallk_kernel<%s, %s, %d, %s, %d>", type_name<T>(), type_name<IT>(), kMax, ragged ? "true" : "false", waves);
  hipLaunchKernelGGL(kern, grid, dim3(waves * kWave), lds, stream, p, rows);
  return check_hip(hipGetLastError(), "spmm (few columns) launch");
}

template <typename T, typename IT, int VEC, int LPG>
int launch_wpr(const SpmmParams& p, int batch, int wpr, int nt, hipStream_t stream) {
  if constexpr (LPG == kWave && VEC * sizeof(T) == 16) {
    // full-width tiles: a wave may cover 2 adjacent tiles (4 waves per row only)
    if (nt == 2 && wpr == 4) return launch_one<T, IT, VEC, LPG, 4, 2>(p, batch, stream);
  }
  switch (wpr) {
    case 1: return launch_one<T, IT, VEC, LPG, 1>(p, batch, stream);
    case 4: return launch_one<T, IT, VEC, LPG, 4>(p, batch, stream);
    case 8: return launch_one<T, IT, VEC, LPG, 8>(p, batch, stream);
  }
  return fail(IEX_ERR_BAD_ARGUMENT, "spmm: waves-per-row must be 1, 4 or 8 (got %d)", wpr);
}

// ---- row kernel with wavefronts per row that follow the row's own length ---------------------------------
template <typename T, typename IT, int VEC, int LPG>
__global__ __launch_bounds__(kRowsWaves * kWave) void spmm_rows_kernel(SpmmParams p, RowClasses rc) {
  __shared__ float red[spmm_rows_lds_floats<VEC>()];
  spmm_rows_block<T, IT, VEC, LPG>(p, rc, blockIdx.x, blockIdx.y, blockIdx.z, red);
}

// From the histogram of row lengths (hist[j] = rows with more than 64 << j nonzeros, j = 0 .. 15) to the five ranges
// of row slots.  A wavefront should get at most `rounds` chunks of 64 nonzeros (a power of two, 1 .. 16): a row of c
// chunks gets the smallest power of two >= c / rounds wavefronts, at most 16.  `rounds` follows the work per
// wavefront slot when every row is cut that way: with fewer chunks than the chip holds wavefronts (256 CUs x 16) one
// chunk per wavefront is the shortest critical path; with more, cutting finer only adds partial sums.
inline RowClasses row_classes(const SpmmParams& p, const int* hist, int tiles, int force_log2_rounds_plus_1, int* rounds_out) {
  const double chunks = (double)p.nnz / kWave * tiles;
  int r = 0;   // log2(rounds)
  while (r < 4 && chunks / (1 << r) > 256.0 * 16) ++r;
  if (force_log2_rounds_plus_1 > 0) r = std::min(force_log2_rounds_plus_1 - 1, 8);
  auto rows_over = [&](int log2_chunks) { return log2_chunks > 15 ? 0 : std::min(p.m, std::max(0, hist[log2_chunks])); };
  RowClasses rc;
  // class c: 16 >> c wavefronts; a row belongs to class c or an earlier one when it has more than (8 >> c) * rounds chunks
  rc.first_row[0] = 0;
  int before = 0;
  for (int c = 0; c < 4; ++c) {
    const int upto = std::max(before, rows_over(3 - c + r));   // rows with more than 64 << (3 - c + r) nonzeros
    rc.first_row[c + 1] = upto;
    before = upto;
  }
  rc.first_row[5] = p.m;
  rc.first_block[0] = 0;
  for (int c = 0; c < 5; ++c) rc.first_block[c + 1] = rc.first_block[c] + ceil_div(rc.first_row[c + 1] - rc.first_row[c], 1 << c);
  rc.log2_rounds = r;
  *rounds_out = 1 << r;
  return rc;
}

template <typename T, typename IT, int VEC, int LPG>
int launch_rows_one(const SpmmParams& p, int batch, const int* hist, int rounds_code, hipStream_t stream) {
  const int tiles = ceil_div(p.n, LPG * VEC);
  int rounds = 1;
  const RowClasses rc = row_classes(p, hist, tiles * batch, rounds_code, &rounds);
  note_kernel("spmm_rows_kernel<%s, %s, %d, %d> (rows by 16/8/4/2/1 waves: %d/%d/%d/%d/%d, %d chunks per wave)", type_name<T>(), type_name<IT>(), VEC, LPG,
              rc.first_row[1], rc.first_row[2] - rc.first_row[1], rc.first_row[3] - rc.first_row[2], rc.first_row[4] - rc.first_row[3],
              rc.first_row[5] - rc.first_row[4], rounds);
  hipLaunchKernelGGL((spmm_rows_kernel<T, IT, VEC, LPG>), dim3(rc.first_block[5], tiles, batch), dim3(kRowsWaves * kWave), 0, stream, p, rc);
  return check_hip(hipGetLastError(), "spmm (rows by length) launch");
}

template <typename T, typename IT>
int launch_rows(const SpmmParams& p, int batch, int lpg, const int* hist, int rounds_code, hipStream_t stream) {
  constexpr int kMax = 16 / (int)sizeof(T);
  switch (lpg) {
    case 8: return launch_rows_one<T, IT, kMax, 8>(p, batch, hist, rounds_code, stream);
    case 16: return launch_rows_one<T, IT, kMax, 16>(p, batch, hist, rounds_code, stream);
    case 32: return launch_rows_one<T, IT, kMax, 32>(p, batch, hist, rounds_code, stream);
    default: return launch_rows_one<T, IT, kMax, 64>(p, batch, hist, rounds_code, stream);
  }
}

// ---- LDS-staged variant -----------------------------------------------------------------
template <typename T, typename IT, int VEC, int RPW>
__global__ __launch_bounds__(kLdsThreads, 4) void spmm_lds_kernel(SpmmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  spmm_lds_block<T, IT, VEC, RPW>(p, blockIdx.x, blockIdx.y, blockIdx.z, smem);
}

template <typename T, typename IT, int VEC, int RPW>
int launch_lds_one(const SpmmParams& p, int batch, hipStream_t stream) {
  dim3 grid(ceil_div(p.m, kLdsWaves * RPW), ceil_div(p.n, kWave * VEC), batch);
  note_kernel("spmm_lds_kernel<%s, %s, %d, %d>", type_name<T>(), type_name<IT>(), VEC, RPW);
  hipLaunchKernelGGL((spmm_lds_kernel<T, IT, VEC, RPW>), grid, dim3(kLdsThreads), kLdsTileBytes, stream, p);
  return check_hip(hipGetLastError(), "spmm (LDS-staged) launch");
}

template <typename T, typename IT, int VEC>
int launch_lds_rpw(const SpmmParams& p, int batch, int rpw, hipStream_t stream) {
  switch (rpw) {
    case 2: return launch_lds_one<T, IT, VEC, 2>(p, batch, stream);
    case 4: return launch_lds_one<T, IT, VEC, 4>(p, batch, stream);
    case 8:
      // 8 rows x 8 accumulators per lane would spill at 4 waves per SIMD: 4 rows per wave then
      if constexpr (VEC < 8) return launch_lds_one<T, IT, VEC, 8>(p, batch, stream);
      else return launch_lds_one<T, IT, VEC, 4>(p, batch, stream);
  }
  return fail(IEX_ERR_BAD_ARGUMENT, "spmm: rows-per-wave of the LDS-staged variant must be 2, 4 or 8 (got %d)", rpw);
}

// ---- matrix-core variant (fp16 / bf16) ----------------------------------------------------
template <bool BF16, typename IT, int LPR>
__global__ __launch_bounds__(kMfmaThreads, 2) void spmm_mfma_kernel(SpmmParams p, int tiles_m) {
  extern __shared__ __align__(16) unsigned char smem[];
  // consecutive workgroups walk the row blocks of one column panel of the dense operand
  spmm_mfma_block<BF16, IT, LPR>(p, blockIdx.x % tiles_m, blockIdx.x / tiles_m, blockIdx.y, smem);
}

template <typename T, typename IT, int LPR>
int launch_mfma_one(const SpmmParams& p, int batch, hipStream_t stream) {
  constexpr bool kBf16 = std::is_same<T, __hip_bfloat16>::value;
  const int tiles_m = ceil_div(p.m, kMfmaBM), tiles_n = ceil_div(p.n, kMfmaBN);
  auto kernel = spmm_mfma_kernel<kBf16, IT, LPR>;
  static thread_local bool raised = false;  // more than 64 KB of dynamic LDS needs the attribute (per instantiation)
  if (!raised) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kMfmaLdsBytes),
                           "hipFuncSetAttribute(LDS size)"))
      return rc;
    raised = true;
  }
  note_kernel("spmm_mfma_kernel<%s, %s, %d>", kBf16 ? "true" : "false", type_name<IT>(), LPR);
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n, batch), dim3(kMfmaThreads), kMfmaLdsBytes, stream, p, tiles_m);
  return check_hip(hipGetLastError(), "spmm (matrix-core) launch");
}

template <typename T, typename IT>
int launch_mfma(const SpmmParams& p, int batch, int lpr, hipStream_t stream) {
  if constexpr (sizeof(T) == 2) {
    switch (lpr) {
      case 8: return launch_mfma_one<T, IT, 8>(p, batch, stream);
      case 16: return launch_mfma_one<T, IT, 16>(p, batch, stream);
    }
    return fail(IEX_ERR_BAD_ARGUMENT, "spmm: lanes-per-row of the matrix-core variant must be 8 or 16 (got %d)", lpr);
  } else {
    return fail(IEX_ERR_UNSUPPORTED, "spmm: the matrix-core variant handles fp16 and bf16 only");
  }
}

template <bool BF16, typename IT, int W, int BKA>
__global__ __launch_bounds__(kMfma2Threads, 2) void spmm_mfma2_kernel(SpmmParams p, int tiles_m) {
  extern __shared__ __align__(16) unsigned char smem[];
  spmm_mfma2_block<BF16, IT, W, BKA>(p, blockIdx.x % tiles_m, blockIdx.x / tiles_m, blockIdx.y, smem);
}

template <typename T, typename IT, int W, int BKA = 128>
int launch_mfma2_one(const SpmmParams& p, int batch, hipStream_t stream) {
  constexpr bool kBf16 = std::is_same<T, __hip_bfloat16>::value;
  constexpr int kMfma2LdsBytes = spmm_mfma2_lds_bytes<BKA>();
  const int tiles_m = ceil_div(p.m, kMfmaBM), tiles_n = ceil_div(p.n, kMfma2BN);
  auto kernel = spmm_mfma2_kernel<kBf16, IT, W, BKA>;
  static thread_local bool raised = false;
  if (!raised) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kMfma2LdsBytes),
                           "hipFuncSetAttribute(LDS size)"))
      return rc;
    raised = true;
  }
  note_kernel("spmm_mfma2_kernel<%s, %s, %d, %d>", kBf16 ? "true" : "false", type_name<IT>(), W, BKA);
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n, batch), dim3(kMfma2Threads), kMfma2LdsBytes, stream, p, tiles_m);
  return check_hip(hipGetLastError(), "spmm (matrix-core, 8 waves) launch");
}

template <typename T, typename IT>
int launch_mfma2(const SpmmParams& p, int batch, int windows, hipStream_t stream) {
  if constexpr (sizeof(T) == 2) {
    switch (windows) {
      case 1: return launch_mfma2_one<T, IT, 1>(p, batch, stream);
      case 2: return launch_mfma2_one<T, IT, 2>(p, batch, stream);
      case 4: return launch_mfma2_one<T, IT, 4>(p, batch, stream);
      case 5: return launch_mfma2_one<T, IT, 5>(p, batch, stream);
    }
    return fail(IEX_ERR_BAD_ARGUMENT, "spmm: windows of the matrix-core variant must be 1, 2, 4 or 5 (got %d)", windows);
  } else {
    return fail(IEX_ERR_UNSUPPORTED, "spmm: the matrix-core variant handles fp16 and bf16 only");
  }
}

template <bool BF16, typename IT, int W>
__global__ __launch_bounds__(kMfma3Threads, 2) void spmm_mfma3_kernel(SpmmParams p, int tiles_m) {
  extern __shared__ __align__(16) unsigned char smem[];
  spmm_mfma3_block<BF16, IT, W>(p, blockIdx.x % tiles_m, blockIdx.x / tiles_m, blockIdx.y, smem);
}

template <typename T, typename IT, int W>
int launch_mfma3_one(const SpmmParams& p, int batch, hipStream_t stream) {
  constexpr bool kBf16 = std::is_same<T, __hip_bfloat16>::value;
  const int tiles_m = ceil_div(p.m, kMfmaBM), tiles_n = ceil_div(p.n, kMfma3BN);
  auto kernel = spmm_mfma3_kernel<kBf16, IT, W>;
  static thread_local bool raised = false;
  if (!raised) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, spmm_mfma3_lds_bytes()),
                           "hipFuncSetAttribute(LDS size)"))
      return rc;
    raised = true;
  }
  note_kernel("spmm_mfma3_kernel<%s, %s, %d>", kBf16 ? "true" : "false", type_name<IT>(), W);
  hipLaunchKernelGGL(kernel, dim3(tiles_m * tiles_n, batch), dim3(kMfma3Threads), spmm_mfma3_lds_bytes(), stream, p, tiles_m);
  return check_hip(hipGetLastError(), "spmm (matrix-core, direct loads) launch");
}

template <typename T, typename IT>
int launch_mfma3(const SpmmParams& p, int batch, int windows, hipStream_t stream) {
  if constexpr (sizeof(T) == 2) {
    if (windows == 1) return launch_mfma3_one<T, IT, 1>(p, batch, stream);
    if (windows == 2) return launch_mfma3_one<T, IT, 2>(p, batch, stream);
    if (windows == 4) return launch_mfma3_one<T, IT, 4>(p, batch, stream);
    return fail(IEX_ERR_BAD_ARGUMENT, "spmm: windows of the direct-load matrix-core variant must be 1, 2 or 4 (got %d)", windows);
  } else {
    return fail(IEX_ERR_UNSUPPORTED, "spmm: the matrix-core variant handles fp16 and bf16 only");
  }
}

// ---- matrix-core variant, fp32 ---------------------------------------------------------------
// arrangement code = MFMA tile height and how the 4 multiplying waves split the C tile:
//   1 = 32 x 64 (4 k slices)    2 = 32 x 128 as 2 x 64 columns (2 k slices)    4 = 32 x 128 (4 k slices)
//   5 = 16 x 64 (4 k slices)    6 = 16 x 128 as 2 x 64 columns (2 k slices)
template <int MT, int NJ, int WAVES_N, int W, bool SPLIT>
__global__ __launch_bounds__(kF32Threads + (SPLIT ? MT * 8 : 0), 2) void spmm_mfma_f32_kernel(SpmmParams p, int tiles_m) {
  extern __shared__ __align__(16) unsigned char smem[];
  spmm_mfma_f32_block<MT, NJ, WAVES_N, W, SPLIT>(p, blockIdx.x % tiles_m, blockIdx.x / tiles_m, blockIdx.y, smem);
}

template <int MT, int NJ, int WAVES_N, int W, bool SPLIT>
int launch_mfma_f32_one(const SpmmParams& p, int batch, hipStream_t stream) {
  constexpr int kBN = MT * NJ * WAVES_N;
  const int tiles_m = ceil_div(p.m, MT), tiles_n = ceil_div(p.n, kBN);
  constexpr int kLds = spmm_mfma_f32_lds_bytes<MT, NJ, WAVES_N>();
  note_kernel("spmm_mfma_f32_kernel<%d, %d, %d, %d, %s>", MT, NJ, WAVES_N, W, SPLIT ? "true" : "false");
  hipLaunchKernelGGL((spmm_mfma_f32_kernel<MT, NJ, WAVES_N, W, SPLIT>), dim3(tiles_m * tiles_n, batch),
                     dim3(kF32Threads + (SPLIT ? MT * 8 : 0)), kLds, stream, p, tiles_m);
  return check_hip(hipGetLastError(), "spmm (matrix-core, fp32) launch");
}

template <int MT, int NJ, int WAVES_N>
int launch_mfma_f32_w(const SpmmParams& p, int batch, int windows, bool split, hipStream_t stream) {
  // with separate expanding waves there are registers for 16 windows (the kernel uses as many
  // of them as the rows of a wave need); waves that do both hold 2, 4 or 8
  if (split) return launch_mfma_f32_one<MT, NJ, WAVES_N, 16, true>(p, batch, stream);
  switch (windows) {
    case 2: return launch_mfma_f32_one<MT, NJ, WAVES_N, 2, false>(p, batch, stream);
    case 4: return launch_mfma_f32_one<MT, NJ, WAVES_N, 4, false>(p, batch, stream);
    case 8: return launch_mfma_f32_one<MT, NJ, WAVES_N, 8, false>(p, batch, stream);
  }
  return fail(IEX_ERR_BAD_ARGUMENT, "spmm: windows of the fp32 matrix-core variant must be 2, 4 or 8 (got %d)", windows);
}

inline int launch_mfma_f32(const SpmmParams& p, int batch, int arrangement, int windows, bool split, hipStream_t stream) {
  switch (arrangement) {
    case 1: return launch_mfma_f32_w<32, 2, 1>(p, batch, windows, split, stream);
    case 2: return launch_mfma_f32_w<32, 2, 2>(p, batch, windows, split, stream);
    case 4: return launch_mfma_f32_w<32, 4, 1>(p, batch, windows, split, stream);
    case 5: return launch_mfma_f32_w<16, 4, 1>(p, batch, windows, split, stream);
    case 6: return launch_mfma_f32_w<16, 4, 2>(p, batch, windows, split, stream);
  }
  return fail(IEX_ERR_BAD_ARGUMENT, "spmm: arrangement of the fp32 matrix-core variant must be 1, 2, 4, 5 or 6 (got %d)", arrangement);
}

struct Choice {
  int wpr = 0;      // wavefronts per row of the row kernel
  bool wpr_forced = false;
  int variant = 0;  // 0 = choose, 1 = row kernel, 2 = LDS-staged kernel, 3 / 4 = matrix-core kernels (16-bit), 5 = (fp32)
  int rpw = 0;      // rows per wavefront of the LDS-staged kernel (0 = choose)
  int nt = 0;       // adjacent column tiles per wavefront of the row kernel (0 = choose)
  int lpg = 0;      // lanes per nonzero of the row kernel: 8, 16, 32 or 64 (0 = choose)
  void* ws = nullptr;   // caller's workspace for the dense form of A (variant 7), may be null
  size_t ws_bytes = 0;
  bool any_order = false;   // columns of a row in any order, possibly repeated: families 1 and 8 only
  const int* hist = nullptr;   // host: rows with more than 64 << j nonzeros, j = 0 .. 15 (iex_spmm_sched), may be null
  bool beside_gather = false;  // the launch shares the chip with a gather-bound one (IEX_SPMM_BESIDE_GATHER_KERNEL)
};

// The LDS-staged kernel needs a full-width tile (64 lanes x VEC, VEC the full or half 128-bit
// vector) and pays off when the rows of a workgroup share dense rows often enough:
// gathers saved per dense row staged = density * rows per workgroup.
template <typename T>
bool lds_variant(const SpmmParams& p, int batch, const Choice& ch, int& vec, int& rpw) {
  constexpr int kMax = 16 / (int)sizeof(T);
  vec = kMax;
  auto fits = [&](int v) {
    return p.n % v == 0 && kWave * v <= p.n && aligned(p.dense, sizeof(T) * v) && aligned(p.out, sizeof(T) * v);
  };
  if (!fits(vec)) vec = kMax / 2;
  if (!fits(vec)) return false;
  const long long tiles = (long long)ceil_div(p.n, kWave * vec) * batch;
  rpw = ch.rpw;
  if (rpw == 0) {
    rpw = 8;  // largest rows-per-wave that still gives every CU two workgroups
    while (rpw > 2 && (long long)ceil_div(p.m, kLdsWaves * rpw) * tiles < 512) rpw >>= 1;
  }
  if (ch.variant == 2) return true;
  if (ch.variant == 1) return false;
  // Measured on MI355X: the staged kernel wins when the rows of a workgroup reuse a staged
  // dense row a dozen times or more (2:4 weights: 4.5 -> 3.6 ms at 4096x4096, n = 8192), and
  // from a reuse of 4 when the slice of the dense operand one column tile touches (k rows of
  // a 64-lane tile) outgrows an XCD's 4 MB L2 (k = 11008: 10.8 -> 4.9 ms).  It loses on small
  // problems (fewer than two workgroups per CU: per-stage barriers expose row-length imbalance)
  // and at low reuse (90 % sparsity: 0.67 -> 0.90 ms).
  const double density = (p.m > 0 && p.k > 0) ? (double)p.nnz / ((double)p.m * p.k) : 0.0;
  const int eff_rpw = (vec * (int)sizeof(T) == 16 && sizeof(T) == 2 && rpw == 8) ? 4 : rpw;
  const double reuse = density * kLdsWaves * eff_rpw;
  const long long groups = (long long)ceil_div(p.m, kLdsWaves * eff_rpw) * tiles;
  const double slice_bytes = (double)p.k * kWave * vec * sizeof(T);
  if (groups < 512) return false;
  return reuse >= 12.0 || (slice_bytes > 6.0 * 1024 * 1024 && reuse >= 4.0);
}

// The matrix-core kernels: 16-bit types, n a multiple of 8, 16-byte aligned dense operands,
// k < 65535 for the 8-wave arrangement (packed columns).  Sets kind = 3 (4 waves, 128 x 256
// tiles; param = lanes per row) or 4 (8 waves, 128 x 512 tiles; param = windows per row);
// kind 0 = use a gather kernel.
// nothing about the row kernel's waves per row was asked for
inline bool flags_wpr_free(const Choice& ch) { return !ch.wpr_forced && (ch.variant == 0 || ch.variant == 1); }

struct MfmaChoice {
  int kind = 0, param = 0;
};

template <typename T>
MfmaChoice mfma_variant(const SpmmParams& p, int batch, const Choice& ch) {
  MfmaChoice mc;
  if (sizeof(T) != 2 || (ch.variant != 0 && ch.variant != 3 && ch.variant != 4)) return mc;
  if (!(p.nnz > 0 && p.n % 8 == 0 && aligned(p.dense, 16) && aligned(p.out, 16))) return mc;  // (also when forced)
  const double density = (p.m > 0 && p.k > 0) ? (double)p.nnz / ((double)p.m * p.k) : 0.0;
  const double run = density * kMfmaBKA;  // nonzeros of a row per 128-column chunk
  const bool wide_ok = p.k < 65535;
  const long long tiles_m = ceil_div(p.m, kMfmaBM);
  const long long wgs_wide = tiles_m * ceil_div(p.n, kMfma2BN) * batch;
  const long long wgs_narrow = tiles_m * ceil_div(p.n, kMfmaBN) * batch;
  int kind = ch.variant;
  if (kind == 0) {
    // Measured on MI355X (fp16, m x k = 11008 x 4096, n = 2048): the gather kernels and the
    // matrix-core kernels meet at about 5 % density (0.34 vs 0.32 ms); at 10 % the matrix cores
    // are 1.7x faster, at 50 % (4096 x 4096, n = 8192) 7x; at 2 % the gather kernel is 2x faster.
    // Small outputs (a handful of tiles) leave most CUs idle and stay with the gather kernels.
    // A tile computes all of its 256 / 512 columns: an n that fills less than three quarters of
    // its tiles wastes the difference (n = 64 on 512-column tiles measured 3.5x slower than the
    // gather kernel).
    if (density < 0.05) return mc;
    const double fill_wide = (double)p.n / ((double)ceil_div(p.n, kMfma2BN) * kMfma2BN);
    const double fill_narrow = (double)p.n / ((double)ceil_div(p.n, kMfmaBN) * kMfmaBN);
    if (wide_ok && wgs_wide >= 128 && fill_wide >= 0.75) kind = 4;
    else if (wgs_narrow >= 128 && fill_narrow >= 0.75) kind = 3;
    else return mc;
  }
  if (kind == 4 && !wide_ok) kind = 3;
  mc.kind = kind;
  if (kind == 3) mc.param = ch.lpg ? ch.lpg : (run > 24.0 ? 16 : 8);
  // windows of 16 nonzeros per row: enough for the run of a chunk (2:4 rows have exactly 64 per
  // chunk and need the fifth, or every row-visit would make one exposed pass to find nothing)
  else mc.param = ch.rpw ? ch.rpw : (run > 56.0 ? 5 : run > 20.0 ? 4 : run > 8.0 ? 2 : 1);
  return mc;
}

// fp32 on the matrix cores: int32 indices, n a multiple of 4, 16-byte aligned dense operands.
// Returns the arrangement code (0 = use a gather kernel) and sets the number of register windows.
template <typename T, typename IT>
int mfma_f32_variant(const SpmmParams& p, int batch, const Choice& ch, int& windows) {
  if (!std::is_same<T, float>::value || !std::is_same<IT, int>::value) return 0;
  if (ch.variant != 0 && ch.variant != 5) return 0;
  if (!(p.nnz > 0 && p.n % 4 == 0 && aligned(p.dense, 16) && aligned(p.out, 16))) return 0;  // (also when forced)
  const double density = (p.m > 0 && p.k > 0) ? (double)p.nnz / ((double)p.m * p.k) : 0.0;
  // 32-row tiles with 128 columns per wave when that still gives most CUs a workgroup; else
  // 16-row tiles (twice the workgroups, twice the reads of the dense operand)
  const long long tiles_m = ceil_div(p.m, 32);
  int arrangement = tiles_m * ceil_div(p.n, 128) * batch >= 200 ? 4 : (p.n <= 64 ? 5 : 6);
  if (ch.nt) arrangement = ch.nt;
  const double run = density * 128;  // nonzeros of a row per chunk
  windows = ch.rpw ? ch.rpw : (run <= 12.0 ? 2 : run <= 40.0 ? 4 : 8);
  if (ch.variant == 5) return arrangement;
  // Measured on MI355X: 70-105 dense-equivalent TFLOP/s (the fp32 MFMA rate is 153; fp32 MFMAs
  // run on the vector ALUs, so the expansion's instructions add to their time instead of hiding
  // behind them).  That beats the gather kernels from 25-30 % density (4096 x 4096 at 50 %,
  // n = 8192: 5.0 -> 2.9 ms; at 30 %, n = 1024: 0.69 -> 0.38 ms; at 30 %, n = 256: 0.19 -> 0.13 ms),
  // ties at 20 % and loses below (11008 x 4096 at 20 %: 6.6 vs 7.3 ms).  The 16-row arrangements
  // for small outputs stay on request: at 30 % and n = 128 they only tie (0.096 vs 0.100 ms).
  const double fill = (double)p.n / ((double)ceil_div(p.n, 128) * 128);  // share of the computed columns that exist
  if (density >= 0.27 && arrangement == 4 && fill >= 0.75) return arrangement;
  // Beside a kernel that is bound by gathers the tie at 20 % goes to the matrix cores, also with the 16-row tiles of
  // n = 128: alone 124 against 118 us (4096 x 4096 at 20 %, n = 256) and 90 against 84 us (30 %, n = 128), but the
  // neighbour then has the L2 -> CU path to itself (the 15 cells of that sweep on two branches of a graph: 654 -> 600 us).
  if (ch.beside_gather && density >= 0.195 && p.n >= 128 && fill >= 0.75) return arrangement;
  return 0;
}

// Windows of 16 nonzeros per row and half chunk of 64 columns for the direct-load matrix-core
// kernel.  One window holds a row's share with a margin of three standard deviations up to 13 %
// density (mean 8.3 of 64), two up to 33 % (mean 21) and exactly at 2:4 sparsity (32 of every 64,
// recognised by nnz being exactly half of m * k); four always do.  A half chunk the windows do not
// hold is multiplied twice, so a wrong guess costs time, not correctness.
inline int mfma3_windows(const SpmmParams& p) {
  const double cells = (double)p.m * p.k;
  const double density = cells > 0 ? (double)p.nnz / cells : 0.0;
  if (density <= 0.13) return 1;
  return (density <= 0.33 || 2.0 * p.nnz == cells) ? 2 : 4;
}

// Dense form of A in the caller's workspace, then the dense GEMM (16-bit types, values shared by
// the batch, plain store, no bias / ReLU).  What the shapes must satisfy, the workspace aside.
inline bool dense_path_fits(int elem_size, const SpmmParams& p, bool flagged) {
  return elem_size == 2 && !flagged && p.nnz > 0 && p.k % 8 == 0 && p.n % 8 == 0 &&
         (long long)p.m * p.k < (1ll << 31) && aligned(p.dense, 16) && aligned(p.out, 16);
}

inline size_t dense_path_bytes(const SpmmParams& p) { return (size_t)p.m * p.k * 2; }

// Whether the dense-form path is the faster one, from a time model fitted on MI355X (fp16):
//   dense form + GEMM: two launches (8 us), m * k * 2 bytes written at 4 TB/s, the product at
//     1000 TFLOP/s or, when the tiles are few, one round of 128 x 128 tiles per 512 tiles at 0.23 us
//     per K step of 32 (4096^2, n <= 512: 40-45 us whatever the sparsity; 1024^2, n = 2048: 21 us);
//   matrix-core SpMM kernels: 720 dense-equivalent TFLOP/s (2:4 4096^2, n = 8192: 0.40 against 0.27 ms
//     for the dense form; 80 % 11008 x 4096: 0.93 / 0.69; 90 %, n = 2048: 0.27 / 0.23);
//   gather kernels: nnz * n * 2 bytes through the L2 -> CU path at 26 TB/s (4096^2 at 70 %, n = 256:
//     110 against 58 us; at 90 %, n = 256: 40 against 58; 11008 x 4096 at 95 %, n = 2048: 0.35 / 0.21 ms).
//   a short K makes the GEMM a writer of its output at 3 TB/s (16 x 4096 x 4096, k = 64: 0.18 ms) and the
//     matrix-core SpMM kernels at 1.2 TB/s (8 x 4096 x 4096, k = 128: 0.24 ms), the gather kernels write it at 4 TB/s, the few-columns kernel at 4.5 TB/s plus 10 clocks of a CU's LDS
//     per nonzero and tile (same shape at 93 % sparsity: 0.15 ms; 8 x 4096 x 4096, k = 128 at 50 %: 0.58
//     against 0.17 for the dense form).
// The dense form has to win by 15 % to be taken.  `few_columns`: the alternative is the few-columns kernel.
// split_room: the workspace has room for the GEMM to take k in parts where it would (few tiles, long k: the K loop of a
// tile then runs on several CUs; 4096^2 at 70-90 %, n = 128 / 256: 40 / 41 -> 27 / 32 us).
inline bool dense_path_wins(const SpmmParams& p, int batch, int matrix_core_kind, bool few_columns, bool split_room = true) {
  const double cells = (double)p.m * p.k, flops = 2.0 * cells * p.n * batch;
  const double out_bytes = (double)p.m * p.n * batch * 2;
  const double tiles = (double)ceil_div(p.m, 128) * ceil_div(p.n, 128) * batch;
  const int parts = split_room && !p.accumulate ? gemm_auto_split_parts(p.m, p.n, p.k, batch) : 1;
  const double product = std::max({flops / 1000e12, std::ceil(tiles / 512.0) * (p.k / 32.0) * 0.23e-6 / parts, out_bytes / 3e12});
  const double dense_form = 8e-6 + cells * 2 / 4e12 + product;
  double other;
  if (few_columns) other = 8e-6 + out_bytes / 4.5e12 + (double)p.nnz * batch * ceil_div(p.n, 512) * 10.0 / (256 * 2.1e9);
  else if (matrix_core_kind) other = 8e-6 + std::max(flops / 720e12, out_bytes / 1.2e12);
  else other = 8e-6 + (double)p.nnz * p.n * batch * 2 / 26e12 + out_bytes / 4e12;
  return 1.15 * dense_form < other;
}

// Behind the dense form (rounded up to 256 bytes) the workspace may hold what the GEMM wants for splitting K over two
// workgroups per tile (few tiles, long k: gemm_auto_split_bytes); the words it wants zero are zeroed by the kernel
// that writes the dense form.
inline size_t dense_path_split_offset(const SpmmParams& p) { return (dense_path_bytes(p) + 255) & ~size_t(255); }
inline size_t dense_path_split_bytes(const SpmmParams& p, int batch) { return p.accumulate ? 0 : gemm_auto_split_bytes(p.m, p.n, p.k, batch); }

inline bool dense_path_has_split_room(const SpmmParams& p, int batch, const Choice& ch) {
  const size_t split = dense_path_split_bytes(p, batch);
  return split > 0 && ch.ws && aligned(ch.ws, 256) && ch.ws_bytes >= dense_path_split_offset(p) + split;
}

template <typename T, typename IT>
int launch_dense_path(const SpmmParams& p, int batch, const Choice& ch, hipStream_t stream) {
  const size_t split = dense_path_split_bytes(p, batch), offset = dense_path_split_offset(p);
  const bool with_split = dense_path_has_split_room(p, batch, ch);
  unsigned char* split_ws = with_split ? static_cast<unsigned char*>(ch.ws) + offset : nullptr;
  size_t flags_at = 0;
  int flag_words = 0;
  if (with_split) gemm_auto_split_flags(p.m, p.n, p.k, batch, &flags_at, &flag_words);
  note_kernel("csr_to_dense_kernel<%s>", type_name<IT>());
  hipLaunchKernelGGL((csr_to_dense_kernel<IT>), dim3(ceil_div(p.m, kDenseRows)), dim3(kDenseThreads), 0, stream, p.m, p.k,
                     p.row_offsets, static_cast<const IT*>(p.cols), static_cast<const uint16_t*>(p.values),
                     static_cast<uint16_t*>(ch.ws), with_split ? reinterpret_cast<int*>(split_ws + flags_at) : nullptr, flag_words);
  if (int rc = check_hip(hipGetLastError(), "spmm dense-form launch")) return rc;
  const int dtype = std::is_same<T, __half>::value ? IEX_F16 : IEX_BF16;
  return gemm_dispatch(dtype, 0, p.m, p.n, p.k, ch.ws, p.dense, p.out, batch, 0, (long long)p.k * p.n, (long long)p.m * p.n, stream,
                       p.bias, p.relu, p.accumulate, split_ws, with_split ? split : 0, with_split);
}

template <typename T, typename IT>
int launch_typed(const SpmmParams& p, int batch, const Choice& given, hipStream_t stream) {
  constexpr int kMax = 16 / (int)sizeof(T);
  Choice ch = given;
  // Columns in any order: the few-columns kernel where it applies (it takes nonzeros as they come), else the row kernel.
  if (ch.any_order && ch.variant == 0) {
    if (smallk_wanted<T>(p, batch)) return launch_smallk<T, IT>(p, batch, stream);
    ch.variant = 1;
  }
  // A with few columns and rows that gather, wide output: the tile of the dense operand in LDS, rows
  // streamed (spmm_smallk_device.cuh; smallk_wanted has the measurements).  16-bit products that are
  // dense enough go to the dense-form path first (time model above).
  if (ch.variant == 0 && smallk_wanted<T>(p, batch)) {
    if constexpr (sizeof(T) == 2) {
      const bool room = ch.ws && aligned(ch.ws, 16) && ch.ws_bytes >= dense_path_bytes(p);
      if (room && dense_path_fits(2, p, p.per_batch_values) && dense_path_wins(p, batch, 0, true, dense_path_has_split_room(p, batch, ch)))
        return launch_dense_path<T, IT>(p, batch, ch, stream);
    }
    return launch_smallk<T, IT>(p, batch, stream);
  }
  if constexpr (std::is_same<T, float>::value && std::is_same<IT, int>::value) {
    int windows = 0;
    if (const int arr = mfma_f32_variant<T, IT>(p, batch, ch, windows)) return launch_mfma_f32(p, batch, arr, windows, ch.lpg != 8, stream);  // (lanes-per-group code 8 = no role split, for tuning)
  }
  if (ch.variant == 6 && sizeof(T) == 2 && p.nnz > 0 && p.n % 8 == 0 && aligned(p.dense, 16) && aligned(p.out, 16))
    return launch_mfma3<T, IT>(p, batch, ch.rpw ? ch.rpw : mfma3_windows(p), stream);
  const MfmaChoice mc = mfma_variant<T>(p, batch, ch);
  if constexpr (sizeof(T) == 2) {
    const bool fits = dense_path_fits(2, p, p.per_batch_values);
    const bool room = ch.ws && aligned(ch.ws, 16) && ch.ws_bytes >= dense_path_bytes(p);
    if (ch.variant == 7) {
      IEX_REQUIRE(fits, IEX_ERR_UNSUPPORTED, "spmm: the dense-form path needs 16-bit values shared by the batch, k and n multiples of 8 and 16-byte aligned operands");
      IEX_REQUIRE(room, IEX_ERR_BAD_ARGUMENT, "spmm: the dense-form path needs a 16-byte aligned workspace of %zu bytes (iex_spmm_ws)", dense_path_bytes(p));
      return launch_dense_path<T, IT>(p, batch, ch, stream);
    }
    if (ch.variant == 0 && fits && room && dense_path_wins(p, batch, mc.kind, false, dense_path_has_split_room(p, batch, ch))) return launch_dense_path<T, IT>(p, batch, ch, stream);
  }
  // Where the 8-wave kernel would run: the direct-load kernel wins on 2:4 weights (4096 x 4096,
  // n = 8192: 0.37 against 0.40-0.46 ms with five windows), ties at 80 % sparsity (11008 x 4096:
  // 0.94 against 0.93; 4096 x 11008: 0.82 both) and loses at 90 % (n = 2048: 0.29 against 0.26);
  // with four windows (denser than 33 %, not 2:4) it spills registers.
  if (mc.kind == 4 && ch.variant == 0 && 2.0 * p.nnz == (double)p.m * p.k) return launch_mfma3<T, IT>(p, batch, 2, stream);
  if (mc.kind == 4) return launch_mfma2<T, IT>(p, batch, mc.param, stream);
  if (mc.kind == 3) return launch_mfma<T, IT>(p, batch, mc.param, stream);
  if (ch.variant == 8) {
    IEX_REQUIRE(smallk_fits<T>(p), IEX_ERR_UNSUPPORTED, "spmm: the few-columns kernel needs k <= %d and an output at least one tile (64 128-bit vectors) wide", kSmallKMax);
    return launch_smallk<T, IT>(p, batch, stream);
  }
  int lvec = 0, rpw = 0;
  if (ch.variant != 11 && lds_variant<T>(p, batch, ch, lvec, rpw)) {
    if (lvec == kMax) return launch_lds_rpw<T, IT, kMax>(p, batch, rpw, stream);
    return launch_lds_rpw<T, IT, kMax / 2>(p, batch, rpw, stream);
  }
  const int wpr = ch.wpr;
  SpmmShape sh = spmm_pick_shape<T>(p.n, p.dense, p.out);
  if (ch.lpg && sh.vec == kMax && ch.lpg <= sh.lpg) sh.lpg = ch.lpg;  // narrower tiles on request
  // The caller knows the pattern's row lengths: wavefronts per row by the row's own length instead of one number for
  // the whole matrix.  Measured on MI355X (fp32, 4096 x 4096, geometric row lengths, us, four waves for every row /
  // this kernel at its best chunks-per-wave): 98 % sparse n = 64 9.0 / 7.6, n = 128 12.5 / 11.2, n = 256 17.2 / 20.0;
  // 95 % 12.7 / 13.9, 19.7 / 22.3, 36.9 / 39.2; 90 % 19.1 / 22.0, 36.7 / 38.6, 69.4 / 67.0; 80 % 33 / 42, 59 / 73,
  // 119 / 122.  The row kernel is bound by the gathers' way from L2 into the CUs (20-26 TB/s on every n = 256
  // cell), not by its longest rows: four waves on every row keep more gathers in flight than a schedule that gives short
  // rows one wave, and that wins wherever the chip is full.  So this kernel is taken where it is not: fewer chunks
  // of 64 nonzeros than the chip holds wavefronts, and narrow tiles (several nonzeros per gather instruction).
  if (ch.variant == 11) IEX_REQUIRE(ch.hist && sh.vec == kMax, IEX_ERR_BAD_ARGUMENT, "spmm: the rows-by-length kernel needs the row-length histogram (iex_spmm_sched) and full 128-bit vectors");
  const double chunk_count = (double)p.nnz / kWave * ceil_div(p.n, sh.lpg * sh.vec) * batch;
  if (ch.hist && sh.vec == kMax && ch.nt <= 1 &&
      (ch.variant == 11 || (flags_wpr_free(ch) && ch.hist[0] > 0 && wpr != 1 && sh.lpg <= 32 && chunk_count <= 8192.0)))
    return launch_rows<T, IT>(p, batch, sh.lpg, ch.hist, ch.variant == 11 ? ch.rpw : 0, stream);
  // Two tiles per wave double the slice of the dense operand that the waves of an XCD share in
  // its L2 and measured slower (2x at k = 4096, n = 8192): only on request.
  const int nt = ch.nt ? ch.nt : 1;
  if (sh.vec == kMax) {
    switch (sh.lpg) {
      case 8: return launch_wpr<T, IT, kMax, 8>(p, batch, wpr, nt, stream);
      case 16: return launch_wpr<T, IT, kMax, 16>(p, batch, wpr, nt, stream);
      case 32: return launch_wpr<T, IT, kMax, 32>(p, batch, wpr, nt, stream);
      default: return launch_wpr<T, IT, kMax, 64>(p, batch, wpr, nt, stream);
    }
  }
  // Rows whose length is not a multiple of the 128-bit vector (n = 785, 197 of the ViT shapes), at least
  // half a tile wide: 128-bit accesses at element alignment instead of narrower vectors.  Measured on
  // the reference's ViT sweep shapes (fp32, batch 384, 97 % sparse): 785 x 785 outputs 865 -> 516 us,
  // 197 x 197 outputs 64 -> 33 us.
  if (p.n % kMax != 0 && p.n >= kWave * kMax / 2 && ch.lpg == 0) return launch_ragged<T, IT, kMax>(p, batch, wpr, stream);
  if constexpr (kMax == 8) {
    if (sh.vec == 4) return launch_wpr<T, IT, 4, 64>(p, batch, wpr, nt, stream);
  }
  if (sh.vec == 2) return launch_wpr<T, IT, 2, 64>(p, batch, wpr, nt, stream);
  return launch_wpr<T, IT, 1, 64>(p, batch, wpr, nt, stream);
}

}  // namespace

// For the fused launcher: the number of register windows if the dispatcher would run this
// fp16 SpMM (one batch entry, nothing forced) on the 8-wave matrix-core kernel, else 0.
int spmm_matrix_core_windows(const SpmmParams& p) {
  const MfmaChoice mc = mfma_variant<__half>(p, 1, Choice{});
  return mc.kind == 4 ? mc.param : 0;
}

int spmm_dispatch(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                  const int* row_indices, const void* values, const int* row_offsets,
                  const void* column_indices, const void* dense, const float* bias, void* out,
                  void* stream, int batch, void* workspace, size_t workspace_bytes, const int* row_histogram = nullptr) {
  IEX_REQUIRE(m >= 0 && k >= 0 && n >= 0 && nonzeros >= 0 && batch >= 0, IEX_ERR_BAD_ARGUMENT,
              "spmm: negative dimension (m=%d k=%d n=%d nnz=%d batch=%d)", m, k, n, nonzeros, batch);
  trail_reset();
  if (m == 0 || n == 0 || batch == 0) return 0;  // empty output: nothing to launch
  IEX_REQUIRE(row_indices && row_offsets && dense && out, IEX_ERR_BAD_ARGUMENT,
              "spmm: null pointer argument");
  IEX_REQUIRE(nonzeros == 0 || (values && column_indices), IEX_ERR_BAD_ARGUMENT,
              "spmm: null values / column_indices with nnz=%d", nonzeros);
  IEX_REQUIRE(batch <= 65535, IEX_ERR_TOO_LARGE, "spmm: batch %d exceeds 65535", batch);
  IEX_REQUIRE((long long)k * n < (1ll << 31) && (long long)m * n < (1ll << 31), IEX_ERR_TOO_LARGE,
              "spmm: a dense operand exceeds 2^31 elements per batch entry");
  IEX_REQUIRE(itype == IEX_I32 || (itype == IEX_I16 && k <= 32768), IEX_ERR_BAD_ARGUMENT,
              "spmm: int16 column indices need k <= 32768 (k=%d)", k);
  Choice ch;
  ch.wpr = (flags >> 8) & 0xff;
  ch.wpr_forced = ch.wpr != 0;
  if (ch.wpr == 0) ch.wpr = spmm_pick_wpr(m, nonzeros, dtype == IEX_F32 ? 4 : 2, n, batch);
  ch.hist = row_histogram;
  ch.variant = (flags >> 16) & 0xf;
  ch.rpw = (flags >> 20) & 0xf;
  ch.nt = (flags >> 24) & 0xf;
  ch.lpg = ((flags >> 28) & 0x7) ? (4 << ((flags >> 28) & 0x7)) : 0;
  ch.ws = workspace;
  ch.ws_bytes = workspace ? workspace_bytes : 0;
  ch.any_order = (flags & IEX_SPMM_ANY_COLUMN_ORDER) != 0;
  ch.beside_gather = (flags & IEX_SPMM_BESIDE_GATHER_KERNEL) != 0 && !ch.any_order;
  SpmmParams p{m, k, n, nonzeros, row_indices, values, row_offsets, column_indices, dense, bias, out,
               (flags & IEX_SPMM_PER_BATCH_VALUES) != 0, (flags & IEX_SPMM_ACCUMULATE) != 0,
               (flags & IEX_SPMM_RELU) != 0};
  // beyond the 256 MB last-level cache an output can only stream; the hint is worth 15-25 % of the write rate
  p.stream_out = (double)m * n * batch * (dtype == IEX_F32 ? 4 : 2) >= 128e6;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (ch.variant == 10 && nonzeros < 8) {   // (its loads of eight values at a time need eight to exist: the row kernel instead)
    ch.variant = 1;
    ch.wpr = spmm_pick_wpr(m, nonzeros, dtype == IEX_F32 ? 4 : 2, n, batch);   // (bits 8..15 meant the dense-block threshold)
    ch.wpr_forced = false;
  }
  const int blocks_ready = ((flags & IEX_SPMM_TABLES_READY) ? 1 : 0) | ((flags & IEX_SPMM_LISTS_READY) ? 2 : 0);
  if (ch.variant == 0 && !ch.any_order && ch.ws && aligned(ch.ws, 16) && spmm_blocks_fits(dtype, itype, p) && spmm_blocks_wins(p, batch) &&
      ch.ws_bytes >= spmm_blocks_bytes(p))
    return launch_spmm_blocks(dtype, p, batch, ch.ws, 0, blocks_ready, s);
  if (ch.variant == 10) {
    IEX_REQUIRE(spmm_blocks_fits(dtype, itype, p), IEX_ERR_UNSUPPORTED,
                "spmm: the dense-blocks kernel needs fp16 / bf16, int32 indices, n a multiple of 64 up to 1024, plain store without bias or ReLU, k <= 65536 and 16-byte aligned dense operands");
    IEX_REQUIRE(ch.ws && aligned(ch.ws, 16) && ch.ws_bytes >= spmm_blocks_bytes(p), IEX_ERR_BAD_ARGUMENT,
                "spmm: the dense-blocks kernel needs a 16-byte aligned workspace of %zu bytes (iex_spmm_ws)", spmm_blocks_bytes(p));
    return launch_spmm_blocks(dtype, p, batch, ch.ws, (flags >> 8) & 0xff, blocks_ready, s);
  }
  if (dtype == IEX_F32 && itype == IEX_I32) return launch_typed<float, int>(p, batch, ch, s);
  if (dtype == IEX_F16 && itype == IEX_I32) return launch_typed<__half, int>(p, batch, ch, s);
  if (dtype == IEX_F16 && itype == IEX_I16) return launch_typed<__half, short>(p, batch, ch, s);
  if (dtype == IEX_BF16 && itype == IEX_I32) return launch_typed<__hip_bfloat16, int>(p, batch, ch, s);
  return fail(IEX_ERR_UNSUPPORTED, "spmm: no kernel for dtype=%d itype=%d", dtype, itype);
}

// Bytes of workspace with which iex_spmm_ws would take the dense-form path for this call (0: it
// would not, whatever the workspace).  Pointers are taken to be 16-byte aligned.
// kind: which family the workspace would serve (0 = none, 7 = dense form, 9 = partial sums of the k split, 10 = the
// tables and lists of the dense-blocks kernel).
static size_t workspace_plan(int dtype, int itype, int flags, int m, int k, int n, int nonzeros, int batch, int* kind) {
  *kind = 0;
  if (m <= 0 || k <= 0 || n <= 0 || nonzeros <= 0 || batch <= 0) return 0;
  const int variant = (flags >> 16) & 0xf;
  if (variant == 0 && (flags & IEX_SPMM_ANY_COLUMN_ORDER)) return 0;   // families 1 and 8 use no workspace
  void* const some_aligned = reinterpret_cast<void*>(size_t(256));
  if (!(dtype == IEX_F16 || dtype == IEX_BF16) || !(itype == IEX_I32 || itype == IEX_I16)) return 0;
  if (variant != 0 && variant != 7 && variant != 10) return 0;
  SpmmParams p{m, k, n, nonzeros, nullptr, nullptr, nullptr, nullptr, some_aligned, nullptr, some_aligned,
               (flags & IEX_SPMM_PER_BATCH_VALUES) != 0, (flags & IEX_SPMM_ACCUMULATE) != 0, (flags & IEX_SPMM_RELU) != 0};
  if (variant != 7 && nonzeros >= 8 && spmm_blocks_fits(dtype, itype, p) && (variant == 10 || spmm_blocks_wins(p, batch))) {
    *kind = 10;
    return spmm_blocks_bytes(p);
  }
  if (variant == 10) return 0;
  if (!dense_path_fits(2, p, (flags & IEX_SPMM_PER_BATCH_VALUES) != 0)) return 0;
  if (variant == 0) {
    Choice ch;
    ch.rpw = (flags >> 20) & 0xf;
    ch.lpg = ((flags >> 28) & 0x7) ? (4 << ((flags >> 28) & 0x7)) : 0;
    const bool few = smallk_wanted<__half>(p, batch);
    if (!dense_path_wins(p, batch, few ? 0 : mfma_variant<__half>(p, batch, ch).kind, few)) return 0;
  }
  *kind = 7;
  const size_t split = dense_path_split_bytes(p, batch);
  return split ? dense_path_split_offset(p) + split : dense_path_bytes(p);
}

size_t spmm_workspace_bytes(int dtype, int itype, int flags, int m, int k, int n, int nonzeros, int batch) {
  int kind;
  return workspace_plan(dtype, itype, flags, m, k, n, nonzeros, batch, &kind);
}

int spmm_workspace_kind(int dtype, int itype, int flags, int m, int k, int n, int nonzeros, int batch) {
  int kind;
  workspace_plan(dtype, itype, flags, m, k, n, nonzeros, batch, &kind);
  return kind;
}

// ---- the library's own scratch memory, for callers that cannot allocate ---------------------------------
// One array per GPU, placed when the code object is loaded on it and held until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress: every use of the memory below goes through
// the per-device pointer that call returned.
constexpr size_t kStaticScratchBytes = IEX_SPMM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_ptr[kMaxDevices] = {};   // per device: each GPU holds its own copy of the array at its own address

// The calling thread's current device's copy of `scratch` (looked up once per device, with that device current).
int static_scratch(void** ptr) {
  int device = -1;
  if (int rc = check_hip(hipGetDevice(&device), "hipGetDevice")) return rc;
  IEX_REQUIRE(device >= 0 && device < kMaxDevices, IEX_ERR_UNSUPPORTED, "spmm: device ordinal %d beyond %d", device, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[device]) {
    void* p = nullptr;
    if (int rc = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return rc;
    IEX_REQUIRE(p != nullptr && aligned(p, 256), IEX_ERR_STATE, "spmm: the library's scratch array has no usable device address");
    scratch_ptr[device] = p;
  }
  *ptr = scratch_ptr[device];
  return 0;
}
}  // namespace

}  // namespace iex

extern "C" {

int iex_spmm_static(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                    const int* row_indices, const void* values, const int* row_offsets,
                    const void* column_indices, const void* dense, const float* bias, void* out,
                    void* stream, int batch) {
  using namespace iex;
  // every call shares the array with whatever ran before it: nothing in it counts as "still there"
  flags &= ~(IEX_SPMM_TABLES_READY | IEX_SPMM_LISTS_READY);
  const size_t need = spmm_workspace_bytes(dtype, itype, flags, m, k, n, nonzeros, batch);
  if (need == 0)  // a call that would not touch a workspace runs as iex_spmm_ex does (a forced family 7 fails there)
    return spmm_dispatch(dtype, itype, flags, m, k, n, nonzeros, row_indices, values, row_offsets, column_indices, dense,
                         bias, out, stream, batch, nullptr, 0);
  IEX_REQUIRE(need <= kStaticScratchBytes, IEX_ERR_TOO_LARGE,
              "spmm (static scratch): this call needs %zu bytes of scratch memory, the library's array holds %zu "
              "(pass a workspace of your own to iex_spmm_ws, or call iex_spmm_ex)", need, kStaticScratchBytes);
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  return spmm_dispatch(dtype, itype, flags, m, k, n, nonzeros, row_indices, values, row_offsets, column_indices, dense,
                       bias, out, stream, batch, ws, kStaticScratchBytes);
}

size_t iex_spmm_static_scratch_bytes(void) { return iex::kStaticScratchBytes; }

int iex_spmm_ex(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                const int* row_indices, const void* values, const int* row_offsets,
                const void* column_indices, const void* dense, const float* bias, void* out,
                void* stream, int batch) {
  return iex::spmm_dispatch(dtype, itype, flags, m, k, n, nonzeros, row_indices, values, row_offsets,
                            column_indices, dense, bias, out, stream, batch, nullptr, 0);
}

int iex_spmm_ws(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                const int* row_indices, const void* values, const int* row_offsets,
                const void* column_indices, const void* dense, const float* bias, void* out,
                void* stream, int batch, void* workspace, size_t workspace_bytes) {
  return iex::spmm_dispatch(dtype, itype, flags, m, k, n, nonzeros, row_indices, values, row_offsets,
                            column_indices, dense, bias, out, stream, batch, workspace, workspace_bytes);
}

int iex_spmm_sched(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                   const int* row_indices, const void* values, const int* row_offsets,
                   const void* column_indices, const void* dense, const float* bias, void* out,
                   void* stream, int batch, void* workspace, size_t workspace_bytes, const int* row_histogram) {
  return iex::spmm_dispatch(dtype, itype, flags, m, k, n, nonzeros, row_indices, values, row_offsets,
                            column_indices, dense, bias, out, stream, batch, workspace, workspace_bytes, row_histogram);
}

size_t iex_spmm_workspace_bytes(int dtype, int itype, int flags, int m, int k, int n, int nonzeros, int batch) {
  return iex::spmm_workspace_bytes(dtype, itype, flags, m, k, n, nonzeros, batch);
}

int iex_spmm_workspace_kind(int dtype, int itype, int flags, int m, int k, int n, int nonzeros, int batch) {
  return iex::spmm_workspace_kind(dtype, itype, flags, m, k, n, nonzeros, batch);
}

int iex_CudaSpmm2(int m, int k, int n, int nonzeros, const int* row_indices, const float* values,
                  const int* row_offsets, const int* column_indices, const float* dense_matrix,
                  float* output_matrix, void* stream, int batch_size) {
  return iex::spmm_dispatch(IEX_F32, IEX_I32, IEX_SPMM_PER_BATCH_VALUES | IEX_SPMM_ACCUMULATE | IEX_SPMM_ANY_COLUMN_ORDER, m, k, n,
                            nonzeros, row_indices, values, row_offsets, column_indices, dense_matrix,
                            nullptr, output_matrix, stream, batch_size, nullptr, 0);
}

int iex_CudaSpmm3(int m, int k, int n, int nonzeros, const int* row_indices, const float* values,
                  const int* row_offsets, const int* column_indices, const float* dense_matrix,
                  float* output_matrix, void* stream, int batch_size) {
  return iex::spmm_dispatch(IEX_F32, IEX_I32, IEX_SPMM_ANY_COLUMN_ORDER, m, k, n, nonzeros, row_indices, values, row_offsets,
                            column_indices, dense_matrix, nullptr, output_matrix, stream, batch_size, nullptr, 0);
}

int iex_CudaSpmm5(int m, int k, int n, int nonzeros, const int* row_indices, const uint16_t* values,
                  const int* row_offsets, const int16_t* column_indices, const uint16_t* dense_matrix,
                  uint16_t* output_matrix, void* stream, int batch_size) {
  return iex::spmm_dispatch(IEX_F16, IEX_I16, IEX_SPMM_ANY_COLUMN_ORDER, m, k, n, nonzeros, row_indices, values, row_offsets,
                            column_indices, dense_matrix, nullptr, output_matrix, stream, batch_size, nullptr, 0);
}

}  // extern "C"
