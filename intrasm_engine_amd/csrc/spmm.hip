// Host side of the CSR SpMM: kernel wrappers, variant selection, argument checks and
// the C entry points.  The device code is in spmm_device.cuh.
#include "spmm_device.cuh"

namespace iex {
namespace {

template <typename T, typename IT, int VEC, int WPR>
__global__ __launch_bounds__(WPR == 16 ? 1024 : 256) void spmm_kernel(SpmmParams p) {
  __shared__ float red[spmm_lds_floats<VEC, WPR>()];
  spmm_block<T, IT, VEC, WPR>(p, blockIdx.x, blockIdx.y, blockIdx.z, red);
}

template <typename T, typename IT, int VEC, int WPR>
int launch_one(const SpmmParams& p, int batch, hipStream_t stream) {
  constexpr int kWavesPerBlock = (WPR == 16) ? 16 : 4;
  constexpr int kRowsPerBlock = kWavesPerBlock / WPR;
  dim3 grid(ceil_div(p.m, kRowsPerBlock), ceil_div(p.n, kWave * VEC), batch);
  dim3 block(kWavesPerBlock * kWave);
  hipLaunchKernelGGL((spmm_kernel<T, IT, VEC, WPR>), grid, block, 0, stream, p);
  return check_hip(hipGetLastError(), "spmm launch");
}

template <typename T, typename IT, int VEC>
int launch_wpr(const SpmmParams& p, int batch, int wpr, hipStream_t stream) {
  switch (wpr) {
    case 1: return launch_one<T, IT, VEC, 1>(p, batch, stream);
    case 4: return launch_one<T, IT, VEC, 4>(p, batch, stream);
    case 16: return launch_one<T, IT, VEC, 16>(p, batch, stream);
  }
  return fail(IEX_ERR_BAD_ARGUMENT, "spmm: waves-per-row must be 1, 4 or 16 (got %d)", wpr);
}

// Widest per-lane vector such that (a) it divides n, (b) a 64-lane tile is not wider than
// n rounded up to 64 lanes (keeps lanes busy for narrow outputs), (c) rows stay aligned.
template <typename T>
int pick_vec(int n, const void* dense, const void* out) {
  constexpr int kMax = 16 / (int)sizeof(T);
  int vec = kMax;
  while (vec > 1 && (n % vec != 0 || kWave * vec > n || !aligned(dense, sizeof(T) * vec) ||
                     !aligned(out, sizeof(T) * vec)))
    vec >>= 1;
  return vec;
}

template <typename T, typename IT>
int launch_typed(const SpmmParams& p, int batch, int wpr, hipStream_t stream) {
  const int vec = pick_vec<T>(p.n, p.dense, p.out);
  if constexpr (sizeof(T) == 2) {
    if (vec == 8) return launch_wpr<T, IT, 8>(p, batch, wpr, stream);
  }
  switch (vec) {
    case 4: return launch_wpr<T, IT, 4>(p, batch, wpr, stream);
    case 2: return launch_wpr<T, IT, 2>(p, batch, wpr, stream);
    default: return launch_wpr<T, IT, 1>(p, batch, wpr, stream);
  }
}

// Waves per row from the mean row length: short rows get a wave each, long rows a
// workgroup, so that the heaviest row of a skewed matrix never runs on a single wave.
int pick_wpr(int m, int nnz) {
  const double mean = m > 0 ? (double)nnz / m : 0.0;
  if (mean >= 768.0) return 16;
  if (mean >= 96.0) return 4;
  return 1;
}

}  // namespace

int spmm_dispatch(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                  const int* row_indices, const void* values, const int* row_offsets,
                  const void* column_indices, const void* dense, const float* bias, void* out,
                  void* stream, int batch) {
  IEX_REQUIRE(m >= 0 && k >= 0 && n >= 0 && nonzeros >= 0 && batch >= 0, IEX_ERR_BAD_ARGUMENT,
              "spmm: negative dimension (m=%d k=%d n=%d nnz=%d batch=%d)", m, k, n, nonzeros, batch);
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
  int wpr = (flags >> 8) & 0xff;
  if (wpr == 0) wpr = pick_wpr(m, nonzeros);
  SpmmParams p{m, k, n, nonzeros, row_indices, values, row_offsets, column_indices, dense, bias, out,
               (flags & IEX_SPMM_PER_BATCH_VALUES) != 0, (flags & IEX_SPMM_ACCUMULATE) != 0,
               (flags & IEX_SPMM_RELU) != 0};
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == IEX_F32 && itype == IEX_I32) return launch_typed<float, int>(p, batch, wpr, s);
  if (dtype == IEX_F16 && itype == IEX_I32) return launch_typed<__half, int>(p, batch, wpr, s);
  if (dtype == IEX_F16 && itype == IEX_I16) return launch_typed<__half, short>(p, batch, wpr, s);
  if (dtype == IEX_BF16 && itype == IEX_I32) return launch_typed<__hip_bfloat16, int>(p, batch, wpr, s);
  return fail(IEX_ERR_UNSUPPORTED, "spmm: no kernel for dtype=%d itype=%d", dtype, itype);
}

}  // namespace iex

extern "C" {

int iex_spmm_ex(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                const int* row_indices, const void* values, const int* row_offsets,
                const void* column_indices, const void* dense, const float* bias, void* out,
                void* stream, int batch) {
  return iex::spmm_dispatch(dtype, itype, flags, m, k, n, nonzeros, row_indices, values, row_offsets,
                            column_indices, dense, bias, out, stream, batch);
}

int iex_CudaSpmm2(int m, int k, int n, int nonzeros, const int* row_indices, const float* values,
                  const int* row_offsets, const int* column_indices, const float* dense_matrix,
                  float* output_matrix, void* stream, int batch_size) {
  return iex::spmm_dispatch(IEX_F32, IEX_I32, IEX_SPMM_PER_BATCH_VALUES | IEX_SPMM_ACCUMULATE, m, k, n,
                            nonzeros, row_indices, values, row_offsets, column_indices, dense_matrix,
                            nullptr, output_matrix, stream, batch_size);
}

int iex_CudaSpmm3(int m, int k, int n, int nonzeros, const int* row_indices, const float* values,
                  const int* row_offsets, const int* column_indices, const float* dense_matrix,
                  float* output_matrix, void* stream, int batch_size) {
  return iex::spmm_dispatch(IEX_F32, IEX_I32, 0, m, k, n, nonzeros, row_indices, values, row_offsets,
                            column_indices, dense_matrix, nullptr, output_matrix, stream, batch_size);
}

int iex_CudaSpmm5(int m, int k, int n, int nonzeros, const int* row_indices, const uint16_t* values,
                  const int* row_offsets, const int16_t* column_indices, const uint16_t* dense_matrix,
                  uint16_t* output_matrix, void* stream, int batch_size) {
  return iex::spmm_dispatch(IEX_F16, IEX_I16, 0, m, k, n, nonzeros, row_indices, values, row_offsets,
                            column_indices, dense_matrix, nullptr, output_matrix, stream, batch_size);
}

}  // extern "C"
