// In-place row-wise softmax over the stored entries of a CSR matrix (wave64):
// values[z, j] <- exp(scale*values[z, j] - max_row) / sum_row for j in row.
// One wavefront per (row, batch entry), the two reductions done with DPP + readlane.  Rows of
// up to 512 entries (sparse attention has hundreds) are held in registers between one read and
// one write; longer rows take three strided passes, the second and third of which hit L1/L2.
#include "iex_common.h"

namespace iex {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void csr_softmax_kernel(int m, int nnz, const int* __restrict__ row_indices,
                                                          const int* __restrict__ row_offsets, T* values,
                                                          float scale) {
  const int lane = lane_id();
  const int row_slot = blockIdx.x * 4 + uniform(threadIdx.x >> 6);
  if (row_slot >= m) return;
  const int row = uniform(row_indices[row_slot]);
  const int start = uniform(row_offsets[row]);
  const int end = uniform(row_offsets[row + 1]);
  if (end <= start) return;
  T* v = values + (size_t)blockIdx.z * nnz;
  // rows of up to 512 entries (sparse attention) stay in registers: one read, one write, one exp
  // per entry, the same arithmetic in the same order as the three passes below
  constexpr int R = 8;
  if (end - start <= R * kWave) {
    float x[R];
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int j = start + r * kWave + lane;
      x[r] = j < end ? scale * elem<T>::to_float(v[j]) : -INFINITY;
      mx = fmaxf(mx, x[r]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int j = start + r * kWave + lane;
      x[r] = j < end ? __expf(x[r] - mx) : 0.f;
      sum += x[r];
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int j = start + r * kWave + lane;
      if (j < end) v[j] = elem<T>::from_float(x[r] * inv);
    }
    return;
  }
  float mx = -INFINITY;
  for (int j = start + lane; j < end; j += kWave) mx = fmaxf(mx, scale * elem<T>::to_float(v[j]));
  mx = wave_max(mx);
  float sum = 0.f;
  for (int j = start + lane; j < end; j += kWave) sum += __expf(scale * elem<T>::to_float(v[j]) - mx);
  sum = wave_sum(sum);
  const float inv = 1.f / sum;
  for (int j = start + lane; j < end; j += kWave)
    v[j] = elem<T>::from_float(__expf(scale * elem<T>::to_float(v[j]) - mx) * inv);
}

}  // namespace
}  // namespace iex

extern "C" int iex_csr_softmax(int dtype, int m, int nonzeros, const int* row_indices, const int* row_offsets,
                               void* values, float scale, void* stream, int batch) {
  using namespace iex;
  IEX_REQUIRE(m >= 0 && nonzeros >= 0 && batch >= 0, IEX_ERR_BAD_ARGUMENT, "csr_softmax: negative dimension");
  if (m == 0 || nonzeros == 0 || batch == 0) return 0;
  IEX_REQUIRE(row_indices && row_offsets && values, IEX_ERR_BAD_ARGUMENT, "csr_softmax: null pointer argument");
  IEX_REQUIRE(batch <= 65535, IEX_ERR_TOO_LARGE, "csr_softmax: batch %d exceeds 65535", batch);
  dim3 grid(ceil_div(m, 4), 1, batch);
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case IEX_F32:
      hipLaunchKernelGGL(csr_softmax_kernel<float>, grid, dim3(256), 0, s, m, nonzeros, row_indices, row_offsets,
                         static_cast<float*>(values), scale);
      break;
    case IEX_F16:
      hipLaunchKernelGGL(csr_softmax_kernel<__half>, grid, dim3(256), 0, s, m, nonzeros, row_indices, row_offsets,
                         static_cast<__half*>(values), scale);
      break;
    case IEX_BF16:
      hipLaunchKernelGGL(csr_softmax_kernel<__hip_bfloat16>, grid, dim3(256), 0, s, m, nonzeros, row_indices,
                         row_offsets, static_cast<__hip_bfloat16*>(values), scale);
      break;
    default:
      return fail(IEX_ERR_UNSUPPORTED, "csr_softmax: no kernel for dtype=%d", dtype);
  }
  return check_hip(hipGetLastError(), "csr_softmax launch");
}
