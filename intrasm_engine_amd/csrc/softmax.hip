// In-place row-wise softmax over the stored entries of a CSR matrix (wave64):
// values[z, j] <- exp(scale*values[z, j] - max_row) / sum_row for j in row.
// One wavefront per (row, batch entry), the two reductions done with DPP + readlane.  Rows of
// up to 512 entries (sparse attention has hundreds) are held in registers between one read and
// one write; longer rows take three strided passes, the second and third of which hit L1/L2.
#include "iex_common.h"

namespace iex {
namespace {

// R slots of W entries per lane (W = 2 for 16-bit types: a lane reads and writes two neighbouring entries with one
// 4-byte access at 2-byte alignment; the pair that would pass the end of the tensor is read one entry earlier).
// Entries are summed in the order slot, lane-pair member, then across lanes, whatever R: the same bits for every R.
template <typename T, int R, int W>
__device__ __forceinline__ void softmax_row_in_registers(T* v, int start, int end, int lane, float scale, T* last_pair) {
  typedef unsigned u32_a2 __attribute__((aligned(2)));
  float x[R][W];
  float mx = -INFINITY;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int j = start + (r * kWave + lane) * W;
    if constexpr (W == 2) {
      T* at = v + j;
      const bool back = at > last_pair;        // only the last entry of the tensor
      const unsigned two = *reinterpret_cast<const u32_a2*>(back ? last_pair : at);
      const unsigned short lo = (unsigned short)(back ? two >> 16 : two), hi = (unsigned short)(two >> 16);
      x[r][0] = j < end ? scale * elem<T>::to_float(__builtin_bit_cast(T, lo)) : -INFINITY;
      x[r][1] = j + 1 < end ? scale * elem<T>::to_float(__builtin_bit_cast(T, hi)) : -INFINITY;
      mx = fmaxf(mx, fmaxf(x[r][0], x[r][1]));
    } else {
      x[r][0] = j < end ? scale * elem<T>::to_float(v[j]) : -INFINITY;
      mx = fmaxf(mx, x[r][0]);
    }
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const int j = start + (r * kWave + lane) * W + w;
      x[r][w] = j < end ? __expf(x[r][w] - mx) : 0.f;
      sum += x[r][w];
    }
  sum = wave_sum(sum);
  const float inv = 1.f / sum;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int j = start + (r * kWave + lane) * W;
    if constexpr (W == 2) {
      const T a = elem<T>::from_float(x[r][0] * inv), b = elem<T>::from_float(x[r][1] * inv);
      if (j + 1 < end)
        *reinterpret_cast<u32_a2*>(v + j) = (unsigned)__builtin_bit_cast(unsigned short, a) | ((unsigned)__builtin_bit_cast(unsigned short, b) << 16);
      else if (j < end)
        v[j] = a;
    } else {
      if (j < end) v[j] = elem<T>::from_float(x[r][0] * inv);
    }
  }
}

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
  // rows of up to 512 entries (sparse attention) stay in registers: one read, one write, one exp per entry; as many
  // entries per lane as the row needs (the instructions of a slot are issued whether or not the row reaches it).
  // 32-bit entries: the same arithmetic in the same order as the three passes below; 16-bit entries are taken in
  // pairs, which orders the sum differently (a difference in rounding only)
  const int len = end - start;
  if constexpr (sizeof(T) == 2) {
    const long long total = (long long)gridDim.z * nnz;   // entries of the whole tensor: a pair is never read past it
    if (total >= 2) {
      T* last_pair = values + total - 2;
      if (len <= 2 * kWave) return softmax_row_in_registers<T, 1, 2>(v, start, end, lane, scale, last_pair);
      if (len <= 6 * kWave) return softmax_row_in_registers<T, 3, 2>(v, start, end, lane, scale, last_pair);
      if (len <= 8 * kWave) return softmax_row_in_registers<T, 4, 2>(v, start, end, lane, scale, last_pair);
    }
  } else {
    if (len <= 2 * kWave) return softmax_row_in_registers<T, 2, 1>(v, start, end, lane, scale, nullptr);
    if (len <= 5 * kWave) return softmax_row_in_registers<T, 5, 1>(v, start, end, lane, scale, nullptr);
    if (len <= 8 * kWave) return softmax_row_in_registers<T, 8, 1>(v, start, end, lane, scale, nullptr);
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
