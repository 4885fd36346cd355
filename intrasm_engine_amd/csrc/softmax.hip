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

// Two floats rounded to nearest even and packed (a, then b in the upper half): one conversion instruction on this part.
template <typename T>
__device__ __forceinline__ unsigned pack_pair(float a, float b) {
  typedef float f2 __attribute__((ext_vector_type(2)));
  const f2 ab = {a, b};
  if constexpr (std::is_same<T, __half>::value) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(unsigned, __builtin_convertvector(ab, h2));
  } else {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(unsigned, __builtin_convertvector(ab, b2));
  }
}

// 16-bit entries, rows of up to 512 entries: four rows per wavefront, 16 lanes per row, P pairs of neighbouring entries
// per lane (one 4-byte access at 2-byte alignment each; the pair that would pass the end of the tensor is read one
// entry earlier).  The one-row-per-wavefront kernel below spends 160 vector instructions per row of 280 entries, most
// of them on the two reductions across 64 lanes and on lanes past the row's end, and that, not the 74 MB it moves, is
// its time (16 heads of 4096 rows: 17 of its 21 us are vector-ALU issue).  Here a reduction is four DPP steps inside
// the 16 lanes of a row and serves four rows at once, and the scale rides in the exponent's multiply-add.
// last_at: index (in this batch entry's v) of the tensor's last pair, or INT_MAX where that lies beyond an int.
template <typename T, int P>
__device__ __forceinline__ void softmax_four_rows(T* v, int start, int end, int gl, float scale, int last_at) {
  typedef unsigned u32_a2 __attribute__((aligned(2)));
  constexpr float kLog2e = 1.44269504088896340736f;
  float x[P][2];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < P; ++i) {
    const int j = start + (i * 16 + gl) * 2;
    const bool back = j > last_at;        // only the last entry of the tensor
    const unsigned two = *reinterpret_cast<const u32_a2*>(v + min(j, last_at));
    const unsigned short lo = (unsigned short)(back ? two >> 16 : two), hi = (unsigned short)(two >> 16);
    x[i][0] = j < end ? elem<T>::to_float(__builtin_bit_cast(T, lo)) : -INFINITY;
    x[i][1] = j + 1 < end ? elem<T>::to_float(__builtin_bit_cast(T, hi)) : -INFINITY;
    mx = fmaxf(mx, fmaxf(x[i][0], x[i][1]));
  }
  // (scale > 0 keeps the order of the entries: the maximum of the scaled entries is the scaled maximum; a scale <= 0
  // is handled by the caller)
  mx = dpp_max_f<0xB1>(mx);
  mx = dpp_max_f<0x4E>(mx);
  mx = dpp_max_f<0x141>(mx);
  mx = dpp_max_f<0x140>(mx);
  const float c = scale * kLog2e, shift = -mx * c;
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < P; ++i)
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      x[i][w] = __builtin_amdgcn_exp2f(fmaf(x[i][w], c, shift));   // (an entry past the row's end: exp2(-inf) = 0)
      sum += x[i][w];
    }
  sum = group_sum<16>(sum);
  const float inv = __builtin_amdgcn_rcpf(sum);
#pragma unroll
  for (int i = 0; i < P; ++i) {
    const int j = start + (i * 16 + gl) * 2;
    const unsigned both = pack_pair<T>(x[i][0] * inv, x[i][1] * inv);
    if (j + 1 < end)
      *reinterpret_cast<u32_a2*>(v + j) = both;
    else if (j < end)
      *reinterpret_cast<unsigned short*>(v + j) = (unsigned short)both;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void csr_softmax16_kernel(int m, int nnz, const int* __restrict__ row_indices,
                                                            const int* __restrict__ row_offsets, T* values, float scale) {
  static_assert(sizeof(T) == 2, "16-bit entries");
  const int lane = lane_id();
  const int gl = lane & 15;
  const int slot = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 4 + (lane >> 4);   // this lane's row slot
  T* v = values + (size_t)blockIdx.z * nnz;
  // (the host launches this kernel for tensors of two entries or more)
  const long long to_last = (long long)(gridDim.z - blockIdx.z) * nnz - 2;
  const int last_pair = (int)min(to_last, (long long)0x7fffffff);
  int start = 0, end = 0;
  if (slot < m) {
    const int row = row_indices[slot];
    start = row_offsets[row];
    end = row_offsets[row + 1];
  }
  const int len = end - start;
  int longest = max(len, __shfl_xor(len, 16));
  longest = max(longest, __shfl_xor(longest, 32));   // of the wavefront's four rows
  if (longest <= 0) return;
  // as many pairs per lane as the longest of the four rows needs (every pair is instructions for all 64 lanes)
  switch ((longest + 31) / 32) {
    case 1: return softmax_four_rows<T, 1>(v, start, end, gl, scale, last_pair);
    case 2: return softmax_four_rows<T, 2>(v, start, end, gl, scale, last_pair);
    case 3: return softmax_four_rows<T, 3>(v, start, end, gl, scale, last_pair);
    case 4: return softmax_four_rows<T, 4>(v, start, end, gl, scale, last_pair);
    case 5: return softmax_four_rows<T, 5>(v, start, end, gl, scale, last_pair);
    case 6: return softmax_four_rows<T, 6>(v, start, end, gl, scale, last_pair);
    case 7: return softmax_four_rows<T, 7>(v, start, end, gl, scale, last_pair);
    case 8: return softmax_four_rows<T, 8>(v, start, end, gl, scale, last_pair);
    case 9: return softmax_four_rows<T, 9>(v, start, end, gl, scale, last_pair);
    case 10: return softmax_four_rows<T, 10>(v, start, end, gl, scale, last_pair);
    case 11: return softmax_four_rows<T, 11>(v, start, end, gl, scale, last_pair);
    case 12: return softmax_four_rows<T, 12>(v, start, end, gl, scale, last_pair);
    case 13: return softmax_four_rows<T, 13>(v, start, end, gl, scale, last_pair);
    case 14: return softmax_four_rows<T, 14>(v, start, end, gl, scale, last_pair);
    case 15: return softmax_four_rows<T, 15>(v, start, end, gl, scale, last_pair);
    case 16: return softmax_four_rows<T, 16>(v, start, end, gl, scale, last_pair);
    default: break;
  }
  // a longer row among the four: the whole wavefront takes them one by one, three strided passes each
#pragma unroll 1
  for (int q = 0; q < 4; ++q) {
    const int s = __shfl(start, q * 16), e = __shfl(end, q * 16);
    if (e <= s) continue;   // (uniform)
    float mx = -INFINITY;
    for (int j = s + lane; j < e; j += kWave) mx = fmaxf(mx, scale * elem<T>::to_float(v[j]));
    mx = wave_max(mx);
    float sum = 0.f;
    for (int j = s + lane; j < e; j += kWave) sum += __expf(scale * elem<T>::to_float(v[j]) - mx);
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int j = s + lane; j < e; j += kWave)
      v[j] = elem<T>::from_float(__expf(scale * elem<T>::to_float(v[j]) - mx) * inv);
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
  dim3 grid(ceil_div(m, 4), 1, batch), grid16(ceil_div(m, 16), 1, batch);
  // 16-bit entries with rows of a few hundred entries at most on average (sparse attention): four rows per wavefront;
  // a positive scale only (the kernel takes the maximum before it scales), and a tensor of two entries or more
  const bool four_rows = scale > 0.f && (long long)batch * nonzeros >= 2 && (double)nonzeros / m <= 512.0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case IEX_F32:
      hipLaunchKernelGGL(csr_softmax_kernel<float>, grid, dim3(256), 0, s, m, nonzeros, row_indices, row_offsets,
                         static_cast<float*>(values), scale);
      break;
    case IEX_F16:
      if (four_rows)
        hipLaunchKernelGGL(csr_softmax16_kernel<__half>, grid16, dim3(256), 0, s, m, nonzeros, row_indices, row_offsets,
                           static_cast<__half*>(values), scale);
      else
        hipLaunchKernelGGL(csr_softmax_kernel<__half>, grid, dim3(256), 0, s, m, nonzeros, row_indices, row_offsets,
                           static_cast<__half*>(values), scale);
      break;
    case IEX_BF16:
      if (four_rows)
        hipLaunchKernelGGL(csr_softmax16_kernel<__hip_bfloat16>, grid16, dim3(256), 0, s, m, nonzeros, row_indices,
                           row_offsets, static_cast<__hip_bfloat16*>(values), scale);
      else
        hipLaunchKernelGGL(csr_softmax_kernel<__hip_bfloat16>, grid, dim3(256), 0, s, m, nonzeros, row_indices,
                           row_offsets, static_cast<__hip_bfloat16*>(values), scale);
      break;
    default:
      return fail(IEX_ERR_UNSUPPORTED, "csr_softmax: no kernel for dtype=%d", dtype);
  }
  return check_hip(hipGetLastError(), "csr_softmax launch");
}
