// Dense form of a CSR matrix with 16-bit values (fp16 / bf16 bit patterns), for the SpMM path
// that hands the product to the dense GEMM: every workgroup that computes a tile of the output
// of a matrix-core SpMM kernel rebuilds the dense form of its rows of A in LDS, once per column
// tile of the output; when the output has many column tiles it is cheaper to build the dense
// form once, in a workspace of m * k * 2 bytes that stays in L2 / MALL, and let the GEMM read it.
//
// One workgroup per row: the row is assembled in LDS (zeros, then the nonzeros scattered to their
// columns) and written with 128-bit stores, so every byte of the workspace is written exactly
// once, by one kind of store, whatever the sparsity.  Rows longer than kDenseSeg columns are done
// in segments.  Needs k % 8 == 0 and a 16-byte aligned workspace; column indices inside a row
// must be distinct (with duplicates the last writer wins instead of the sum).
#pragma once
#include "iex_common.h"

namespace iex {

constexpr int kDenseSeg = 16384;  // columns of a row assembled at a time (32 KB of LDS)
constexpr int kDenseThreads = 256;

template <typename IT>
__global__ __launch_bounds__(kDenseThreads) void csr_to_dense_kernel(int k, const int* __restrict__ row_offsets,
                                                                     const IT* __restrict__ cols,
                                                                     const uint16_t* __restrict__ values,
                                                                     uint16_t* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char smem[];
  uint16_t* srow = reinterpret_cast<uint16_t*>(smem);
  const int tid = threadIdx.x;
  const int row = blockIdx.x;
  const int start = row_offsets[row], end = row_offsets[row + 1];
  uint16_t* orow = out + (size_t)row * k;
  for (int c0 = 0; c0 < k; c0 += kDenseSeg) {
    const int len = min(kDenseSeg, k - c0);  // a multiple of 8
    for (int i = tid * 8; i < len; i += kDenseThreads * 8) *reinterpret_cast<uint4*>(srow + i) = uint4{0u, 0u, 0u, 0u};
    __syncthreads();
    for (int j = start + tid; j < end; j += kDenseThreads) {
      const int c = (int)cols[j] - c0;
      if ((unsigned)c < (unsigned)len) srow[c] = values[j];
    }
    __syncthreads();
    for (int i = tid * 8; i < len; i += kDenseThreads * 8)
      *reinterpret_cast<uint4*>(orow + c0 + i) = *reinterpret_cast<const uint4*>(srow + i);
    __syncthreads();  // the next segment clears the row again
  }
}

}  // namespace iex
