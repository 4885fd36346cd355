// Dense form of a CSR matrix with 16-bit values (fp16 / bf16 bit patterns), for the SpMM path
// that hands the product to the dense GEMM: every workgroup that computes a tile of the output
// of a matrix-core SpMM kernel rebuilds the dense form of its rows of A in LDS, once per column
// tile of the output; when the output has many column tiles it is cheaper to build the dense
// form once, in a workspace of m * k * 2 bytes that stays in L2 / MALL, and let the GEMM read it.
//
// One workgroup of four wavefronts per row: the row is assembled in LDS (zeros, then the nonzeros scattered to their
// columns, each wavefront taking a contiguous quarter of them) and written with 128-bit stores, so every byte of the
// workspace is written exactly once, by one kind of store, whatever the sparsity.  What a row costs is the chain of
// "load 256 nonzeros, scatter them" steps of its wavefronts, each a round trip to memory: with one wavefront per row
// the longest row set the kernel's time (4096 nonzeros: 16 steps, 24 us where the bytes written take 8).
// Rows longer than kDenseSeg columns are done in segments, every wavefront with a cursor into its quarter of the
// row's ascending column indices.  Needs k % 8 == 0 and a 16-byte aligned workspace; column indices inside a row must
// ascend strictly (canonical CSR).
#pragma once
#include "iex_common.h"

namespace iex {

constexpr int kDenseSeg = 4096;  // columns of a row assembled at a time (8 KB of LDS per wavefront)
constexpr int kDenseWaves = 4;
constexpr int kDenseThreads = kDenseWaves * kWave;

template <typename IT>
__global__ __launch_bounds__(kDenseThreads) void csr_to_dense_kernel(int m, int k, const int* __restrict__ row_offsets,
                                                                     const IT* __restrict__ cols,
                                                                     const uint16_t* __restrict__ values,
                                                                     uint16_t* __restrict__ out, int* __restrict__ zero_words,
                                                                     int n_zero_words) {
  __shared__ __align__(16) uint16_t srow[kDenseSeg];
  // (words that the kernel after this one wants zero at its launch, a few hundred at most: cheaper here than a launch)
  if (blockIdx.x == 0)
    for (int i = threadIdx.x; i < n_zero_words; i += kDenseThreads) zero_words[i] = 0;
  const int lane = lane_id();
  const int wave = uniform(threadIdx.x >> 6);
  const int row = blockIdx.x;   // (the grid has m workgroups)
  const int first = uniform(row_offsets[row]), last = uniform(row_offsets[row + 1]);
  // this wavefront's quarter of the row's nonzeros, in whole chunks of 64
  const int share = ((max(last - first, 0) + kWave * kDenseWaves - 1) / (kWave * kDenseWaves)) * kWave;
  int pos = min(first + wave * share, last);
  const int end = min(pos + share, last);
  uint16_t* orow = out + (size_t)row * k;
  for (int c0 = 0; c0 < k; c0 += kDenseSeg) {
    const int len = min(kDenseSeg, k - c0);  // a multiple of 8
    if (c0) __syncthreads();   // the previous segment has been copied out
    for (int i = threadIdx.x * 8; i < len; i += kDenseThreads * 8) *reinterpret_cast<uint4*>(srow + i) = uint4{0u, 0u, 0u, 0u};
    __syncthreads();
    // the nonzeros of this segment: 64 at a time from the cursor, four chunks in flight
    for (bool more = pos < end; more;) {
      int c[4];
      uint16_t v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = min(pos + u * kWave + lane, end - 1);
        c[u] = (int)cols[j] - c0;
        v[u] = values[j];
      }
      int taken = 0;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        // (canonical CSR: c >= 0, earlier segments took what lies before c0; the test keeps a row whose
        // columns do not ascend inside the row's slice of LDS -- its result is then undefined, not a fault)
        const bool mine = pos + u * kWave + lane < end && c[u] < len && c[u] >= 0;
        if (mine) srow[c[u]] = v[u];
        taken += __popcll(__ballot(mine));
      }
      pos += taken;
      more = taken == 4 * kWave;  // a short take: the quarter ended or its next nonzero lies beyond this segment
    }
    __syncthreads();
    for (int i = threadIdx.x * 8; i < len; i += kDenseThreads * 8)
      *reinterpret_cast<uint4*>(orow + c0 + i) = *reinterpret_cast<const uint4*>(srow + i);
  }
}

}  // namespace iex
