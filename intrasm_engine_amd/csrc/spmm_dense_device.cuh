// Dense form of a CSR matrix with 16-bit values (fp16 / bf16 bit patterns), for the SpMM path
// that hands the product to the dense GEMM: every workgroup that computes a tile of the output
// of a matrix-core SpMM kernel rebuilds the dense form of its rows of A in LDS, once per column
// tile of the output; when the output has many column tiles it is cheaper to build the dense
// form once, in a workspace of m * k * 2 bytes that stays in L2 / MALL, and let the GEMM read it.
//
// One workgroup of four wavefronts per pair of rows (the loads of both rows in flight together): each row is assembled
// in LDS (zeros, then the nonzeros scattered to their columns, each wavefront taking a contiguous quarter of them) and written with 128-bit stores, so every byte of the
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

constexpr int kDenseRows = 2;     // rows per workgroup, side by side: the loads of both are in flight together

template <typename IT>
__global__ __launch_bounds__(kDenseThreads) void csr_to_dense_kernel(int m, int k, const int* __restrict__ row_offsets,
                                                                     const IT* __restrict__ cols,
                                                                     const uint16_t* __restrict__ values,
                                                                     uint16_t* __restrict__ out, int* __restrict__ zero_words,
                                                                     int n_zero_words) {
  __shared__ __align__(16) uint16_t srow[kDenseRows][kDenseSeg];
  // (words that the kernel after this one wants zero at its launch, a few hundred at most: cheaper here than a launch)
  if (blockIdx.x == 0)
    for (int i = threadIdx.x; i < n_zero_words; i += kDenseThreads) zero_words[i] = 0;
  const int lane = lane_id();
  const int wave = uniform(threadIdx.x >> 6);
  // this wavefront's quarter of each row's nonzeros, in whole chunks of 64
  int pos[kDenseRows], end[kDenseRows];
#pragma unroll
  for (int r = 0; r < kDenseRows; ++r) {
    const int row = min((int)blockIdx.x * kDenseRows + r, m - 1);   // (the grid has ceil(m / kDenseRows) workgroups)
    const int first = uniform(row_offsets[row]);
    const int last = (int)blockIdx.x * kDenseRows + r < m ? uniform(row_offsets[row + 1]) : first;   // (past the matrix: an empty row, not stored)
    const int share = ((max(last - first, 0) + kWave * kDenseWaves - 1) / (kWave * kDenseWaves)) * kWave;
    pos[r] = min(first + wave * share, last);
    end[r] = min(pos[r] + share, last);
  }
  for (int c0 = 0; c0 < k; c0 += kDenseSeg) {
    const int len = min(kDenseSeg, k - c0);  // a multiple of 8
    if (c0) __syncthreads();   // the previous segment has been copied out
#pragma unroll
    for (int r = 0; r < kDenseRows; ++r)
      for (int i = threadIdx.x * 8; i < len; i += kDenseThreads * 8) *reinterpret_cast<uint4*>(srow[r] + i) = uint4{0u, 0u, 0u, 0u};
    __syncthreads();
    // the nonzeros of this segment: 64 at a time from the cursors, four chunks of each row in flight
    bool more[kDenseRows];
#pragma unroll
    for (int r = 0; r < kDenseRows; ++r) more[r] = pos[r] < end[r];
    static_assert(kDenseRows == 2, "the loop below names both rows");
    while (more[0] || more[1]) {
      int c[kDenseRows][4];
      uint16_t v[kDenseRows][4];
#pragma unroll
      for (int r = 0; r < kDenseRows; ++r)
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int j = max(min(pos[r] + u * kWave + lane, end[r] - 1), 0);   // (a row without nonzeros: entry 0, never used)
          c[r][u] = (int)cols[j] - c0;
          v[r][u] = values[j];
        }
#pragma unroll
      for (int r = 0; r < kDenseRows; ++r) {
        int taken = 0;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          // (canonical CSR: c >= 0, earlier segments took what lies before c0; the test keeps a row whose
          // columns do not ascend inside the row's slice of LDS -- its result is then undefined, not a fault)
          const bool mine = more[r] && pos[r] + u * kWave + lane < end[r] && c[r][u] < len && c[r][u] >= 0;
          if (mine) srow[r][c[r][u]] = v[r][u];
          taken += __popcll(__ballot(mine));
        }
        pos[r] += taken;
        more[r] = taken == 4 * kWave;  // a short take: the quarter ended or its next nonzero lies beyond this segment
      }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kDenseRows; ++r) {
      const int row = (int)blockIdx.x * kDenseRows + r;
      if (row < m)
        for (int i = threadIdx.x * 8; i < len; i += kDenseThreads * 8)
          *reinterpret_cast<uint4*>(out + (size_t)row * k + c0 + i) = *reinterpret_cast<const uint4*>(srow[r] + i);
    }
  }
}

}  // namespace iex
