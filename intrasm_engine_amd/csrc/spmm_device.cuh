// CSR SpMM device code for gfx950 (wave64): out[z, r, :] = sum_j values[j] * dense[z, col[j], :].
//
// Work decomposition
//   * a wavefront owns one CSR row (taken in swizzled order: heavy rows are launched
//     first) and one tile of 64*VEC output columns; lane l owns VEC adjacent columns,
//     so every gather of a dense row is one fully coalesced 64*VEC*sizeof(T) access;
//   * values / column indices are read 64 nonzeros at a time, one per lane
//     (coalesced), and handed to the whole wave through v_readlane: the column index
//     and the value of the nonzero being processed live in scalar registers, the
//     address arithmetic runs on the scalar unit and the vector unit only issues the
//     gather and the FMAs;
//   * long rows are split over WPR wavefronts of one workgroup (chunks of 64 nonzeros
//     dealt round-robin); partial sums meet in LDS, so the result is deterministic and
//     needs no atomics.
// Accumulation is fp32 for every element type.
#pragma once
#include "iex_common.h"

namespace iex {

struct SpmmParams {
  int m, k, n, nnz;
  const int* row_indices;
  const void* values;
  const int* row_offsets;
  const void* cols;
  const void* dense;
  const float* bias;
  void* out;
  int per_batch_values, accumulate, relu;
};

constexpr int kUnroll = 8;

template <int VEC, int WPR>
constexpr int spmm_lds_floats() { return (WPR > 1) ? WPR * kWave * VEC : 1; }

// One workgroup's share: block (bx, by, bz) of the grid
//   (ceil(m / rows_per_block), ceil(n / (64*VEC)), batch).
// `red` must hold spmm_lds_floats<VEC,WPR>() floats.  Every thread of the workgroup
// must call this when WPR > 1 (it contains a barrier).
template <typename T, typename IT, int VEC, int WPR>
__device__ __forceinline__ void spmm_block(const SpmmParams& p, int bx, int by, int bz, float* red) {
  constexpr int kWavesPerBlock = (WPR == 16) ? 16 : 4;
  constexpr int kRowsPerBlock = kWavesPerBlock / WPR;
  const int lane = lane_id();
  const int wave = uniform(threadIdx.x >> 6);
  const int z = bz;
  const int row_slot = bx * kRowsPerBlock + wave / WPR;
  const int part = wave % WPR;  // which share of the row this wave sums

  const int col0 = by * (kWave * VEC) + lane * VEC;
  const bool lane_live = col0 < p.n;
  const int col_ld = lane_live ? col0 : 0;  // idle lanes gather a valid address, result unused

  float acc[VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) acc[i] = 0.f;

  const bool row_live = row_slot < p.m;  // wave-uniform
  int row = 0;
  if (row_live) {
    row = uniform(p.row_indices[row_slot]);
    const int start = uniform(p.row_offsets[row]);
    const int end = uniform(p.row_offsets[row + 1]);
    const T* __restrict__ values = static_cast<const T*>(p.values) +
                                   (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
    const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
    const T* __restrict__ dense = static_cast<const T*>(p.dense) + (size_t)z * p.k * p.n + col_ld;

    for (int base = start + part * kWave; base < end; base += kWave * WPR) {
      const int j = base + lane;
      float v = 0.f;
      int c = 0;
      if (j < end) {
        v = elem<T>::to_float(values[j]);
        c = (int)cols[j];
      }
      const int cnt = min(kWave, end - base);  // wave-uniform
      int t = 0;
      for (; t + kUnroll <= cnt; t += kUnroll) {
        vec_t<T, VEC> bv[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int cu = bcast_i(c, t + u);
          bv[u] = load_vec<T, VEC>(dense + (size_t)cu * p.n);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const float vu = bcast_f(v, t + u);
#pragma unroll
          for (int i = 0; i < VEC; ++i) acc[i] = fmaf(vu, elem<T>::to_float(bv[u].v[i]), acc[i]);
        }
      }
      for (; t < cnt; ++t) {
        const int cu = bcast_i(c, t);
        const float vu = bcast_f(v, t);
        const vec_t<T, VEC> bv = load_vec<T, VEC>(dense + (size_t)cu * p.n);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = fmaf(vu, elem<T>::to_float(bv.v[i]), acc[i]);
      }
    }
  }

  if (WPR > 1) {
    // Every wave of the block reaches this barrier (row_live is uniform per block here
    // because a block holds exactly one row when WPR equals the waves per block, and
    // otherwise idle waves fall through with zero partials).
#pragma unroll
    for (int i = 0; i < VEC; ++i) red[(wave * VEC + i) * kWave + lane] = acc[i];
    __syncthreads();
    if (part != 0) return;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float s = acc[i];
      for (int w = 1; w < WPR; ++w) s += red[((wave + w) * VEC + i) * kWave + lane];
      acc[i] = s;
    }
  }

  if (!row_live || !lane_live) return;
  const float bias = p.bias ? p.bias[row] : 0.f;
  T* __restrict__ out = static_cast<T*>(p.out) + ((size_t)z * p.m + row) * p.n + col0;
  vec_t<T, VEC> o;
  if (p.accumulate) {
    const vec_t<T, VEC> prev = load_vec<T, VEC>(out);
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] += elem<T>::to_float(prev.v[i]);
  }
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    float r = acc[i] + bias;
    if (p.relu) r = fmaxf(r, 0.f);
    o.v[i] = elem<T>::from_float(r);
  }
  store_vec<T, VEC>(out, o);
}


}  // namespace iex
