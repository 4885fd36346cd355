// CSR SpMM for a sparse operand with few columns (k <= 128) and a wide output: the products of
// sparse attention-style sweeps, a[M x K] * b[K x N] with K = 32 .. 128 and N in the thousands, where
// the output (batch * m * n elements) is the traffic that has to happen and everything else should
// stay out of its way.
//
// The row kernel spends a wavefront per (row, 64 * VEC columns): three dependent memory latencies
// (row offsets -> column indices / values -> dense row) to write one kilobyte, and every nonzero
// gathers its dense row segment from L2 although all rows of A share the same k dense rows.
// Here a workgroup of 8 (k <= 64) or 16 wavefronts owns one tile of 64 * VEC columns, one batch entry and a long
// run of consecutive rows:
//   * the k x (64 * VEC) tile of the dense operand is loaded into LDS once (k KB), lane i's
//     vector of every dense row at [row][i]: the layout the gather reads;
//   * a wavefront walks its rows in natural order, so their nonzeros are one contiguous range:
//     row offsets are read 64 at a time, column indices and values 64 at a time (coalesced, one
//     per lane) and handed out with v_readlane; a nonzero is one 128-bit LDS read and VEC FMAs;
//   * what is left per row is the store of its 64 * VEC outputs, and stores do not wait.
// Accumulation is fp32, in ascending nonzero order (the order of the row kernel with one wavefront
// per row, so results are bit-equal to it); the swizzle (row_indices) is ignored: it only
// schedules.  Needs n % VEC == 0 and 16-byte aligned dense operand and output (full vectors), or
// RAGGED: any n >= VEC at element alignment -- rows then start at any element, vectors are moved with
// element-aligned 128-bit accesses, and the one lane per row whose vector would pass the row's end
// works on the last VEC elements of the row instead (shifted back), computes all of them and stores
// only the ones it owns (the others belong to the lane to its left, which stores the same values).
#pragma once
#include "spmm_device.cuh"

namespace iex {

constexpr int kSmallKMax = 128;   // dense rows (KB of LDS) a tile may have
// 8 wavefronts per workgroup up to 64 dense rows (two workgroups per CU), 16 beyond (the 65-128 KB tile
// leaves room for one workgroup per CU only, which then brings the wavefronts)
constexpr int smallk_waves(int k) { return k <= 64 ? 8 : 16; }

template <typename T, typename IT, int VEC, bool RAGGED = false, int WAVES = 8>
__device__ __forceinline__ void spmm_smallk_block(const SpmmParams& p, int rows_per_wave, int bx, int by, int bz,
                                                  unsigned char* smem) {
  typedef vec_t<T, VEC> V;
  V* tile = reinterpret_cast<V*>(smem);  // [k][64]
  const int lane = lane_id();
  const int wave = uniform(threadIdx.x >> 6);
  const int z = bz;
  const int col0 = by * (kWave * VEC) + lane * VEC;
  const bool lane_live = col0 < p.n;
  const int shift = (RAGGED && lane_live && col0 + VEC > p.n) ? col0 + VEC - p.n : 0;
  const T* __restrict__ dense = static_cast<const T*>(p.dense) + (size_t)z * p.k * p.n + min(col0 - shift, p.n - VEC);
  for (int kr = wave; kr < p.k; kr += WAVES) tile[kr * kWave + lane] = load_vec<T, VEC, !RAGGED>(dense + (size_t)kr * p.n);
  __syncthreads();

  const T* __restrict__ values = static_cast<const T*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
  const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
  const int r_begin = min(p.m, (bx * WAVES + wave) * rows_per_wave);
  const int r_end = min(p.m, r_begin + rows_per_wave);
  int cbase = -kWave;  // first nonzero held in (cc, vv); none yet
  int cc = 0;
  float vv = 0.f;
  for (int g0 = r_begin; g0 < r_end; g0 += kWave - 1) {
    // offsets of up to 63 rows: lane l holds row_offsets[g0 + l]
    const int rows = min(kWave - 1, r_end - g0);
    const int off = p.row_offsets[min(g0 + lane, p.m)];
    for (int i = 0; i < rows; ++i) {
      const int row = g0 + i;
      const int s = bcast_i(off, i), e = bcast_i(off, i + 1);
      float acc[VEC];
#pragma unroll
      for (int u = 0; u < VEC; ++u) acc[u] = 0.f;
      for (int j = s; j < e;) {
        if (j - cbase >= kWave) {  // (uniform) the next 64 nonzeros, one per lane
          cbase = j;
          const int idx = min(j + lane, p.nnz - 1);
          cc = (int)cols[idx];
          vv = elem<T>::to_float(values[idx]);
        }
        // the row's nonzeros that (cc, vv) holds, four LDS reads in flight, summed in order
        const int tl = min(e, cbase + kWave) - cbase;
        int t = j - cbase;
        for (; t + 4 <= tl; t += 4) {
          V bv[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) bv[u] = tile[bcast_i(cc, t + u) * kWave + lane];
#pragma unroll
          for (int u = 0; u < 4; ++u) fma_vec<T, VEC>(acc, bcast_f(vv, t + u), bv[u]);
        }
        for (; t < tl; ++t) fma_vec<T, VEC>(acc, bcast_f(vv, t), tile[bcast_i(cc, t) * kWave + lane]);
        j = cbase + tl;
      }
      if (!lane_live) continue;
      T* __restrict__ out = static_cast<T*>(p.out) + ((size_t)z * p.m + row) * p.n + col0 - shift;
      if (p.accumulate) {
        const V prev = load_vec<T, VEC, !RAGGED>(out);
#pragma unroll
        for (int u = 0; u < VEC; ++u) acc[u] += elem<T>::to_float(prev.v[u]);
      }
      const float bias = p.bias ? p.bias[row] : 0.f;
      V o;
#pragma unroll
      for (int u = 0; u < VEC; ++u) {
        float r = acc[u] + bias;
        if (p.relu) r = fmaxf(r, 0.f);
        o.v[u] = elem<T>::from_float(r);
      }
      if (RAGGED && shift > 0) {
#pragma unroll
        for (int u = 0; u < VEC; ++u)
          if (u >= shift) out[u] = o.v[u];
      } else if (p.stream_out) {
        store_vec_stream<T, VEC, !RAGGED>(out, o);  // leaves L2 to the tile loads
      } else {
        store_vec<T, VEC, !RAGGED>(out, o);
      }
    }
  }
}

}  // namespace iex
