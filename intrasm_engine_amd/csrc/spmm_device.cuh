// CSR SpMM device code for gfx950 (wave64): out[z, r, :] = sum_j values[j] * dense[z, col[j], :].
//
// Work decomposition
//   * a wavefront owns one CSR row (taken in swizzled order: heavy rows are launched
//     first) and one tile of LPG*VEC output columns.  The 64 lanes form G = 64/LPG groups
//     of LPG lanes; lane l of a group owns VEC adjacent columns, so a group gathers one
//     dense row as one contiguous LPG*VEC*sizeof(T) access (128-bit per lane whenever the
//     shape allows) and the G groups work on G different nonzeros at the same time.
//     Wide outputs use G = 1 (the whole wave on one nonzero), narrow ones (n = 64 fp32:
//     LPG = 16, G = 4) keep every lane busy with full-width loads;
//   * values / column indices are read 64 nonzeros at a time, one per lane (coalesced).
//     With G = 1 they are handed to the wave through v_readlane: column index and value of
//     the current nonzero live in scalar registers, the address arithmetic runs on the
//     scalar unit and the vector unit only issues the gather and the FMAs.  With G > 1
//     each group fetches its nonzero with ds_bpermute and the G partial sums are combined
//     once per row with cross-lane shuffles;
//   * long rows are split over WPR wavefronts of one workgroup (chunks of 64 nonzeros
//     dealt round-robin); partial sums meet in LDS, so the result is deterministic and
//     needs no atomics.
// Accumulation is fp32 for every element type.  Padding slots are never dereferenced.
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

constexpr int kSpmmUnroll = 8;

template <int VEC, int WPR>
constexpr int spmm_lds_floats() { return (WPR > 1) ? WPR * kWave * VEC : 1; }

template <typename T, int VEC>
__device__ __forceinline__ void fma_vec(float (&acc)[VEC], float a, const vec_t<T, VEC>& b) {
#pragma unroll
  for (int i = 0; i < VEC; ++i) acc[i] = fmaf(a, elem<T>::to_float(b.v[i]), acc[i]);
}

// One workgroup's share: block (bx, by, bz) of the grid
//   (ceil(m / rows_per_block), ceil(n / (LPG*VEC)), batch).
// `red` must hold spmm_lds_floats<VEC,WPR>() floats.  Every thread of the workgroup
// must call this when WPR > 1 (it contains a barrier).
// WIN = gathers a wave keeps in flight (rolling window); raise it where few waves fit a CU.
template <typename T, typename IT, int VEC, int LPG, int WPR, int WIN = kSpmmUnroll>
__device__ __forceinline__ void spmm_block(const SpmmParams& p, int bx, int by, int bz, float* red) {
  constexpr int kWavesPerBlock = (WPR > 4) ? WPR : 4;
  constexpr int kRowsPerBlock = kWavesPerBlock / WPR;
  constexpr int G = kWave / LPG;
  const int lane = lane_id();
  const int wave = uniform(threadIdx.x >> 6);
  const int z = bz;
  const int row_slot = bx * kRowsPerBlock + wave / WPR;
  const int part = wave % WPR;  // which share of the row this wave sums
  const int grp = lane / LPG;   // which nonzero of a step this lane works on (0 when G == 1)

  const int col0 = by * (LPG * VEC) + (lane % LPG) * VEC;
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
    const T* __restrict__ values =
        static_cast<const T*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
    const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
    const T* __restrict__ dense = static_cast<const T*>(p.dense) + (size_t)z * p.k * p.n + col_ld;

    // (value, column) of nonzero base+lane; the next chunk is fetched while the current
    // one is being processed, so its latency hides behind the gathers.
    int base = start + part * kWave;
    float v = 0.f;
    int c = 0;
    if (base + lane < end) {
      v = elem<T>::to_float(values[base + lane]);
      c = (int)cols[base + lane];
    }
    while (base < end) {
      const int next = base + kWave * WPR;
      float v_next = 0.f;
      int c_next = 0;
      if (next + lane < end) {
        v_next = elem<T>::to_float(values[next + lane]);
        c_next = (int)cols[next + lane];
      }
      const int cnt = min(kWave, end - base);  // wave-uniform
      if constexpr (G == 1) {
        auto gather = [&](int t) { return load_vec<T, VEC>(dense + (size_t)bcast_i(c, t) * p.n); };
        if (cnt == kWave) {
          // full chunk: rolling window of WIN gathers in flight, refilled after every FMA
          vec_t<T, VEC> bv[WIN];
#pragma unroll
          for (int u = 0; u < WIN; ++u) bv[u] = gather(u);
#pragma unroll
          for (int t = 0; t < kWave; ++t) {
            fma_vec<T, VEC>(acc, bcast_f(v, t), bv[t % WIN]);
            if (t + WIN < kWave) bv[t % WIN] = gather(t + WIN);
          }
        } else {
          int t = 0;
          for (; t + WIN <= cnt; t += WIN) {
            vec_t<T, VEC> bv[WIN];
#pragma unroll
            for (int u = 0; u < WIN; ++u) bv[u] = gather(t + u);
#pragma unroll
            for (int u = 0; u < WIN; ++u) fma_vec<T, VEC>(acc, bcast_f(v, t + u), bv[u]);
          }
          for (; t < cnt; ++t) fma_vec<T, VEC>(acc, bcast_f(v, t), gather(t));
        }
      } else {
        // step s: group g works on nonzero s*G + g of this chunk
        constexpr int kSteps = kWave / G;
        constexpr int kWin = kSteps < WIN ? kSteps : WIN;
        auto fetch = [&](int s, float& vs) {
          const int src = ((s * G + grp) & (kWave - 1)) << 2;
          vs = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(v)));
          return __builtin_amdgcn_ds_bpermute(src, c);
        };
        if (cnt == kWave) {
          vec_t<T, VEC> bv[kWin];
          float vv[kWin];
#pragma unroll
          for (int u = 0; u < kWin; ++u) bv[u] = load_vec<T, VEC>(dense + (size_t)fetch(u, vv[u]) * p.n);
#pragma unroll
          for (int s = 0; s < kSteps; ++s) {
            fma_vec<T, VEC>(acc, vv[s % kWin], bv[s % kWin]);
            if (s + kWin < kSteps) bv[s % kWin] = load_vec<T, VEC>(dense + (size_t)fetch(s + kWin, vv[s % kWin]) * p.n);
          }
        } else {
          const int steps = cnt / G;  // full steps: every group has a real nonzero
          int s = 0;
          for (; s + kWin <= steps; s += kWin) {
            vec_t<T, VEC> bv[kWin];
            float vv[kWin];
#pragma unroll
            for (int u = 0; u < kWin; ++u) bv[u] = load_vec<T, VEC>(dense + (size_t)fetch(s + u, vv[u]) * p.n);
#pragma unroll
            for (int u = 0; u < kWin; ++u) fma_vec<T, VEC>(acc, vv[u], bv[u]);
          }
          for (; s * G < cnt; ++s) {
            float vu;
            const int cu = fetch(s, vu);
            if (s * G + grp < cnt) fma_vec<T, VEC>(acc, vu, load_vec<T, VEC>(dense + (size_t)cu * p.n));
          }
        }
      }
      base = next;
      v = v_next;
      c = c_next;
    }
  }

  if constexpr (G > 1) {
    // combine the G groups: afterwards every lane holds the sum for its columns
#pragma unroll
    for (int off = LPG; off < kWave; off <<= 1) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[i] += __shfl_xor(acc[i], off, kWave);
    }
  }

  if constexpr (WPR > 1) {
    // Every wave of the block reaches this barrier: a block holds exactly one row when
    // WPR > 1, so row_live is uniform over the block and idle blocks fall through with
    // zero partials.
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

  if (!row_live || !lane_live || grp != 0) return;
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

// Host-side shape choice shared by the stand-alone and the fused launcher.
// VEC: widest per-lane vector that divides n and keeps rows aligned.  LPG: lanes per
// nonzero; below 64 only for full 128-bit vectors (narrow outputs then run several
// nonzeros per wave instead of idling lanes).
struct SpmmShape {
  int vec, lpg;
};
template <typename T>
inline SpmmShape spmm_pick_shape(int n, const void* dense, const void* out) {
  constexpr int kMax = 16 / (int)sizeof(T);
  int vec = kMax;
  while (vec > 1 && (n % vec != 0 || !aligned(dense, sizeof(T) * vec) || !aligned(out, sizeof(T) * vec))) vec >>= 1;
  int lpg = kWave;
  if (vec == kMax) {
    while (lpg > 8 && (lpg / 2) * vec >= n) lpg >>= 1;
  } else {
    while (vec > 1 && kWave * vec / 2 >= n) vec >>= 1;  // narrow, unaligned shapes: shrink the vector instead
  }
  return {vec, lpg};
}

// Waves per row from the mean row length.  Splitting a row over the 4 wavefronts of a
// workgroup shortens the dependent chain "fetch 64 nonzeros -> gather" of the heaviest row,
// which is what the kernel time of a skewed matrix follows; measured on MI355X it wins from
// a mean of a few dozen nonzeros per row upwards (8 or 16 waves per row were slower).
inline int spmm_pick_wpr(int m, int nnz) {
  const double mean = m > 0 ? (double)nnz / m : 0.0;
  return mean >= 24.0 ? 4 : 1;
}

}  // namespace iex
