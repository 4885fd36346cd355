// CSR SpMM with the dense operand staged through LDS (gfx950, wave64).
//
// The row kernel of spmm_device.cuh gathers every dense row it needs from L2: nnz * tile
// bytes of L2 -> CU traffic, which is what bounds it.  When a block of rows shares a dense
// row often enough (density * rows-per-workgroup of a dozen or more), or when the slice of
// the dense operand that the row kernel keeps re-reading no longer fits an XCD's L2 (large
// k), it is cheaper to stream the dense operand through LDS once per workgroup and gather
// from LDS, whose gather bandwidth is about three times that of L2 on this part.  The kernel
// is then bound by vector-ALU issue (8 FMAs + 3 bookkeeping instructions per nonzero and
// 128-bit column vector).
//
// Workgroup = 8 wavefronts, owns RB = 8 * RPW consecutive CSR rows (swizzled order, so rows
// of similar length share a workgroup) and one tile of 64*VEC output columns.
//   for each block of KB dense rows (KB * tile bytes = 64 KB):
//     all threads copy dense[kb0 : kb0+KB, tile] into LDS (the global loads of block i+1 are
//     issued before block i is processed and land in registers meanwhile);
//     every wave walks its RPW rows: column indices are ascending inside a row, so the
//     nonzeros that fall into this block are a contiguous run found with one ballot; each
//     one is a v_readlane broadcast of (column, value) and one LDS read of VEC elements.
// A row keeps its current 64 nonzeros in two VGPRs (one per lane) plus the next 64
// prefetched.  Two workgroups fit a CU (2 x 64 KB of the 160 KB LDS), so one stages while the
// other gathers.  fp32 accumulation; deterministic; padding slots are never dereferenced.
#pragma once
#include "spmm_device.cuh"

namespace iex {

constexpr int kLdsWaves = 8;
constexpr int kLdsThreads = kLdsWaves * kWave;
constexpr int kLdsTileBytes = 64 * 1024;

template <typename T, int VEC>
constexpr int spmm_lds_kb() { return kLdsTileBytes / (kWave * VEC * (int)sizeof(T)); }

template <typename T, typename IT, int VEC, int RPW>
__device__ __forceinline__ void spmm_lds_block(const SpmmParams& p, int bx, int by, int bz, unsigned char* smem) {
  constexpr int KB = spmm_lds_kb<T, VEC>();              // dense rows per stage
  constexpr int kUnits = KB * kWave;                     // VEC-element units per stage
  constexpr int kUnitsPerThread = kUnits / kLdsThreads;  // 8 for every (T, VEC)
  typedef vec_t<T, VEC> V;
  V* tile = reinterpret_cast<V*>(smem);                  // [KB][64]

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = uniform(tid >> 6);
  const int z = bz;
  const int col0 = by * (kWave * VEC) + lane * VEC;
  const bool lane_live = col0 < p.n;

  const T* __restrict__ values = static_cast<const T*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
  const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
  const T* __restrict__ dense = static_cast<const T*>(p.dense) + (size_t)z * p.k * p.n;

  // ---- per-row state (RPW rows per wave, statically indexed) ------------------------
  int row[RPW], end[RPW], nbase[RPW], pos[RPW], cnt[RPW];
  float v[RPW], vn[RPW];
  int c[RPW], cn[RPW];
  float acc[RPW][VEC];
  constexpr int kNoCol = 0x7fffffff;
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int slot = (bx * kLdsWaves + wave) * RPW + r;
    row[r] = -1;
    end[r] = nbase[r] = pos[r] = cnt[r] = 0;
    v[r] = vn[r] = 0.f;
    c[r] = cn[r] = kNoCol;
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[r][i] = 0.f;
    if (slot < p.m) {
      row[r] = uniform(p.row_indices[slot]);
      const int start = uniform(p.row_offsets[row[r]]);
      end[r] = uniform(p.row_offsets[row[r] + 1]);
      cnt[r] = min(kWave, end[r] - start);
      if (start + lane < end[r]) {
        v[r] = elem<T>::to_float(values[start + lane]);
        c[r] = (int)cols[start + lane];
      }
      nbase[r] = start + kWave;
      if (nbase[r] + lane < end[r]) {
        vn[r] = elem<T>::to_float(values[nbase[r] + lane]);
        cn[r] = (int)cols[nbase[r] + lane];
      }
    }
  }

  // ---- staging: unit u of a stage = dense[kb0 + u / 64][tile column (u % 64) * VEC ..] ---
  V stage[kUnitsPerThread];
  auto load_stage = [&](int kb0) {
#pragma unroll
    for (int i = 0; i < kUnitsPerThread; ++i) {
      const int u = i * kLdsThreads + tid;
      const int kr = kb0 + u / kWave;
      const int cc = by * (kWave * VEC) + (u % kWave) * VEC;
      if (kr < p.k && cc < p.n) {
        stage[i] = load_vec<T, VEC>(dense + (size_t)kr * p.n + cc);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) stage[i].v[e] = elem<T>::from_float(0.f);
      }
    }
  };
  auto store_stage = [&]() {
#pragma unroll
    for (int i = 0; i < kUnitsPerThread; ++i) tile[i * kLdsThreads + tid] = stage[i];
  };

  load_stage(0);
  for (int kb0 = 0; kb0 < p.k; kb0 += KB) {
    __syncthreads();  // every wave is done gathering from the previous stage
    store_stage();
    __syncthreads();
    if (kb0 + KB < p.k) load_stage(kb0 + KB);  // lands while this stage is processed
    const int kb_end = kb0 + KB;
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      if (row[r] < 0) continue;  // wave-uniform
      while (true) {
        // ascending columns: the nonzeros of this chunk that fall into [kb0, kb_end) are the
        // run that starts at pos
        const unsigned long long inb = __ballot(lane >= pos[r] && lane < cnt[r] && c[r] < kb_end);
        const int num = __popcll(inb);
        int t = pos[r];
        const int te = t + num;
        for (; t + 4 <= te; t += 4) {  // (8 in flight measured no faster and costs registers)
          V bv[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) bv[u] = tile[(bcast_i(c[r], t + u) - kb0) * kWave + lane];
#pragma unroll
          for (int u = 0; u < 4; ++u) fma_vec<T, VEC>(acc[r], bcast_f(v[r], t + u), bv[u]);
        }
        for (; t < te; ++t) fma_vec<T, VEC>(acc[r], bcast_f(v[r], t), tile[(bcast_i(c[r], t) - kb0) * kWave + lane]);
        pos[r] = te;
        if (te < cnt[r] || nbase[r] >= end[r]) break;  // next nonzero lies beyond this stage, or the row is done
        // chunk exhausted: the prefetched one becomes current, prefetch the one after it
        v[r] = vn[r];
        c[r] = cn[r];
        cnt[r] = min(kWave, end[r] - nbase[r]);
        pos[r] = 0;
        nbase[r] += kWave;
        vn[r] = 0.f;
        cn[r] = kNoCol;
        if (nbase[r] + lane < end[r]) {
          vn[r] = elem<T>::to_float(values[nbase[r] + lane]);
          cn[r] = (int)cols[nbase[r] + lane];
        }
      }
    }
  }

  if (!lane_live) return;
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    if (row[r] < 0) continue;
    const float bias = p.bias ? p.bias[row[r]] : 0.f;
    T* __restrict__ out = static_cast<T*>(p.out) + ((size_t)z * p.m + row[r]) * p.n + col0;
    if (p.accumulate) {
      const V prev = load_vec<T, VEC>(out);
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[r][i] += elem<T>::to_float(prev.v[i]);
    }
    V o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float x = acc[r][i] + bias;
      if (p.relu) x = fmaxf(x, 0.f);
      o.v[i] = elem<T>::from_float(x);
    }
    store_vec<T, VEC>(out, o);
  }
}

}  // namespace iex
