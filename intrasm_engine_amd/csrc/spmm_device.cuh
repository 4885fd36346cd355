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
  int stream_out = 0;  // the output is far larger than the caches: store it with the streaming hint
};

// The kernel for 16-bit sparse operands with structure and 64 output columns (spmm_blocks.hip)
bool spmm_blocks_fits(int dtype, int itype, const SpmmParams& p);
bool spmm_blocks_wins(const SpmmParams& p, int batch);
size_t spmm_blocks_bytes(const SpmmParams& p);
int launch_spmm_blocks(int dtype, const SpmmParams& p, int batch, void* ws, int dense_code, int ready, hipStream_t stream);

constexpr int kSpmmUnroll = 8;

template <int VEC, int WPR, int NT = 1>
constexpr int spmm_lds_floats() { return (WPR > 1) ? WPR * kWave * VEC * NT : 1; }

template <typename T, int VEC>
__device__ __forceinline__ void fma_vec(float (&acc)[VEC], float a, const vec_t<T, VEC>& b) {
#pragma unroll
  for (int i = 0; i < VEC; ++i) acc[i] = fmaf(a, elem<T>::to_float(b.v[i]), acc[i]);
}

// NT adjacent column tiles of one dense row (NT * LPG*VEC contiguous elements).
template <typename T, int VEC, int NT>
struct row_slab {
  vec_t<T, VEC> t[NT];
};

// One wavefront's share of one row: the sums of the nonzeros in the chunks part, part + wpr, part + 2 wpr ... (64
// nonzeros each) of CSR row `row`, for the NT column tiles that start at col_ld[] (element offsets inside a dense
// row; lanes beyond n point at a valid address and their sums are never stored).  Any wpr >= 1 and any part < wpr
// give a correct partition of the row's nonzeros over the wpr wavefronts that call this for the row.
// WIN = gathers a wave keeps in flight (rolling window); raise it where few waves fit a CU.
// RAGGED = vectors at element alignment (n not a multiple of VEC).
template <typename T, typename IT, int VEC, int LPG, int WIN, int NT, bool RAGGED>
__device__ __forceinline__ void spmm_range_partial(const SpmmParams& p, int z, int start, int end, int part, int wpr, const int (&col_ld)[NT],
                                                   float (&acc)[NT][VEC]) {
  // (the row's nonzeros are start .. end - 1, wave-uniform: for a caller that has read the row's offsets already)
  constexpr int G = kWave / LPG;
  typedef row_slab<T, VEC, NT> Slab;
  const int lane = lane_id();
  const int grp = lane / LPG;   // which nonzero of a step this lane works on (0 when G == 1)
  const T* __restrict__ values =
      static_cast<const T*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
  const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
  const T* __restrict__ dense = static_cast<const T*>(p.dense) + (size_t)z * p.k * p.n;

  auto load_row = [&](int column) {
    Slab s;
    const T* r = dense + (size_t)column * p.n;
#pragma unroll
    for (int t = 0; t < NT; ++t) s.t[t] = load_vec<T, VEC, !RAGGED>(r + col_ld[t]);
    return s;
  };
  auto fma_row = [&](float a, const Slab& s) {
#pragma unroll
    for (int t = 0; t < NT; ++t) fma_vec<T, VEC>(acc[t], a, s.t[t]);
  };

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
    const int next = base + kWave * wpr;
    float v_next = 0.f;
    int c_next = 0;
    if (next + lane < end) {
      v_next = elem<T>::to_float(values[next + lane]);
      c_next = (int)cols[next + lane];
    }
    const int cnt = min(kWave, end - base);  // wave-uniform
    if constexpr (G == 1) {
      auto gather = [&](int t) { return load_row(bcast_i(c, t)); };
      if (cnt == kWave) {
        // full chunk: rolling window of WIN gathers in flight, refilled after every FMA
        Slab bv[WIN];
#pragma unroll
        for (int u = 0; u < WIN; ++u) bv[u] = gather(u);
#pragma unroll
        for (int t = 0; t < kWave; ++t) {
          fma_row(bcast_f(v, t), bv[t % WIN]);
          if (t + WIN < kWave) bv[t % WIN] = gather(t + WIN);
        }
      } else {
        int t = 0;
        for (; t + WIN <= cnt; t += WIN) {
          Slab bv[WIN];
#pragma unroll
          for (int u = 0; u < WIN; ++u) bv[u] = gather(t + u);
#pragma unroll
          for (int u = 0; u < WIN; ++u) fma_row(bcast_f(v, t + u), bv[u]);
        }
        for (; t < cnt; ++t) fma_row(bcast_f(v, t), gather(t));
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
        Slab bv[kWin];
        float vv[kWin];
#pragma unroll
        for (int u = 0; u < kWin; ++u) bv[u] = load_row(fetch(u, vv[u]));
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
          fma_row(vv[s % kWin], bv[s % kWin]);
          if (s + kWin < kSteps) bv[s % kWin] = load_row(fetch(s + kWin, vv[s % kWin]));
        }
      } else {
        const int steps = cnt / G;  // full steps: every group has a real nonzero
        int s = 0;
        for (; s + kWin <= steps; s += kWin) {
          Slab bv[kWin];
          float vv[kWin];
#pragma unroll
          for (int u = 0; u < kWin; ++u) bv[u] = load_row(fetch(s + u, vv[u]));
#pragma unroll
          for (int u = 0; u < kWin; ++u) fma_row(vv[u], bv[u]);
        }
        for (; s * G < cnt; ++s) {
          float vu;
          const int cu = fetch(s, vu);
          if (s * G + grp < cnt) fma_row(vu, load_row(cu));
        }
      }
    }
    base = next;
    v = v_next;
    c = c_next;
  }
  if constexpr (G > 1) {
    // combine the G groups: afterwards every lane holds the sum for its columns
#pragma unroll
    for (int off = LPG; off < kWave; off <<= 1) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[0][i] += __shfl_xor(acc[0][i], off, kWave);
    }
  }
}

template <typename T, typename IT, int VEC, int LPG, int WIN, int NT, bool RAGGED>
__device__ __forceinline__ void spmm_row_partial(const SpmmParams& p, int z, int row, int part, int wpr, const int (&col_ld)[NT],
                                                 float (&acc)[NT][VEC]) {
  spmm_range_partial<T, IT, VEC, LPG, WIN, NT, RAGGED>(p, z, uniform(p.row_offsets[row]), uniform(p.row_offsets[row + 1]), part, wpr, col_ld, acc);
}

// Bias, ReLU, accumulation and the store of one row's sums (lanes of group 0 only; col0 = first column of tile 0).
template <typename T, int VEC, int LPG, int NT, bool RAGGED>
__device__ __forceinline__ void spmm_store_row(const SpmmParams& p, int z, int row, int col0, int shift, float (&acc)[NT][VEC]) {
  constexpr int TW = LPG * VEC;
  const float bias = p.bias ? p.bias[row] : 0.f;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int col = col0 + t * TW;
    if (col >= p.n) continue;
    T* __restrict__ out = static_cast<T*>(p.out) + ((size_t)z * p.m + row) * p.n + col - shift;
    vec_t<T, VEC> o;
    if (p.accumulate) {
      const vec_t<T, VEC> prev = load_vec<T, VEC, !RAGGED>(out);
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc[t][i] += elem<T>::to_float(prev.v[i]);
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      float r = acc[t][i] + bias;
      if (p.relu) r = fmaxf(r, 0.f);
      o.v[i] = elem<T>::from_float(r);
    }
    if (RAGGED && shift > 0) {
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        if (i >= shift) out[i] = o.v[i];  // the elements before `shift` belong to the lane to the left
    } else if (p.stream_out) {
      store_vec_stream<T, VEC, !RAGGED>(out, o);
    } else {
      store_vec<T, VEC, !RAGGED>(out, o);
    }
  }
}

// One workgroup's share: block (bx, by, bz) of the grid
//   (ceil(m / rows_per_block), ceil(n / (NT*LPG*VEC)), batch).
// `red` must hold spmm_lds_floats<VEC,WPR,NT>() floats.  Every thread of the workgroup
// must call this when WPR > 1 (it contains a barrier).
// NT  = adjacent 64*VEC-column tiles a wave covers (G == 1 only): per nonzero the wave then
//       reads NT*64*VEC contiguous elements of one dense row, which amortises the broadcast
//       of (column, value) and keeps very wide dense operands on fewer pages.
// RAGGED = n is not a multiple of VEC: vectors are moved at element alignment, and the one lane of a
//       row whose vector would reach past the row's end reads VEC elements ending at the row's end
//       instead (shifted back by `shift`), sums all of them and stores only the ones it owns.
template <typename T, typename IT, int VEC, int LPG, int WPR, int WIN = kSpmmUnroll, int NT = 1, bool RAGGED = false>
__device__ __forceinline__ void spmm_block(const SpmmParams& p, int bx, int by, int bz, float* red) {
  static_assert(!RAGGED || (NT == 1 && LPG == kWave), "ragged rows: one full-width tile per wave");
  constexpr int kWavesPerBlock = (WPR > 4) ? WPR : 4;
  constexpr int kRowsPerBlock = kWavesPerBlock / WPR;
  constexpr int G = kWave / LPG;
  constexpr int TW = LPG * VEC;  // columns of one tile
  static_assert(NT == 1 || G == 1, "several tiles per wave need the whole wave on one nonzero");
  const int lane = lane_id();
  const int wave = uniform(threadIdx.x >> 6);
  const int z = bz;
  const int row_slot = bx * kRowsPerBlock + wave / WPR;
  const int part = wave % WPR;  // which share of the row this wave sums
  const int grp = lane / LPG;   // which nonzero of a step this lane works on (0 when G == 1)

  const int col0 = by * (NT * TW) + (lane % LPG) * VEC;  // first tile; tile t starts TW*t further
  const int shift = (RAGGED && col0 < p.n && col0 + VEC > p.n) ? col0 + VEC - p.n : 0;  // (n >= VEC, checked by the host)
  int col_ld[NT];                                         // idle lanes gather a valid address, result unused
#pragma unroll
  for (int t = 0; t < NT; ++t) col_ld[t] = (col0 + t * TW < p.n) ? col0 + t * TW - shift : 0;

  float acc[NT][VEC];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[t][i] = 0.f;

  const bool row_live = row_slot < p.m;  // wave-uniform
  int row = 0;
  if (row_live) {
    row = uniform(p.row_indices[row_slot]);
    spmm_row_partial<T, IT, VEC, LPG, WIN, NT, RAGGED>(p, z, row, part, WPR, col_ld, acc);
  }

  if constexpr (WPR > 1) {
    // Every wave of the block reaches this barrier: a block holds exactly one row when
    // WPR > 1, so row_live is uniform over the block and idle blocks fall through with
    // zero partials.
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < VEC; ++i) red[((wave * NT + t) * VEC + i) * kWave + lane] = acc[t][i];
    __syncthreads();
    if (part != 0) return;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float s = acc[t][i];
        for (int w = 1; w < WPR; ++w) s += red[(((wave + w) * NT + t) * VEC + i) * kWave + lane];
        acc[t][i] = s;
      }
  }

  if (!row_live || grp != 0) return;
  spmm_store_row<T, VEC, LPG, NT, RAGGED>(p, z, row, col0, shift, acc);
}

// ---- wavefronts per row that follow the row's own length ------------------------------------------------
// The rows come sorted by decreasing length (row_indices), so "rows that deserve 16 wavefronts, then those that deserve
// 8, 4, 2, 1" are five consecutive ranges of row slots, and a workgroup of 16 wavefronts serves 1, 2, 4, 8 or 16 rows
// of one range.  Workgroup ids run through the ranges in that order: the longest rows start first.  The ranges come
// from the host (counted once per pattern) and settle how many wavefronts a row slot HAS.  Into how many parts a row's
// nonzeros are cut, and so the order of its sum, follows from the row's own length alone: with the ranges the host
// derives from a true histogram and rows in that order the two agree; with any other ranges or order a row that has
// fewer wavefronts than parts lets one of them take all its parts, one that has more lets some idle -- time, never a
// different bit of the result.
constexpr int kRowsWaves = 16;
struct RowClasses {
  int first_row[6];     // class c (16 >> c wavefronts per row) holds row slots first_row[c] .. first_row[c + 1] - 1
  int first_block[6];   // ... served by workgroups first_block[c] .. first_block[c + 1] - 1
  int log2_rounds;      // a row of more than 64 << (3 - c + log2_rounds) nonzeros is cut into 16 >> c parts or more
};

template <int VEC>
constexpr int spmm_rows_lds_floats() { return kRowsWaves * kWave * VEC; }

template <typename T, typename IT, int VEC, int LPG>
__device__ __forceinline__ void spmm_rows_block(const SpmmParams& p, const RowClasses& rc, int bx, int by, int bz, float* red) {
  constexpr int TW = LPG * VEC;
  const int lane = lane_id();
  const int wave = uniform(threadIdx.x >> 6);
  int cls = 0;
#pragma unroll
  for (int c = 1; c < 5; ++c) cls += (bx >= rc.first_block[c]) ? 1 : 0;   // (uniform; empty classes share a first block)
  const int wpr = kRowsWaves >> cls;
  const int slot0 = rc.first_row[cls] + ((bx - rc.first_block[cls]) << cls);   // the workgroup's first row slot
  const int mine = wave / wpr;                                                  // this wavefront's row slot among them
  const int part = wave % wpr;
  const int grp = lane / LPG;
  const int col0 = by * TW + (lane % LPG) * VEC;
  int col_ld[1] = {col0 < p.n ? col0 : 0};
  float acc[1][VEC];
#pragma unroll
  for (int i = 0; i < VEC; ++i) acc[0][i] = 0.f;
  const bool row_live = slot0 + mine < rc.first_row[cls + 1];   // wave-uniform
  // (all of this is wave-uniform: scalar loads)
  auto parts_of = [&](int len) {   // of a row, by its own length
    int own = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) own += (len > (kWave << (3 - c + rc.log2_rounds))) ? 0 : 1;
    return kRowsWaves >> own;
  };
  int row = 0, start = 0, end = 0, parts = 1;
  if (row_live) {
    row = uniform(p.row_indices[slot0 + mine]);
    start = uniform(p.row_offsets[row]);
    end = uniform(p.row_offsets[row + 1]);
    parts = parts_of(end - start);
  }
  // A row slot with as many wavefronts as its row has parts, or more: a part each (the others idle), and the partial
  // sums meet in LDS.  With fewer -- only where the ranges or the order of the rows are not what the kernel expects --
  // the slot's first wavefront takes all parts, one after the other, and adds them in the same order.  Either way a
  // wavefront decides from its own row alone, and every wavefront of the workgroup reaches the one barrier.
  if (row_live) {
    if (parts <= wpr) {
      if (part < parts) spmm_range_partial<T, IT, VEC, LPG, kSpmmUnroll, 1, false>(p, bz, start, end, part, parts, col_ld, acc);
    } else if (part == 0) {
      spmm_range_partial<T, IT, VEC, LPG, kSpmmUnroll, 1, false>(p, bz, start, end, 0, parts, col_ld, acc);
      for (int q = 1; q < parts; ++q) {
        float more[1][VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) more[0][i] = 0.f;
        spmm_range_partial<T, IT, VEC, LPG, kSpmmUnroll, 1, false>(p, bz, start, end, q, parts, col_ld, more);
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[0][i] += more[0][i];
      }
    }
  }
  if (cls < 4) {   // (uniform over the workgroup) the parts of a row are added in their order: bit-stable
#pragma unroll
    for (int i = 0; i < VEC; ++i) red[(wave * VEC + i) * kWave + lane] = acc[0][i];
    __syncthreads();
    if (part != 0) return;
    if (parts <= wpr) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        float s = acc[0][i];
        for (int w = 1; w < parts; ++w) s += red[((wave + w) * VEC + i) * kWave + lane];
        acc[0][i] = s;
      }
    }
  }
  if (!row_live || grp != 0) return;
  spmm_store_row<T, VEC, LPG, 1, false>(p, bz, row, col0, 0, acc);
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
// a mean of a few dozen nonzeros per row upwards (8 or 16 waves per row were slower) -- as long
// as whole rows would leave the chip short of wavefronts.  With more than one full round of
// wavefronts (256 CUs x 32) from whole rows alone, splitting only adds the partial sums' trip
// through LDS: 16 heads of 4096 x 4096 at 93 % sparsity, n = 64, fp16: 163 us split, 93 us whole.
// elem_size, n and batch size the launch: lanes per row = n / (elements per 128-bit vector),
// at least 8; 64 / that many rows share a wavefront.
inline int spmm_pick_wpr(int m, int nnz, int elem_size = 4, int n = 0, int batch = 1) {
  const double mean = m > 0 ? (double)nnz / m : 0.0;
  if (mean < 24.0) return 1;
  if (n > 0) {
    const int vec = 16 / elem_size;
    int lanes = 8;
    while (lanes < kWave && lanes * vec < n) lanes <<= 1;
    const long long tiles_n = (n + kWave * vec - 1) / (kWave * vec);
    const long long waves = ((long long)m * lanes + kWave - 1) / kWave * tiles_n * batch;
    if (waves >= 256 * 32) return 1;
  }
  return 4;
}

// Defined with the dispatcher (spmm.hip): register windows of the 8-wave matrix-core kernel if
// that is what an fp16 SpMM of this shape runs on, else 0.
int spmm_matrix_core_windows(const SpmmParams& p);

}  // namespace iex
