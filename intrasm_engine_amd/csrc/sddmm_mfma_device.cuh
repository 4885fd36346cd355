// CSR SDDMM for attention-like masks (gfx950, fp16 / bf16, k = 32, 64 or 128): where the mask is dense the scores
// come from the matrix cores, tile by tile, and are sampled inside the workgroup without ever being stored; where it
// is thin the few dot products are computed one by one.
//
// The gather kernel (sddmm.hip) reads k * 2 bytes of rhs per nonzero through the L2 -> CU path; for an attention
// mask (a dense band plus scattered entries, 5-10 % dense) that is 2.4 GB per 16 heads and that path is what bounds
// it.  A dense product of everything (34 GFLOP) is cheap on the matrix cores but wasted on the nine tenths of the
// 128 x 128 tiles that hold one entry per row.  So a workgroup (4 wavefronts) owns 128 consecutive rows of one batch
// entry, and the column tiles (128 columns each) of its rows are sorted by how many nonzeros they hold:
//   * dense tiles (dense_min nonzeros or more in the 128 x 128 block): the rhs rows of the tile come from global
//     memory straight into LDS (global_load_lds_dwordx4, double-buffered, 16-byte chunks permuted so that the
//     operand reads are conflict-free), 2 x 2 x k/16 MFMAs of 32 x 32 x 16 per wavefront (each owns 64 x 64 of the
//     tile; the lhs fragments stay in registers for the whole phase), operands swapped so that a lane ends up with
//     4 adjacent columns of one row and writes them to the score tile in LDS with one 64-bit store, already rounded
//     to the element type.  Sampling, two ways per (row, tile): up to 4 nonzeros -> the row's own lane (threads
//     0..127) copies the scores named by a packed word; more -> a wavefront takes four rows at a time, 16 lanes per
//     row: a 128-bit mask of the row's columns in the tile tells each lane which of its 8 columns are present and, by
//     a population count of the bits below, where in the row's output they go; all 8 present is one 16-byte store.
//     No column index is read from memory in this phase.
//   * the nonzeros elsewhere: k / 8 lanes per row walk the row's list of them (column, position in the output), the
//     row's lhs in registers: 16 bytes of the rhs row per lane from memory, v_dot2 in fp32, summed across the lanes,
//     rounded once, stored at the position.
// What the kernel needs to know about the mask comes from two small kernels that run first, once per call for all
// batch entries, into the caller's workspace (functions of the index arrays only: a caller whose mask stays keeps
// them): the tables -- tile_ptr[t][row] = position of the row's first nonzero with column >= 128 t (columns ascend
// inside a row), brief[t][row] = count and in-tile columns of up to 4 nonzeros, packed in one word, and
// mask[t][row] for the pairs with more -- and, from the tables, the lists: per block of 128 rows its dense tiles,
// per row its nonzeros outside them, compacted.  The SpMM for the same patterns (spmm_blocks_device.cuh) reads both.
// The dense phase runs on a hand-counted pipeline: all its global reads (rhs rows for the next dense tile, the
// per-row words two dense tiles ahead) are direct-to-LDS loads in inline assembly, invisible to the compiler's
// wait-count pass; each wavefront issues a fixed number of them per tile and waits with s_waitcnt vmcnt(N), N =
// the loads it issued after the ones it needs (the counter retires loads in order, and the stores of the previous
// tile's sampling are older than these loads, so nothing ever waits for the current tile's stores).  The
// workgroup barriers in that loop wait for LDS traffic only.
#pragma once
#include "gemm_dma_device.cuh"

namespace iex {

constexpr int kSdBM = 128, kSdBN = 128, kSdThreads = 256;
constexpr int kSdShort = 4;           // nonzeros of a (row, tile) pair that the row's own lane samples
constexpr int kSdLd = kSdBN + 8;      // halves per row of the score tile (272 bytes)
constexpr int kSdMaxTiles = 512;      // column tiles per row (n <= 65536): the tile list lives in LDS
// Nonzeros in a 128 x 128 block from which it counts as dense (matrix cores).  Measured on unstructured masks (16 heads of
// 4096 x 4096, every block alike): laying a block out / sampling it costs the same whatever it holds, the nonzeros taken one
// by one cost per nonzero; the two meet near 1150 nonzeros per block for the SpMM and near 1650 for the SDDMM, and the lists
// are shared by both.  On config 3 (band + scattered) 1024 .. 1792 give the same times, 2048 two microseconds more for the SpMM.
constexpr int kSdDenseMin = 1536;
constexpr int kSdSlot = kSdBM * (4 + 4 + 16);   // bytes of per-row words of one dense tile: cursor, packed word, mask

struct SddmmMfmaParams {
  int m, k, n, nnz;
  const int* cols;
  const void* lhs;
  const void* rhs;
  void* out;
  const u32x4* mask;     // [tiles_n][m], written only where brief says "more than kSdShort"
  const int* tile_ptr;   // [(tiles_n + 1)][m]
  const int* brief;      // [tiles_n][m]
  int tiles_n;
  const int* row_offsets;
  const struct SbEntry* thin_ent;     // lists (see SbLists below)
  const int* thin_cnt;
  const unsigned short* dense_list;
};

// Workgroup barrier for LDS traffic only.  __syncthreads() also waits until the thread's global stores have
// reached L2; in a loop that stores every iteration that is a round trip to L2 per iteration.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// 4 bytes per lane from global memory straight into LDS at lds_base_uniform + 4 * lane.
__device__ __forceinline__ void lds_dma4(const void* g, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off" ::"v"(g), "s"(lds_base_uniform) : "memory", "m0");
}

template <int CTRL>
__device__ __forceinline__ unsigned dpp_u(unsigned v) {
  return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
__device__ __forceinline__ unsigned wave_sum_u(unsigned v) {
  v += dpp_u<0xB1>(v);
  v += dpp_u<0x4E>(v);
  v += dpp_u<0x141>(v);
  v += dpp_u<0x140>(v);
  return (unsigned)bcast_i((int)v, 0) + (unsigned)bcast_i((int)v, 16) + (unsigned)bcast_i((int)v, 32) + (unsigned)bcast_i((int)v, 48);
}

template <int KS>
constexpr int sddmm_mfma_lds_bytes() {
  return kSdBM * kSdLd * 2 + 2 * kSdBN * KS * 32 + 3 * kSdSlot + 16;
}

// Words of workspace per call: masks first (16-byte entries), then the cursors, then the packed words.
inline size_t sddmm_mfma_words(int m, int tiles_n) { return (size_t)m * (4 * (size_t)tiles_n + (tiles_n + 1) + tiles_n); }

// tile_ptr[t][row] for t = 0 .. tiles_n, brief[t][row] and (where needed) mask[t][row] for t < tiles_n: one
// wavefront per row.  brief packs what a lane needs to sample a (row, tile) pair without touching the column indices
// again: bits 28..30 = number of nonzeros of the row in the tile (0..4, or 7 for "more"), bits 7u .. 7u + 6 =
// column of nonzero u inside the tile.  The mask of a pair with more has bit c set when column 128 t + c is present,
// and its packed word then holds the number of nonzeros in the first 32, 64 and 96 columns of the tile (bits 0..5,
// 6..12, 13..19).
// The row's columns are first marked in a bit map in LDS (n bits); counts, cursors and packed words come from the
// map, 64 tiles at a time, one tile per lane.
// A row's cursors, packed words and masks from its bit map (one wavefront; the map is complete and visible to it).
__device__ __forceinline__ void sd_row_tables(const unsigned* mine, int lane, int r, int m, int tiles_n, int s, int e,
                                              int* __restrict__ tile_ptr, int* __restrict__ brief, u32x4* __restrict__ mask) {
  int running = s;   // position of the first nonzero of tile base_t
  for (int base_t = 0; base_t < tiles_n; base_t += kWave) {
    const int t = base_t + lane;
    const bool in = t < tiles_n;
    u32x4 w = {0u, 0u, 0u, 0u};
    if (in) w.x = mine[t * 4], w.y = mine[t * 4 + 1], w.z = mine[t * 4 + 2], w.w = mine[t * 4 + 3];
    const int count = __popc(w.x) + __popc(w.y) + __popc(w.z) + __popc(w.w);
    int upto = count;   // inclusive prefix sum over the 64 tiles
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int v = __shfl_up(upto, d, kWave);
      if (lane >= d) upto += v;
    }
    if (in) {
      tile_ptr[(size_t)t * m + r] = running + upto - count;
      int word = (count <= kSdShort ? count : 7) << 28;
      if (count > kSdShort) {
        mask[(size_t)t * m + r] = w;
        const int cx = __popc(w.x), cy = cx + __popc(w.y), cz = cy + __popc(w.z);
        word |= cx | (cy << 6) | (cz << 13);
      } else {
        unsigned left[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int u = 0; u < kSdShort; ++u) {   // the u-th lowest set bit of the 128
          int at = -1;
#pragma unroll
          for (int q = 3; q >= 0; --q)
            if (left[q]) at = q;
          if (at >= 0) {
            const unsigned v = at == 0 ? left[0] : at == 1 ? left[1] : at == 2 ? left[2] : left[3];
            word |= (at * 32 + __builtin_ctz(v)) << (7 * u);
#pragma unroll
            for (int q = 0; q < 4; ++q)
              if (q == at) left[q] = v & (v - 1);
          }
        }
      }
      brief[(size_t)t * m + r] = word;
    }
    running += __builtin_amdgcn_readlane(upto, kWave - 1);
  }
  if (lane == 0) tile_ptr[(size_t)tiles_n * m + r] = e;
}

static __global__ __launch_bounds__(256) void sddmm_tile_ptr_kernel(int m, int tiles_n, const int* __restrict__ row_offsets,
                                                             const int* __restrict__ cols, int* __restrict__ tile_ptr,
                                                             int* __restrict__ brief, u32x4* __restrict__ mask) {
  __shared__ unsigned bits[4][kSdMaxTiles * 4];
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int r = blockIdx.x * 4 + wave;
  if (r >= m) return;   // (no workgroup barrier below: every wavefront works alone)
  unsigned* mine = bits[wave];
  const int s = uniform(row_offsets[r]), e = uniform(row_offsets[r + 1]);
  for (int i = lane; i < tiles_n * 4; i += kWave) mine[i] = 0;
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
  for (int base = s; base < e; base += 4 * kWave) {   // four loads in flight
    int c[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = base + u * kWave + lane;
      c[u] = j < e ? cols[j] : -1;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (c[u] >= 0) atomicOr(&mine[min(c[u] >> 5, tiles_n * 4 - 1)], 1u << (c[u] & 31));
  }
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
  sd_row_tables(mine, lane, r, m, tiles_n, s, e, tile_ptr, brief, mask);
}

// Where the three tables sit in a workspace of sddmm_mfma_words(m, tiles_n) words, and the launch that fills them.
struct SdTables {
  u32x4* mask;
  int* tile_ptr;
  int* brief;
};
inline SdTables sd_tables(void* workspace, int m, int tiles_n) {
  SdTables t;
  t.mask = static_cast<u32x4*>(workspace);
  t.tile_ptr = reinterpret_cast<int*>(t.mask + (size_t)tiles_n * m);
  t.brief = t.tile_ptr + (size_t)(tiles_n + 1) * m;
  return t;
}
inline int sd_write_tables(const SdTables& t, int m, int tiles_n, const int* row_offsets, const int* cols, hipStream_t stream) {
  note_kernel("sddmm_tile_ptr_kernel");
  hipLaunchKernelGGL(sddmm_tile_ptr_kernel, dim3(ceil_div(m, 4)), dim3(256), 0, stream, m, tiles_n, row_offsets, cols, t.tile_ptr, t.brief, t.mask);
  return check_hip(hipGetLastError(), "row-cursor launch");
}

// Which column tiles of the workgroup's 128 rows (row0 ..) are dense: nonzeros of the rows in tile t = sum over the
// rows of tile_ptr[t + 1] - tile_ptr[t].  Leaves the dense tiles, ascending, at the front of list[0 .. tiles_n) and
// the others, descending, at its back, and their number in *n_dense.  colsum: tiles_n + 1 words of LDS that the
// caller may reuse afterwards.  All 256 threads call it (it holds two workgroup barriers, the last one at its end).
__device__ __forceinline__ void sd_sort_tiles(const int* __restrict__ tile_ptr, int m, int tiles_n, int row0, int dense_min,
                                              unsigned* colsum, unsigned short* list, int* n_dense) {
  typedef unsigned short u16;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int ra = min(row0 + lane, m - 1), rb = min(row0 + kWave + lane, m - 1);
  for (int t0 = wave; t0 <= tiles_n; t0 += 32) {   // 8 tiles per step: 16 loads in flight
    unsigned v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int t = min(t0 + 4 * u, tiles_n);
      v[u] = (row0 + lane < m ? (unsigned)tile_ptr[(size_t)t * m + ra] : 0u) + (row0 + kWave + lane < m ? (unsigned)tile_ptr[(size_t)t * m + rb] : 0u);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const unsigned sum = wave_sum_u(v[u]);
      if (lane == 0 && t0 + 4 * u <= tiles_n) colsum[t0 + 4 * u] = sum;
    }
  }
  __syncthreads();
  if (wave == 0) {
    int nd = 0, ns = 0;
    for (int base = 0; base < tiles_n; base += kWave) {
      const int t = base + lane;
      const bool in = t < tiles_n;
      const int tc = min(t, tiles_n - 1);
      const bool dense = in && (int)(colsum[tc + 1] - colsum[tc]) >= dense_min;
      const unsigned long long dm = __ballot(dense), sm = __ballot(in && !dense);
      const unsigned long long below = (1ull << lane) - 1;
      if (dense) list[nd + __popcll(dm & below)] = (u16)t;
      if (in && !dense) list[tiles_n - 1 - ns - __popcll(sm & below)] = (u16)t;
      nd += __popcll(dm);
      ns += __popcll(sm);
    }
    if (lane == 0) *n_dense = nd;
  }
  __syncthreads();
}

constexpr int kSbZeroWords = 64;               // 256 bytes of zeros: what the lanes of an absent nonzero read

struct SbEntry {
  int col, pos;   // column of a nonzero outside the dense tiles and its position in the CSR arrays
};

// Behind the tables in the same workspace: the lists that depend on which tiles count as dense (read by the SDDMM
// below and by the SpMM for the same patterns, spmm_blocks_device.cuh).
struct SbLists {
  unsigned* zeros;                  // [kSbZeroWords]
  SbEntry* thin_ent;                // [nnz]: row r's entries outside dense tiles, in row order, from thin_ent[row_offsets[r]]
  int* thin_cnt;                    // [m]: how many
  unsigned short* dense_list;       // [row blocks][tiles_k + 2]: number of dense tiles of the 128 rows, then the tiles, ascending
};
inline size_t sb_lists_offset_words(int m, int tiles_k) { return (sddmm_mfma_words(m, tiles_k) + 3) & ~size_t(3); }
inline size_t sb_words(int m, int tiles_k, int nnz) {
  return sb_lists_offset_words(m, tiles_k) + kSbZeroWords + 2 * (size_t)nnz + m + ((size_t)ceil_div(m, kSdBM) * (tiles_k + 2) + 1) / 2;
}
inline SbLists sb_lists(void* workspace, int m, int tiles_k, int nnz) {
  SbLists l;
  l.zeros = static_cast<unsigned*>(workspace) + sb_lists_offset_words(m, tiles_k);
  l.thin_ent = reinterpret_cast<SbEntry*>(l.zeros + kSbZeroWords);
  l.thin_cnt = reinterpret_cast<int*>(l.thin_ent + nnz);
  l.dense_list = reinterpret_cast<unsigned short*>(l.thin_cnt + m);
  return l;
}


// The lists, one wavefront per row (4 rows per workgroup, all in one block of 128 rows).  Every workgroup first sorts the
// column tiles of its block of rows into dense and other (33 x 128 cursors out of L2: cheaper than a launch of its own
// for the 32 blocks); the workgroup with the block's first rows also writes that list: dense_list[block][0] = number of
// dense tiles, then the tiles.  Then each wavefront compacts the nonzeros of its row that lie outside the dense tiles,
// in row order: column and position in the CSR arrays.
static __global__ __launch_bounds__(kSdThreads) void sb_lists_kernel(int m, int tiles_k, int dense_min, const int* __restrict__ tile_ptr,
                                                                     const int* __restrict__ row_offsets, const int* __restrict__ cols,
                                                                     unsigned short* __restrict__ dense_list, unsigned* __restrict__ zeros,
                                                                     int* __restrict__ thin_cnt, SbEntry* __restrict__ thin_ent) {
  __shared__ unsigned colsum[kSdMaxTiles + 1];
  __shared__ unsigned short list[kSdMaxTiles];
  __shared__ int n_dense;
  __shared__ unsigned is_dense[kSdMaxTiles / 32];
  const int lane = lane_id();
  const int wave = threadIdx.x >> 6;
  const int r = blockIdx.x * 4 + wave;
  const int block = (blockIdx.x * 4) / kSdBM;
  if (threadIdx.x < kSdMaxTiles / 32) is_dense[threadIdx.x] = 0;
  sd_sort_tiles(tile_ptr, m, tiles_k, block * kSdBM, dense_min, colsum, list, &n_dense);
  const int nd = n_dense;
  if ((blockIdx.x * 4) % kSdBM == 0) {
    unsigned short* mine = dense_list + (size_t)block * (tiles_k + 2);
    if (threadIdx.x == 0) mine[0] = (unsigned short)nd;
    for (int i = threadIdx.x; i < nd; i += kSdThreads) mine[1 + i] = list[i];
  }
  if (blockIdx.x == 0 && threadIdx.x < kSbZeroWords) zeros[threadIdx.x] = 0u;
  for (int i = threadIdx.x; i < nd; i += kSdThreads) {
    const int t = list[i];
    atomicOr(&is_dense[t >> 5], 1u << (t & 31));
  }
  __syncthreads();
  if (r >= m) return;   // (no workgroup barrier below: every wavefront works alone)
  const int s = uniform(row_offsets[r]), e = uniform(row_offsets[r + 1]);
  int count = 0;
  for (int base = s; base < e; base += 4 * kWave) {   // four loads in flight
    int c[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = base + u * kWave + lane;
      c[u] = j < e ? cols[j] : -1;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int t = min(max(c[u], 0) >> 7, tiles_k - 1);
      const bool thin = c[u] >= 0 && !((is_dense[t >> 5] >> (t & 31)) & 1);
      const unsigned long long b = __ballot(thin);
      if (thin) {
        SbEntry en;
        en.col = c[u];
        en.pos = base + u * kWave + lane;
        thin_ent[s + count + __popcll(b & ((1ull << lane) - 1))] = en;
      }
      count += __popcll(b);
    }
  }
  if (lane == 0) thin_cnt[r] = count;
}

inline int sb_write_lists(const SdTables& t, const SbLists& l, int m, int tiles_n, int dense_min, const int* row_offsets, const int* cols, hipStream_t stream) {
  note_kernel("sb_lists_kernel");
  hipLaunchKernelGGL(sb_lists_kernel, dim3(ceil_div(m, 4)), dim3(kSdThreads), 0, stream, m, tiles_n, dense_min, t.tile_ptr, row_offsets, cols, l.dense_list,
                     l.zeros, l.thin_cnt, l.thin_ent);
  return check_hip(hipGetLastError(), "list kernel launch");
}

// dense_code (for tests and tuning): 0 = the built-in threshold, 1 = every tile on the matrix cores, 255 = none, else
// 64 * code nonzeros per 128 x 128 block.
inline int sb_dense_min(int dense_code) {
  return dense_code == 0 ? kSdDenseMin : dense_code == 1 ? 0 : dense_code == 255 ? kSdBM * kSdBN + 1 : 64 * dense_code;
}

// Whatever of tables and lists the caller does not vouch for (ready: bit 0 = the tables are in the workspace, bit 1 = the
// lists too, made with this dense_code).
inline int sb_setup(const SdTables& t, const SbLists& l, int m, int tiles, int dense_code, int ready, const int* row_offsets, const int* cols,
                    hipStream_t stream) {
  const int dense_min = sb_dense_min(dense_code);
  if (!(ready & 1)) {
    if (int rc = sd_write_tables(t, m, tiles, row_offsets, cols, stream)) return rc;
  }
  if ((ready & 3) != 3) {
    if (int rc = sb_write_lists(t, l, m, tiles, dense_min, row_offsets, cols, stream)) return rc;
  }
  return 0;
}

// acc + <a, b> over 8 elements of 16 bits, products and sums in fp32
template <bool BF16>
__device__ __forceinline__ float dot8(u32x4 a, u32x4 b, float acc) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  const unsigned aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (BF16)
      acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, aw[i]), __builtin_bit_cast(b2, bw[i]), acc, false);
    else
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, aw[i]), __builtin_bit_cast(h2, bw[i]), acc, false);
  }
  return acc;
}

template <bool BF16, int KS>
__global__ __launch_bounds__(kSdThreads, KS == 8 ? 1 : 2) void sddmm_mfma_kernel(SddmmMfmaParams p) {
  constexpr int RB = KS * 32;            // bytes of a k row
  constexpr int CH = RB / 16;            // 16-byte chunks per k row
  constexpr int RPI = kWave / CH;        // rhs rows per direct load
  constexpr int STAGE = kSdBN * RB;
  static_assert(KS == 2 || KS == 4 || KS == 8, "k = 32, 64 or 128");
  typedef unsigned short u16;
  typedef u32x4 u128_a2 __attribute__((aligned(2)));   // eight neighbouring scores stored at once
  typedef __attribute__((address_space(3))) unsigned char lds_u8;
  extern __shared__ __align__(16) unsigned char smem[];
  u16* S = reinterpret_cast<u16*>(smem);                                      // [128][kSdLd]; before the loop: column sums
  unsigned char* sR = smem + kSdBM * kSdLd * 2;                               // [2][128][RB]
  unsigned char* sM = sR + 2 * STAGE;                                         // [3] slots of per-row words
  unsigned long long* long_rows = reinterpret_cast<unsigned long long*>(sM + 3 * kSdSlot);   // [2] rows with more than kSdShort
  const unsigned ldsR = (unsigned)(size_t)(lds_u8*)sR;
  const unsigned ldsM = (unsigned)(size_t)(lds_u8*)sM;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave >> 1, wc = wave & 1;
  // Workgroups go to the 8 XCDs round-robin by their linear id; renumbered so that an XCD gets all row blocks of
  // a batch entry (and then of the next): the rhs rows they all read stay in that XCD's L2.
  const int row_blocks = gridDim.x, total = row_blocks * gridDim.y;
  int id = blockIdx.x + row_blocks * blockIdx.y;
  // The two workgroups that share a CU take the two phases below in opposite order, so that one phase's matrix-core
  // and LDS work runs beside the other's waiting for memory.  (Which two share a CU is the dispatcher's business:
  // neighbours in launch order on the XCD, or 32 apart; the parity below differs in both cases.)
  const int launch_slot = id / 8;
  const bool thin_first = ((launch_slot ^ (launch_slot >> 5)) & 1) != 0;
  if (total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
  const int z = id / row_blocks;
  const int row0 = (id % row_blocks) * kSdBM;
  const u16* __restrict__ lhs = static_cast<const u16*>(p.lhs) + (size_t)z * p.m * p.k;
  const unsigned char* rhs = reinterpret_cast<const unsigned char*>(static_cast<const u16*>(p.rhs) + (size_t)z * p.n * p.k);
  u16* __restrict__ out = static_cast<u16*>(p.out) + (size_t)z * p.nnz;
  const int tiles_n = p.tiles_n;

  // the dense tiles of this block of rows (sorted out by the list kernel)
  const u16* __restrict__ list = p.dense_list + (size_t)(row0 / kSdBM) * (tiles_n + 2);
  const int nd = __builtin_amdgcn_readfirstlane((int)list[0]);
  ++list;

  for (int phase = 0; phase < 2; ++phase) {
  // ---- dense tiles
  if ((phase == 0) != thin_first) {
   if (nd > 0) {
    auto sw = [](int row) { return CH == 4 ? (row >> 2) & 3 : CH == 8 ? (row >> 1) & 7 : row & 15; };
    // direct loads of one tile of rhs rows: instruction g = wave * KS + q fills rows g * RPI .. + RPI - 1
    const int dl_row = lane / CH, dl_slot = lane % CH;
    auto issue_rows = [&](int i) {   // the i-th dense tile (past the end the last one again, into a stage nobody reads)
      const int ct = __builtin_amdgcn_readfirstlane((int)list[min(i, nd - 1)]);
      const unsigned base = ldsR + (i & 1) * STAGE;
#pragma unroll
      for (int q = 0; q < KS; ++q) {
        const int row = (wave * KS + q) * RPI + dl_row;
        const int grow = min(ct * kSdBN + row, p.n - 1);   // past the last column: a valid row nobody samples
        lds_dma16(rhs + (size_t)grow * RB + ((dl_slot ^ sw(row)) << 4), __builtin_amdgcn_readfirstlane(base + (wave * KS + q) * 1024));
      }
    };
    // per-row words of the i-th dense tile: wavefronts 0, 1 fetch cursor and packed word of their 64 rows (two
    // loads each), wavefronts 2, 3 the masks of 64 rows (one load each)
    const int meta_row = min(row0 + (wave & 1) * kWave + lane, p.m - 1);
    auto issue_words = [&](int i) {
      const int ct = __builtin_amdgcn_readfirstlane((int)list[min(i, nd - 1)]);
      const unsigned base = ldsM + (i % 3) * kSdSlot;
      if (wave < 2) {
        lds_dma4(p.tile_ptr + (size_t)ct * p.m + meta_row, __builtin_amdgcn_readfirstlane(base + wave * 256));
        lds_dma4(p.brief + (size_t)ct * p.m + meta_row, __builtin_amdgcn_readfirstlane(base + 512 + wave * 256));
      } else {
        lds_dma16(p.mask + (size_t)ct * p.m + meta_row, __builtin_amdgcn_readfirstlane(base + 1024 + (wave - 2) * 1024));
      }
    };
    issue_rows(0);
    issue_words(0);
    issue_rows(1);
    issue_words(1);

    // this wavefront's lhs fragments: rows wr * 64 + i * 32 + lane % 32, k entries ks * 16 + (lane / 32) * 8 .. + 7
    const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
    u32x4 fl[2][KS];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = min(row0 + wr * 64 + i * 32 + frag_row, p.m - 1);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) fl[i][ks] = *reinterpret_cast<const u32x4*>(lhs + (size_t)row * p.k + ks * 16 + frag_k);
    }
    const bool owner = tid < kSdBM && row0 + tid < p.m;   // threads 0..127: one row each
    // what a lane needs to find its 8 columns in a long row's words (sampling below): which of the step's four rows,
    // which group of 8 columns, the mask word with their bits, the bits below them in it, and the field of the packed
    // word that counts the nonzeros of the mask words before
    const int own_row = lane >> 4, own_col8 = lane & 15;
    const int own_word = own_col8 >> 2, own_bit = (own_col8 & 3) * 8;
    const unsigned own_below = (1u << own_bit) - 1u;
    const int own_shift = own_word == 2 ? 6 : own_word == 3 ? 13 : 0;
    const unsigned own_field = own_word == 0 ? 0u : own_word == 1 ? 0x3fu : 0x7fu;

    wait_vmcnt<0>();        // the first tile's rhs rows, the first words and the lhs fragments have landed
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(fl[i][ks]));

    for (int i = 0; i < nd; ++i) {
      lds_barrier();        // everybody's loads for this tile have landed; the previous tile's sampling is over
      const unsigned char* slot = sM + (i % 3) * kSdSlot;
      int pk = 0, tp = 0;
      if (tid < kSdBM) {
        tp = reinterpret_cast<const int*>(slot)[tid];
        pk = reinterpret_cast<const int*>(slot + 512)[tid];
      }
      const int count = owner ? (pk >> 28) & 7 : 0;
      const unsigned long long longs = __ballot(count == 7);
      if (tid < kSdBM && lane == 0) long_rows[wave] = longs;

      // ---- scores of the tile: S[r][c] = <lhs[r], rhs[c0 + c]>, rounded to the element type
      f32x16 acc[2][2];
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
      const unsigned char* stage = sR + (i & 1) * STAGE;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        u32x4 fr[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const int c = wc * 64 + b * 32 + frag_row;
          fr[b] = *reinterpret_cast<const u32x4*>(stage + c * RB + (((ks * 2 + (lane >> 5)) ^ sw(c)) << 4));
        }
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b) acc[a][b] = mfma_32x32x16<BF16>(fr[b], fl[a][ks], acc[a][b]);
      }
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            u16 h[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = f32_to_16(acc[a][b][q * 4 + e], BF16);
            u32x2 w;
            w.x = (unsigned)h[0] | ((unsigned)h[1] << 16);
            w.y = (unsigned)h[2] | ((unsigned)h[3] << 16);
            *reinterpret_cast<u32x2*>(S + (wr * 64 + a * 32 + frag_row) * kSdLd + wc * 64 + b * 32 + q * 8 + (lane >> 5) * 4) = w;
          }
      // The next tile's rhs rows and words, asked for a whole tile ago (below, before the previous tile's
      // sampling), must have landed before the barrier.
      wait_vmcnt<0>();
      lds_barrier();
      issue_rows(i + 2);    // into the stage whose MFMAs everybody has just finished
      issue_words(i + 2);   // into the slot of the tile before this one

      // ---- sampling: short runs by the row's own lane
      if (count >= 1 && count <= kSdShort) {
#pragma unroll
        for (int u = 0; u < kSdShort; ++u)
          if (u < count) out[tp + u] = S[tid * kSdLd + ((pk >> (7 * u)) & 127)];
      }
      // long runs: this wavefront takes rows 32 * wave .. + 31, four consecutive rows per step, 16 lanes per row: a
      // lane owns 8 neighbouring columns.  It reads the mask word that holds their bits, the row's packed word and
      // cursor and its 8 scores from LDS; the nonzeros below its first column (those of the mask words before its
      // own, from the packed word, plus the bits below in its own) give the position of its first score in the row's
      // output.  All 8 present (the inside of a band): one 16-byte store at 2-byte alignment, four rows per
      // instruction.  Else (the edge of a run): a 2-byte store per score present.  What this step costs is
      // instructions and LDS round trips per row, which is why it works on as many rows per instruction as it can.
      unsigned todo = (unsigned)(long_rows[wave >> 1] >> ((wave & 1) * 32));
      todo = __builtin_amdgcn_readfirstlane(todo);
      struct Words {
        unsigned word, packed;
        int start;
        u32x4 sc;
      };
      auto read_words = [&](int g) {   // (every group is read, also one without long rows: no branch around LDS reads)
        const int r = wave * 32 + 4 * g + own_row;
        Words w;
        w.word = *reinterpret_cast<const unsigned*>(slot + 1024 + r * 16 + own_word * 4);
        w.start = reinterpret_cast<const int*>(slot)[r];
        w.packed = reinterpret_cast<const unsigned*>(slot + 512)[r];
        w.sc = *reinterpret_cast<const u32x4*>(S + r * kSdLd + 8 * own_col8);
        return w;
      };
      if (todo) {
        Words next = read_words(0);
#pragma unroll
        for (int g = 0; g < 8; ++g) {
          const Words cur = next;
          if (g + 1 < 8) next = read_words(g + 1);   // in flight while this group is stored
          const unsigned four = (todo >> (4 * g)) & 0xfu;
          if (!four) continue;   // (uniform)
          const unsigned have = ((four >> own_row) & 1u) ? (cur.word >> own_bit) & 0xffu : 0u;
          const int at = cur.start + (int)((cur.packed >> own_shift) & own_field) + __popc(cur.word & own_below);
          if (have == 0xffu) *reinterpret_cast<u128_a2*>(out + min(at, max(p.nnz - 8, 0))) = cur.sc;   // (never clamped when the tables fit the arrays)
          const unsigned some = have == 0xffu ? 0u : have;
          if (__ballot(some != 0)) {
            const unsigned w[4] = {cur.sc.x, cur.sc.y, cur.sc.z, cur.sc.w};
            int k = min(at, p.nnz - 1);
#pragma unroll
            for (int b = 0; b < 8; ++b) {
              if ((some >> b) & 1u) {
                out[min(k, p.nnz - 1)] = (u16)((b & 1) ? w[b >> 1] >> 16 : w[b >> 1]);
                ++k;
              }
            }
          }
        }
      }
    }
    wait_vmcnt<0>();   // the loads issued past the last dense tile: nothing may still be writing LDS when the phase ends
   }
  } else {

  // ---- the nonzeros outside dense tiles, from the per-row lists (column, position in the output) that the list
  // kernel compacted.  A group of LPN = k / 8 lanes takes a row: lane j of the group keeps elements 8 j .. 8 j + 7 of the
  // row's lhs in registers for the whole row.  Two rows of a group side by side, LPN entries of each per step: lane j
  // reads entry j of the step, the group's lanes exchange the columns, every lane reads its 16 bytes of the LPN rhs
  // rows, v_dot2 in fp32, summed over the group's lanes; lane j
  // keeps the result of entry j and stores it at the entry's position.  The entries of the next step are fetched
  // before this step's dot products.
  {
    constexpr int LPN = CH;              // lanes per row
    constexpr int G = kWave / LPN;       // rows side by side in a wavefront
    constexpr int ROUNDS = 32 / G;       // rounds of G rows over the wavefront's 32
    constexpr int RS = 2;                // rows of a group side by side (4 for k = 64 filled the register file for 2 % of the time)
    static_assert(ROUNDS % RS == 0, "rows side by side");
    const int g = lane / LPN, sl = lane % LPN, gl = lane - sl;
    const int last = p.nnz - 1;
    for (int h = 0; h < ROUNDS; h += RS) {
      int base[RS], cnt[RS], nmax = 0;
      u32x4 lf[RS];
      SbEntry en[RS];
#pragma unroll
      for (int w = 0; w < RS; ++w) {
        const int r = row0 + wave * 32 + (h + w) * G + g;
        const int rc = min(r, p.m - 1);
        base[w] = p.row_offsets[rc];
        cnt[w] = r < p.m ? p.thin_cnt[rc] : 0;
        lf[w] = *reinterpret_cast<const u32x4*>(lhs + (size_t)rc * p.k + sl * 8);
      }
#pragma unroll
      for (int w = 0; w < RS; ++w) {
        nmax = max(nmax, cnt[w]);
        en[w] = p.thin_ent[min(base[w] + min(sl, max(cnt[w] - 1, 0)), last)];
      }
      for (int st = 0; __ballot(st * LPN < nmax); ++st) {
        u32x4 rv[RS][LPN];
        int at[RS];
#pragma unroll
        for (int w = 0; w < RS; ++w) {
          at[w] = en[w].pos;
#pragma unroll
          for (int u = 0; u < LPN; ++u) {
            // (an entry past the end of the row's list is a copy of the row's last one, or -- a row without a list --
            // whatever the slot holds: the column is clamped into the operand and the result never stored)
            const unsigned cu = min((unsigned)__shfl(en[w].col, gl + u, kWave), (unsigned)(p.n - 1));
            rv[w][u] = *reinterpret_cast<const u32x4*>(rhs + (size_t)cu * RB + sl * 16);
          }
        }
#pragma unroll
        for (int w = 0; w < RS; ++w) en[w] = p.thin_ent[min(base[w] + min((st + 1) * LPN + sl, max(cnt[w] - 1, 0)), last)];
#pragma unroll
        for (int w = 0; w < RS; ++w) {
          float res = 0.f;
#pragma unroll
          for (int u = 0; u < LPN; ++u) {
            const float acc = group_sum<LPN>(dot8<BF16>(lf[w], rv[w][u], 0.f));
            res = sl == u ? acc : res;
          }
          if (st * LPN + sl < cnt[w]) out[min((unsigned)at[w], (unsigned)last)] = f32_to_16(res, BF16);
        }
      }
    }
  }
  }
  }
}

}  // namespace iex
