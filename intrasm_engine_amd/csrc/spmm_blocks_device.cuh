// CSR SpMM for attention-like sparse operands (gfx950, fp16 / bf16, 64 output columns per workgroup, wider outputs in
// slices of 64): out = A * dense with A a
// mask with structure (a dense band plus scattered entries) whose values differ per batch entry -- the second
// product of sparse attention, probabilities times V.
//
// The row kernel (spmm_device.cuh) reads n * 2 bytes of the dense operand per nonzero through the L2 -> CU path;
// for 16 heads of a 4096 x 4096 mask with 7 % of its entries that is 2.4 GB and that path bounds it.  This kernel
// is the mirror image of the SDDMM for such masks (sddmm_mfma_device.cuh) and works from the same tables, written
// by the same setup kernel into the caller's workspace (tile_ptr, brief, mask: per row and 128-column tile of A the
// position of the row's first nonzero there, and which of the tile's columns the row holds), plus two lists that
// one more small kernel derives from the tables (they depend on the pattern and on the threshold below, not on
// values: a caller whose pattern stays keeps them): per block of 128 rows the column tiles that hold dense_min
// nonzeros or more ("dense"), and per row its nonzeros outside those tiles, compacted.
// A workgroup (4 wavefronts) owns 128 consecutive rows of one batch entry, a wavefront 32 of them:
//   * dense tiles: the block of A is laid out as a dense 32 x 128 tile per wavefront in LDS -- zeros, then the
//     values: up to 4 per (row, tile) by the row's own lane from the packed word, more by the whole wavefront, four
//     rows per step and 16 lanes per row, from the row's 128-bit mask: a lane owns 8 neighbouring columns, a
//     population count of the mask bits below them gives the position of its first value in the row's values, one
//     16-byte load from there holds all it owns (no column index is read), and they are spread over the columns
//     present by byte selectors (v_perm) that a table in LDS holds for each of the 256 patterns of 8 columns, one
//     ds_write_b128 per lane; all loads of a tile are issued before the first is used -- and multiplied on the matrix
//     cores with the 128 rows of the dense operand that the tile names: they go through registers into LDS once per
//     workgroup, double-buffered, 16-byte chunks permuted so that the transposing operand reads (ds_read_tr16_b64)
//     are conflict-free.  Operands swapped (out^T = dense^T * A^T) so that a lane ends up with 4 adjacent output
//     columns of one row.
//   * everything else: 8 lanes per row walk the row's list, two rows at a time, 8 nonzeros of each per step: 16
//     bytes of the dense operand's row per lane and nonzero, fp32 FMAs, no reduction across lanes.
// Both parts meet in LDS: the matrix-core sums of a wavefront's 32 rows are written there as fp32, each lane adds
// its own sums of the second kind to the 8 of them it owns, rounds once and stores 16 bytes.  The order of the
// additions is fixed: results are bit-stable from call to call.
// The tile of A holds explicit zeros: a non-finite entry in a row of the dense operand that a dense tile covers
// reaches the output rows of that tile's 128-row block whether or not they reference it (0 * inf = NaN).
#pragma once
#include "sddmm_mfma_device.cuh"

namespace iex {

constexpr int kSbN = 64;                       // output columns per workgroup (a wider output is served in slices of 64)
constexpr int kSbTileBytes = 32 * kSdLd * 2;   // a wavefront's 32 x 128 tile of A (rows padded to 272 bytes); later its 32 x 64 fp32 sums
constexpr int kSbStage = kSdBN * kSbN * 2;     // 128 rows of the dense operand
constexpr int kSbRows = 2;                     // rows whose nonzeros outside dense tiles a lane group gathers side by side (1, 2 or 4)
struct SpmmBlocksParams {
  int m, k, nnz;
  const int* row_offsets;
  const void* values;
  size_t values_stride;   // elements between batch entries (0: shared)
  const void* dense;      // (batch, k, n)
  void* out;              // (batch, m, n)
  int n;                  // a multiple of 64: gridDim.y = batch * n / 64, a workgroup serves 64 columns
  const u32x4* mask;      // [tiles_k][m]
  const int* tile_ptr;    // [(tiles_k + 1)][m]
  const int* brief;       // [tiles_k][m]
  int tiles_k;
  const unsigned* zeros;
  const SbEntry* thin_ent;
  const int* thin_cnt;
  const unsigned short* dense_list;
};

constexpr int spmm_blocks_lds_bytes() { return 4 * kSbTileBytes + 2 * kSbStage + 4 * 32 * 32 + 256 * 32; }

template <bool BF16>
__global__ __launch_bounds__(kSdThreads, 2) void spmm_blocks_kernel(SpmmBlocksParams p) {
  typedef unsigned short u16;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  typedef u32x4 u128_a2 __attribute__((aligned(2)));               // loads of eight and four values at the alignment of one
  typedef unsigned long long u64_a2 __attribute__((aligned(2)));
  constexpr int NT = kSbN / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sV = smem + 4 * kSbTileBytes;                               // [2][128][128 bytes]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  unsigned* rec = reinterpret_cast<unsigned*>(sV + 2 * kSbStage) + wave * (32 * 8);
  unsigned* spread = reinterpret_cast<unsigned*>(sV + 2 * kSbStage) + 4 * (32 * 8);   // [256][8]: see the dense part                                 // [32][8]: what a wavefront's rows know of the current tile
  // Workgroups go to the 8 XCDs round-robin by their linear id; renumbered so that an XCD gets all row blocks of a
  // batch entry (and then of the next): the dense operand of that entry stays in that XCD's L2.
  const int row_blocks = gridDim.x, total = row_blocks * gridDim.y;
  int id = blockIdx.x + row_blocks * blockIdx.y;
  // the two workgroups that share a CU take the two parts in opposite order (matrix cores and LDS beside gathers)
  const int launch_slot = id / 8;
  const bool thin_first = ((launch_slot ^ (launch_slot >> 5)) & 1) != 0;
  if (total % 8 == 0) id = (id % 8) * (total / 8) + id / 8;
  const int slices = p.n / kSbN;                     // (the slices of a batch entry are neighbours in this order: same XCD)
  const int z = (id / row_blocks) / slices, slice = (id / row_blocks) % slices;
  const int ld = p.n;                                // elements between rows of the dense operand and of the output
  const int row_block = id % row_blocks;
  const int row0 = row_block * kSdBM;
  const u16* __restrict__ vals = static_cast<const u16*>(p.values) + (size_t)z * p.values_stride;
  const u16* __restrict__ V = static_cast<const u16*>(p.dense) + (size_t)z * p.k * ld + slice * kSbN;
  u16* __restrict__ out = static_cast<u16*>(p.out) + (size_t)z * p.m * ld + slice * kSbN;
  const int m = p.m;
  const int last = p.nnz - 1;   // (the host does not launch this kernel without nonzeros)
  const u16* __restrict__ list = p.dense_list + (size_t)row_block * (p.tiles_k + 2);
  const int nd = __builtin_amdgcn_readfirstlane((int)list[0]);
  ++list;

  unsigned char* Pw = smem + wave * kSbTileBytes;   // this wavefront's tile of A
  u16* P16 = reinterpret_cast<u16*>(Pw);
  const int wrow0 = row0 + wave * 32;               // first of this wavefront's rows

  float* T = reinterpret_cast<float*>(Pw);           // after the dense tiles: the matrix-core sums of the 32 rows, fp32
  constexpr int TLD = kSdLd / 2;                     // 68 floats = the 272 bytes of a row of the tile
  float tacc[4][8];   // sums over the nonzeros outside dense tiles: row it * 8 + lane / 8, columns (lane % 8) * 8 .. + 7
#pragma unroll
  for (int it = 0; it < 4; ++it)
#pragma unroll
    for (int c = 0; c < 8; ++c) tacc[it][c] = 0.f;

  for (int phase = 0; phase < 2; ++phase) {
    if ((phase == 0) != thin_first) {
      // ---- dense tiles
      f32x16 acc[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
      if (nd > 0) {
        // 128 rows x 128 bytes of the dense operand: chunk L = q * 256 + tid sits at LDS byte 16 L and holds global
        // chunk (L % 8) ^ 4 * ((row / 2) % 2) of row L / 8
        auto load_rows = [&](int i, u32x4 (&rv)[4]) {
          const int ct = __builtin_amdgcn_readfirstlane((int)list[min(i, nd - 1)]);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int L = q * kSdThreads + tid;
            const int row = L >> 3, pos = L & 7;
            const int g = pos ^ (((row >> 1) & 1) << 2);
            const int krow = ct * kSdBN + row;
            const u32x4 got = *reinterpret_cast<const u32x4*>(V + (size_t)min(krow, p.k - 1) * ld + g * 8);
            const u32x4 zero = {0u, 0u, 0u, 0u};
            rv[q] = krow < p.k ? got : zero;
          }
        };
        auto store_rows = [&](int i, const u32x4 (&rv)[4]) {
          unsigned char* base = sV + (i & 1) * kSbStage;
#pragma unroll
          for (int q = 0; q < 4; ++q) *reinterpret_cast<u32x4*>(base + (q * kSdThreads + tid) * 16) = rv[q];
        };
        // what lanes 0..31 know of their row in a tile: cursor, packed word, mask
        const int meta_row = min(wrow0 + (lane & 31), m - 1);
        const bool meta_valid = lane < 32 && wrow0 + lane < m;
        auto load_meta = [&](int i, int& tp, int& bf, u32x4& mk) {
          const int ct = __builtin_amdgcn_readfirstlane((int)list[min(i, nd - 1)]);
          tp = p.tile_ptr[(size_t)ct * m + meta_row];
          bf = p.brief[(size_t)ct * m + meta_row];
          mk = p.mask[(size_t)ct * m + meta_row];
        };

        // transposing operand reads of the dense operand's tile: lane group lane / 16 covers column half (group % 2)
        // and k half (group / 2) of a 16-wide k step; lane r of a group points at k row r / 4, columns 4 (r % 4) .. + 3
        const int fkh = lane >> 5;
        const int tr_k = fkh * 8 + ((lane & 15) >> 2);
        const int tr_sw = ((tr_k >> 1) & 1) << 2;
        int v_off[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          const int chunk = (t * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1)) ^ tr_sw;
          v_off[t] = tr_k * (kSbN * 2) + chunk * 16 + (lane & 1) * 8;
        }
        const int p_off = (lane & 31) * (kSdLd * 2) + fkh * 16;
        // what a lane needs to find the 8 columns that it owns in a long row: which of a step's four rows, which group
        // of 8 columns, the mask word that holds their bits and the bits below them in it
        const int own_row = lane >> 4, own_col8 = lane & 15;
        const int own_word = own_col8 >> 2, own_bit = (own_col8 & 3) * 8;
        const unsigned own_below = (1u << own_bit) - 1u;
        // spread[pattern]: for each of the 256 patterns of 8 columns, byte selectors (v_perm) that take value j of 16 loaded
        // bytes to the j-th column present and zeros to the others: words 0..3 select from the first 8 bytes (one word
        // per pair of columns), words 4..7 from the last 8
        {
          const unsigned pattern = (unsigned)tid;
          unsigned lo_sel[4] = {0u, 0u, 0u, 0u}, hi_sel[4] = {0u, 0u, 0u, 0u};
          unsigned k = 0;
#pragma unroll
          for (int c = 0; c < 8; ++c) {
            const bool present = (pattern >> c) & 1u;
            const unsigned two = 2u * (k & 3u);
            const unsigned pick = two | ((two + 1u) << 8), none = 0x0c0cu;
            const unsigned from_first = present && k < 4 ? pick : none, from_last = present && k >= 4 ? pick : none;
            lo_sel[c >> 1] |= from_first << ((c & 1) * 16);
            hi_sel[c >> 1] |= from_last << ((c & 1) * 16);
            k += present;
          }
          *reinterpret_cast<u32x4*>(spread + pattern * 8) = u32x4{lo_sel[0], lo_sel[1], lo_sel[2], lo_sel[3]};
          *reinterpret_cast<u32x4*>(spread + pattern * 8 + 4) = u32x4{hi_sel[0], hi_sel[1], hi_sel[2], hi_sel[3]};
        }
        u32x4 rv[4];
        int tp, bf;
        u32x4 mk;
        load_rows(0, rv);
        load_meta(0, tp, bf, mk);
        store_rows(0, rv);
        __syncthreads();

        for (int i = 0; i < nd; ++i) {
          int tp_n, bf_n;
          u32x4 mk_n;
          const bool more = i + 1 < nd;
          if (more) load_rows(i + 1, rv);
          load_meta(i + 1, tp_n, bf_n, mk_n);

          // ---- this wavefront's 32 x 128 tile of A: zeros ...
          {
            const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int q = 0; q < 8; ++q) {
              const int c = q * kWave + lane;
              *reinterpret_cast<u32x4*>(Pw + (c >> 4) * (kSdLd * 2) + (c & 15) * 16) = zero;
            }
          }
          const int count = meta_valid ? (bf >> 28) & 7 : 0;
          // ... up to 4 values of a row by the row's lane: the 8 bytes from the row's first value in the tile (a load
          // at 2-byte alignment; moved back where it would pass the end of the values, and shifted to make up) ...
          const int s_at = min(max(tp, 0), last - 3);
          const int s_shift = min(max(tp, 0) - s_at, 3) * 16;   // (more than 3 only for rows without values here)
          const unsigned long long sv = *reinterpret_cast<const u64_a2*>(vals + s_at);
          // ... longer runs by the wavefront, four consecutive rows per step, 16 lanes per row: a lane owns 8
          // neighbouring columns.  Lanes 0..31 publish what they know of their rows in LDS (mask, nonzeros below each
          // mask word, cursor); every lane picks from there what concerns its 8 columns: the number of the row's
          // nonzeros below its first column is the position of its first value among the row's values in the tile,
          // and the 16 bytes from there (one load at 2-byte alignment, moved back where it would pass the end of the
          // values) hold all the values it owns; byte selectors from the table of patterns spread them over the columns
          // present (and zeros over the others).  All loads of the tile first.
          const unsigned longs = (unsigned)__ballot(count == 7);
          if (lane < 32) {
            const unsigned cx = __popc(mk.x), cy = cx + __popc(mk.y), cz = cy + __popc(mk.z);
            *reinterpret_cast<u32x4*>(rec + lane * 8) = mk;
            *reinterpret_cast<u32x2*>(rec + lane * 8 + 4) = u32x2{(cx << 8) | (cy << 16) | (cz << 24), (unsigned)max(tp, 0)};
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();
          u32x4 got[8];
          unsigned have[8], back[8];
#pragma unroll
          for (int g = 0; g < 8; ++g) {
            got[g] = u32x4{0u, 0u, 0u, 0u};
            have[g] = 0;
            back[g] = 0;
            const unsigned four = (longs >> (4 * g)) & 0xfu;
            if (four) {   // (uniform)
              const int r = 4 * g + own_row;
              const unsigned word = rec[r * 8 + own_word];
              const u32x2 pt = *reinterpret_cast<const u32x2*>(rec + r * 8 + 4);
              const int at = (int)(pt.y + ((pt.x >> (own_word * 8)) & 0xffu)) + __popc(word & own_below);
              const int at_c = max(min(at, last - 7), 0);
              have[g] = ((four >> own_row) & 1u) ? (word >> own_bit) & 0xffu : 0u;
              back[g] = (unsigned)min(at - at_c, 7);   // (values that the load was moved back by: only at the end of the values)
              got[g] = *reinterpret_cast<const u128_a2*>(vals + at_c);
            }
          }
          if (count >= 1 && count <= kSdShort) {
#pragma unroll
            for (int u = 0; u < kSdShort; ++u)
              if (u < count) P16[lane * kSdLd + ((bf >> (7 * u)) & 127)] = (u16)(sv >> ((s_shift + 16 * u) & 63));
          }
#pragma unroll
          for (int g = 0; g < 8; ++g) {
            const unsigned four = (longs >> (4 * g)) & 0xfu;
            if (!four) continue;   // (uniform)
            u32x4 in = got[g];
            const unsigned h = have[g];
            if (__ballot(h != 0 && back[g] != 0)) {   // (only at the end of the values: the load was moved back, move its bytes forward)
              typedef unsigned long long u64;
              const u64 lo = (u64)in.x | ((u64)in.y << 32), hi = (u64)in.z | ((u64)in.w << 32);
              const int sh = (int)back[g] * 16;
              const u64 nlo = sh == 0 ? lo : sh >= 64 ? hi >> ((sh - 64) & 63) : (lo >> sh) | (hi << ((64 - sh) & 63));
              const u64 nhi = sh == 0 ? hi : sh >= 64 ? 0ull : hi >> sh;
              in = u32x4{(unsigned)nlo, (unsigned)(nlo >> 32), (unsigned)nhi, (unsigned)(nhi >> 32)};
            }
            // value j of the 16 bytes goes to the j-th column present: byte selectors by pattern, from the table --
            // unless every lane that stores has all 8 of its columns (the inside of a band): as loaded
            u32x4 put = in;
            if (__ballot(h != 0u && h != 0xffu)) {   // (uniform)
              const u32x4 from_lo = *reinterpret_cast<const u32x4*>(spread + h * 8), from_hi = *reinterpret_cast<const u32x4*>(spread + h * 8 + 4);
              put.x = __builtin_amdgcn_perm(in.y, in.x, from_lo.x) | __builtin_amdgcn_perm(in.w, in.z, from_hi.x);
              put.y = __builtin_amdgcn_perm(in.y, in.x, from_lo.y) | __builtin_amdgcn_perm(in.w, in.z, from_hi.y);
              put.z = __builtin_amdgcn_perm(in.y, in.x, from_lo.z) | __builtin_amdgcn_perm(in.w, in.z, from_hi.z);
              put.w = __builtin_amdgcn_perm(in.y, in.x, from_lo.w) | __builtin_amdgcn_perm(in.w, in.z, from_hi.w);
            }
            if (h) *reinterpret_cast<u32x4*>(Pw + (4 * g + own_row) * (kSdLd * 2) + own_col8 * 16) = put;
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();

          // ---- out^T (64 x 32 per wavefront) += dense^T (64 x 128) * A^T (128 x 32)
          const unsigned char* stage = sV + (i & 1) * kSbStage;
#pragma unroll
          for (int ks = 0; ks < kSdBN / 16; ++ks) {
            const u32x4 pf = *reinterpret_cast<const u32x4*>(Pw + p_off + ks * 32);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              const unsigned char* q0 = stage + ks * 16 * (kSbN * 2) + v_off[t];
              const s16x4 l4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0));
              const s16x4 h4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0 + 4 * (kSbN * 2)));
              const u32x2 l2 = __builtin_bit_cast(u32x2, l4), h2 = __builtin_bit_cast(u32x2, h4);
              acc[t] = mfma_32x32x16<BF16>(u32x4{l2.x, l2.y, h2.x, h2.y}, pf, acc[t]);
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
          __builtin_amdgcn_wave_barrier();

          if (more) store_rows(i + 1, rv);   // into the stage that everybody left before the last barrier
          tp = tp_n, bf = bf_n, mk = mk_n;
          __syncthreads();
        }
      }
      // the sums leave the registers here (the other part needs them for loads in flight): this wavefront's tile, no
      // longer read by anybody, takes them as fp32
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4 x = {acc[t][q * 4], acc[t][q * 4 + 1], acc[t][q * 4 + 2], acc[t][q * 4 + 3]};
          *reinterpret_cast<f32x4*>(T + (lane & 31) * TLD + t * 32 + q * 8 + (lane >> 5) * 4) = x;
        }
    } else {
      // ---- nonzeros outside dense tiles: lane group g = lane / 8 takes rows g, 8 + g, 16 + g, 24 + g of the
      // wavefront's 32, two at a time, 8 nonzeros of each per step: lane sl of the group reads entry sl of the step
      // (column, position) and its value, the group's lanes exchange them, and every lane reads its 16 bytes of the
      // 8 rows of the dense operand.  The lanes of an absent nonzero read zeros instead (never a row of the dense
      // operand that the row does not reference).  The entries of the next step are fetched before this step's sums.
      const int g = lane >> 3, sl = lane & 7, gl = lane & ~7;
      const u16* __restrict__ zeros = reinterpret_cast<const u16*>(p.zeros);
      int base[4], cnt[4];
#pragma unroll
      for (int it = 0; it < 4; ++it) {
        const int r = wrow0 + it * 8 + g;
        const int rc = min(r, m - 1);
        base[it] = p.row_offsets[rc];
        cnt[it] = r < m ? p.thin_cnt[rc] : 0;
      }
#pragma unroll
      for (int h = 0; h < 4; h += kSbRows) {
        int nmax = 0;
        SbEntry en[kSbRows];
#pragma unroll
        for (int w = 0; w < kSbRows; ++w) {
          nmax = max(nmax, cnt[h + w]);
          en[w] = p.thin_ent[min(base[h + w] + min(sl, max(cnt[h + w] - 1, 0)), last)];
        }
        for (int st = 0; __ballot(st * 8 < nmax); ++st) {
          u16 pv[kSbRows];
          u32x4 v[kSbRows][8];
          int colw[kSbRows];
#pragma unroll
          for (int w = 0; w < kSbRows; ++w) {
            pv[w] = vals[min((unsigned)en[w].pos, (unsigned)last)];
            colw[w] = en[w].col;
          }
#pragma unroll
          for (int w = 0; w < kSbRows; ++w)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              const int cu = __shfl(colw[w], gl + u, kWave);
              const u16* src = st * 8 + u < cnt[h + w] ? V + (size_t)cu * ld + sl * 8 : zeros + sl * 8;
              v[w][u] = *reinterpret_cast<const u32x4*>(src);
            }
#pragma unroll
          for (int w = 0; w < kSbRows; ++w) {
            if (st * 8 + sl >= cnt[h + w]) pv[w] = 0;
            en[w] = p.thin_ent[min(base[h + w] + min((st + 1) * 8 + sl, max(cnt[h + w] - 1, 0)), last)];
          }
#pragma unroll
          for (int w = 0; w < kSbRows; ++w)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              const float pf = f16_to_32((u16)__shfl((int)pv[w], gl + u, kWave), BF16);
              const unsigned x[4] = {v[w][u].x, v[w][u].y, v[w][u].z, v[w][u].w};
#pragma unroll
              for (int c = 0; c < 4; ++c) {
                tacc[h + w][2 * c] = fmaf(pf, f16_to_32((u16)(x[c] & 0xffffu), BF16), tacc[h + w][2 * c]);
                tacc[h + w][2 * c + 1] = fmaf(pf, f16_to_32((u16)(x[c] >> 16), BF16), tacc[h + w][2 * c + 1]);
              }
            }
        }
      }
    }
  }

  // ---- both parts meet: every lane adds its own sums to the 8 matrix-core sums it owns, rounds and stores 16 bytes
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
  {
    const int g = lane >> 3, sl = lane & 7;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int row = it * 8 + g;
      const f32x4 x0 = *reinterpret_cast<const f32x4*>(T + row * TLD + sl * 8);
      const f32x4 x1 = *reinterpret_cast<const f32x4*>(T + row * TLD + sl * 8 + 4);
      const float y[8] = {x0[0] + tacc[it][0], x0[1] + tacc[it][1], x0[2] + tacc[it][2], x0[3] + tacc[it][3],
                          x1[0] + tacc[it][4], x1[1] + tacc[it][5], x1[2] + tacc[it][6], x1[3] + tacc[it][7]};
      u32x4 w;
      w.x = (unsigned)f32_to_16(y[0], BF16) | ((unsigned)f32_to_16(y[1], BF16) << 16);
      w.y = (unsigned)f32_to_16(y[2], BF16) | ((unsigned)f32_to_16(y[3], BF16) << 16);
      w.z = (unsigned)f32_to_16(y[4], BF16) | ((unsigned)f32_to_16(y[5], BF16) << 16);
      w.w = (unsigned)f32_to_16(y[6], BF16) | ((unsigned)f32_to_16(y[7], BF16) << 16);
      if (wrow0 + row < m) *reinterpret_cast<u32x4*>(out + (size_t)(wrow0 + row) * ld + sl * 8) = w;
    }
  }
}

}  // namespace iex
