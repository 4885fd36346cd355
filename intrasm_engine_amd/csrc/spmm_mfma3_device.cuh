// CSR SpMM on the matrix cores, third arrangement (fp16 / bf16): 8 wavefronts (2 x 4), C tile
// 128 x 512, K steps of 32, and no staging registers on the dense side, as in the GEMM of
// gemm_dma_device.cuh:
//   B (k x n, dense) is loaded from global memory straight into a ring of three LDS stages
//     (global_load_lds_dwordx4, chunk-permuted rows, no registers and no ds_write on the way);
//   A (sparse) is expanded 64 columns (two K steps) at a time: while the two steps of one half
//     chunk are multiplied, every lane group (16 lanes, 4 rows) scatters the nonzeros of its rows
//     that fall into the next 64 columns into the other A stage (128 rows x 64 columns, chunk-
//     permuted, zero-filled first by the same wavefront), two rows per step.
// A row's share of a half chunk sits in W register windows of 16 nonzeros (W = 1, 2 or 4; 4 always
// holds it).  With fewer, a row that has more (seen exactly, by one look-ahead load per row)
// raises a flag, and the workgroup multiplies that half chunk once more with what the windows
// left behind.  The host picks W from the density; a wrong guess costs time, not correctness.
// Every load of the main loop is unconditional with a fixed count per step: the hand-written wait
// for the direct loads relies on it (the window loads are ordinary loads, counted by the compiler;
// it does not see the direct loads, so its waits are a few loads stricter than needed, never
// laxer).  A step always requests the B tile that follows the next step's; when a half chunk is
// repeated that is a tile already in LDS, fetched again to the same place.
// LDS: 2 x 16 KB (A) + 3 x 32 KB (B).  The dense form of A never exists anywhere else.
// Requirements (checked by the host): n % 8 == 0, 16-byte aligned dense operand and output,
// nnz > 0, ascending column indices without duplicates inside a row.  Like every matrix-core
// family it multiplies the explicit zeros of the expanded tile with the dense operand.
#pragma once
#include "gemm_dma_device.cuh"
#include "spmm_mfma_device.cuh"

namespace iex {

constexpr int kMfma3BN = 512;
constexpr int kMfma3Threads = 512;
constexpr int kMfma3Stages = 3;
constexpr int kMfma3G = 64;                          // columns of A expanded at a time
constexpr int kMfma3AStage = kMfmaBM * kMfma3G * 2;  // bytes of one A stage
constexpr int kMfma3BStage = 32 * kMfma3BN * 2;      // bytes of one B stage
constexpr int spmm_mfma3_lds_bytes() { return 2 * kMfma3AStage + kMfma3Stages * kMfma3BStage + 16 + kMfma3Threads * 4; }

template <bool BF16, typename IT, int W>
__device__ __forceinline__ void spmm_mfma3_block(const SpmmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = kMfmaBM, BN = kMfma3BN, BK = 32, STAGES = kMfma3Stages, G = kMfma3G;
  constexpr int WM = 2, WN = 4, WCN = 4, WAVES = 8;
  constexpr int LPR = 16;                        // lanes per row-visit = nonzeros per window
  constexpr bool PEEK = W * LPR < G;             // the windows may not hold a half chunk's share: look ahead
  constexpr int GROUPS = kMfma3Threads / LPR;    // 32 lane groups
  constexpr int R = BM / GROUPS;                 // 4 rows per group, 2 expanded per step
  constexpr int RB = G * 2;                      // bytes of an A stage row
  constexpr int B_INSTR = kMfma3BStage / 1024 / WAVES;           // direct loads per wavefront and step (4)
  constexpr int WINDOW_LOADS = 2 * (W * 2 + (PEEK ? 1 : 0));     // ordinary loads per lane and step
  constexpr int NM = WM * WN;
  static_assert(W == 1 || W == 2 || W == 4, "windows per row");
  static_assert((STAGES - 2) * WINDOW_LOADS + (STAGES - 3) * B_INSTR < 64, "the load counter has 6 bits");
  typedef unsigned short u16;
  typedef __attribute__((address_space(3))) unsigned char lds_u8;

  unsigned char* sA = smem;                      // [2][BM][G] halves, chunk-permuted rows
  unsigned char* sB = smem + 2 * kMfma3AStage;   // [STAGES][32][BN] halves, chunk-permuted rows
  int* again = reinterpret_cast<int*>(sB + STAGES * kMfma3BStage);  // [3]: raised, read and cleared in turn
  // One word per lane that absorbs the writes of lanes with nothing to write: a predicated store is a
  // branch around it, and branches cut the step into blocks across which the compiler cannot
  // interleave the expansion with the MFMAs.
  int* sink = again + 4 + threadIdx.x;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WCN, wn = wave % WCN;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const u16* __restrict__ values = static_cast<const u16*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
  const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
  const u16* __restrict__ B = static_cast<const u16*>(p.dense) + (size_t)z * p.k * p.n;
  u16* __restrict__ C = static_cast<u16*>(p.out) + (size_t)z * p.m * p.n;
  const unsigned ldsB = (unsigned)(size_t)(lds_u8*)sB;
  const int KT = (p.k + BK - 1) / BK;            // K steps
  const int HT = (p.k + G - 1) / G;              // half chunks

  // ---- direct loads of B: instruction q of this wavefront fills k row wave * B_INSTR + q of a stage
  const u16* b_col[B_INSTR];
#pragma unroll
  for (int q = 0; q < B_INSTR; ++q) {
    const int kr = wave * B_INSTR + q;
    const int c = lane ^ ((kr & 3) << 2);        // which 16-byte chunk of the row this lane fetches
    b_col[q] = B + min(n0 + c * 8, p.n - 8);
  }
  auto issue_one = [&](int kt, int q) {
    const int t = min(kt, KT - 1);               // past the end: the last tile again, into a stage nobody reads
    const int kr = wave * B_INSTR + q;
    lds_dma16(b_col[q] + (size_t)min(t * BK + kr, p.k - 1) * p.n,
              __builtin_amdgcn_readfirstlane(ldsB + (kt % STAGES) * kMfma3BStage + kr * 1024));
  };

  // ---- expansion state: cursor, row end and the windows for each of the 4 rows
  const int sub = tid % LPR;
  const int group = tid / LPR;
  const int gshift = lane & ~(LPR - 1);
  const int last_nz = p.nnz - 1;
  int pos[R], end[R];
  u16 wval[R][W];
  IT wcol[R][W];
  IT wpeek[R];
  auto load_windows = [&](int j) {
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const int safe = min(pos[j] + w * LPR + sub, last_nz);  // raw, clamped; validity is decided at use
      wval[j][w] = values[safe];
      wcol[j][w] = cols[safe];
    }
    if constexpr (PEEK) wpeek[j] = cols[min(pos[j] + W * LPR, last_nz)];
  };
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int slot = m0 + group + j * GROUPS;
    pos[j] = end[j] = 0;
    if (slot < p.m) {
      const int row = p.row_indices[slot];
      pos[j] = p.row_offsets[row];
      end[j] = p.row_offsets[row + 1];
    }
    load_windows(j);
  }
  const int asw8 = ((group >> 1) & 7) << 3;      // chunk permutation of this group's rows ((row >> 1) & 7), as a column XOR
  auto zero_rows = [&](unsigned char* abuf) {    // the 4 rows of this group: 512 bytes, 32 per lane
#pragma unroll
    for (int h = 0; h < 2; ++h)
      *reinterpret_cast<u32x4*>(abuf + (group + (sub >> 2) * GROUPS) * RB + ((sub & 3) * 2 + h) * 16) = u32x4{0u, 0u, 0u, 0u};
  };
  // columns [k0, k0 + G) of row j of this group -> A stage `abuf`
  auto expand_row = [&](int j, int k0, unsigned char* abuf, int* flag) {
    u16* rowp = reinterpret_cast<u16*>(abuf + (group + j * GROUPS) * RB);
    const int kend = k0 + G;
    int consumed = 0;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const int c = (int)wcol[j][w];
      const bool in = pos[j] + w * LPR + sub < end[j] && c < kend;
      u16* dst = in ? rowp + ((c - k0) ^ asw8) : reinterpret_cast<u16*>(sink);
      *dst = wval[j][w];
      consumed += __popcll((__ballot(in) >> gshift) & 0xffffull);
    }
    if constexpr (PEEK) {
      const bool more = consumed == W * LPR && pos[j] + W * LPR < end[j] && (int)wpeek[j] < kend;
      *(more ? flag : sink) = 1;
    }
    pos[j] += consumed;
    load_windows(j);
  };

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- operand read addresses inside a stage (bytes): one per 16-wide sub-step of an A stage
  const int frow = lane & 31, fkh = lane >> 5;
  const int fsw = (frow >> 1) & 7;
  int a_off[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) a_off[ks] = (wm * WM * 32 + frow) * RB + (((ks * 2 + fkh) ^ fsw) * 16);
  int b_off[WN];
  {
    const int kr = fkh * 8 + ((lane & 15) >> 2);
    const int s = ((lane >> 2) & 3) << 2;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int c = ((wn * WN + j) * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1)) ^ s;
      b_off[j] = kr * (BN * 2) + c * 16 + (lane & 1) * 8;
    }
  }
  u32x4 fa[2][WM], fb[2][WN];
  // sub-step ks (0..3) of A stage `a`, sub-step ks % 2 of B stage `b`
  auto read_frags = [&](const unsigned char* a, const unsigned char* b, int ks, int buf) {
#pragma unroll
    for (int i = 0; i < WM; ++i) fa[buf][i] = *reinterpret_cast<const u32x4*>(a + a_off[ks] + i * 32 * RB);
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
      const unsigned char* q0 = b + b_off[j] + (ks & 1) * 16 * (BN * 2);
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0 + 4 * (BN * 2)));
      const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      fb[buf][j] = u32x4{l2.x, l2.y, h2.x, h2.y};
    }
  };

  // ---- prologue: A stage of half chunk 0, B tiles 0 .. STAGES-2, everything landed (one exposed latency)
  if (tid < 3) again[tid] = 0;
  zero_rows(sA);
  __syncthreads();
#pragma unroll
  for (int j = 0; j < R; ++j) expand_row(j, 0, sA, again);
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
#pragma unroll
    for (int q = 0; q < B_INSTR; ++q) issue_one(s, q);
  wait_vmcnt<0>();
  __syncthreads();
  read_frags(sA, sB, 0, 0);
  bool repeat = PEEK && __builtin_amdgcn_readfirstlane(again[0]) != 0;

  // Round i multiplies half chunk hm (K steps 2 hm and 2 hm + 1) out of A stage i % 2 and expands
  // half chunk he (hm again when the last expansion left nonzeros behind, else hm + 1) into the
  // other one, rows 0-1 during the first step, rows 2-3 during the second.  One step: sub-step 0
  // multiplies the fragments read before, reads those of sub-step 1 and expands two rows between
  // its MFMAs; then: wait for my direct loads of the next step's B tile, barrier, read the first
  // fragments of the next step, and request the tile after that one between the MFMAs of sub-step 1.
  // Loads younger than the awaited tile's at the wait: the windows of this step.
  int hm = 0;
  for (int i = 0; hm < HT; ++i) {
    const int he = repeat ? hm : hm + 1;
    const unsigned char* a = sA + (i & 1) * kMfma3AStage;
    unsigned char* a_next = sA + ((i + 1) & 1) * kMfma3AStage;
    int* flag = again + (i + 1) % 3;
    zero_rows(a_next);
#pragma unroll
    for (int J = 0; J < 2; ++J) {
      const int km = 2 * hm + J;                       // K step multiplied now
      const int kn = J == 0 ? km + 1 : 2 * he;         // K step multiplied next
      read_frags(a, sB + (km % STAGES) * kMfma3BStage, 2 * J + 1, 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mi = 0; mi < WM; ++mi)
#pragma unroll
        for (int j = 0; j < WN; ++j) {
          acc[mi][j] = mfma_32x32x16<BF16>(fb[0][j], fa[0][mi], acc[mi][j]);
          const int m = mi * WN + j;
          if (m % (NM / 2) == 0) expand_row(2 * J + m / (NM / 2), he * G, a_next, flag);
        }
      wait_vmcnt<(STAGES - 2) * WINDOW_LOADS + (STAGES - 3) * B_INSTR>();
      __syncthreads();
      // (past the last step: read, never used)
      read_frags(J == 0 ? a : a_next, sB + (kn % STAGES) * kMfma3BStage, J == 0 ? 2 : 0, 0);
      if constexpr (PEEK) {
        if (J == 1) {
          repeat = __builtin_amdgcn_readfirstlane(*flag) != 0;
          if (tid == 0) again[i % 3] = 0;  // read one round ago, raised again two rounds from now
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mi = 0; mi < WM; ++mi)
#pragma unroll
        for (int j = 0; j < WN; ++j) {
          acc[mi][j] = mfma_32x32x16<BF16>(fb[1][j], fa[1][mi], acc[mi][j]);
          const int m = mi * WN + j;
          if (m % (NM / B_INSTR) == 0) issue_one(kn + STAGES - 2, m / (NM / B_INSTR));
        }
    }
    hm = he;
  }
  wait_vmcnt<0>();  // the re-fetched last tiles: nothing may still be writing LDS when the workgroup ends

  spmm_mfma_epilogue<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, smem);
}

}  // namespace iex
