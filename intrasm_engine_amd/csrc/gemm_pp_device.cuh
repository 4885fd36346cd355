// Dense GEMM tile for gfx950 by eight wavefronts in two groups that alternate roles ("ping-pong").
//
// The direct-load tile of gemm_dma_device.cuh interleaves three things in one instruction stream: MFMAs,
// LDS reads of the next operand fragments and the direct loads of a later tile.  Every wait of that
// stream (fragments not there yet, my loads of the next tile not landed, the barrier) is a bubble in the
// matrix pipeline of its SIMD, because nothing else runs there.  Here a SIMD holds two wavefronts, one of
// each group, and the groups run half a K step apart:
//
//     interval      2p-1          2p            2p+1          2p+2
//     group 0       M(p)          C(p)          M(p+1)        C(p+1)
//     group 1       C(p-1)        M(p)          C(p)          M(p+1)
//
//   M(p)  = memory phase p: read the operand fragments of 32 k of the tile from LDS into registers,
//           issue my share of the direct loads (global memory -> LDS) of the tile STAGES - 1 ahead;
//   C(p)  = compute phase p: the WM x WN x 2 MFMAs on those fragments, nothing else.
// Intervals are separated by workgroup barriers, so on every SIMD one wavefront feeds the matrix cores while
// the other one waits for LDS and issues loads, and all waits hide behind the other group's MFMAs.
// A wavefront owns WM x WN MFMA tiles of 32 x 32 (128 x 64 of a 256 x 256 tile with WM = 4, WN = 2, WCN = 4).
//
// Stage reuse: what phase p reads was last needed by phase p (group 1 reads it one interval after group 0), and the
// loads that overwrite it go out in later M phases.  A wavefront waits for its own loads of what phase p + 1 reads at
// the end of the interval before group 0 reads it (group 0: after C(p), group 1: after M(p)) and the barrier publishes
// them.  Chunk permutations and the hand-written load counts follow gemm_dma_device.cuh; per accumulator the MFMAs
// run in the same k order, so results are bit-equal to that kernel's.
#pragma once
#include "gemm_dma_device.cuh"

namespace iex {

// Stages.  A rows are K-contiguous, and a direct load moves 16 bytes per lane: with 32 k per stage a row is
// 64 bytes, half a cache line, and every line of A crosses the L1 twice, a K step apart (counters on 8192^3: 13.0 GB
// requested from L2 for 8.6 GB of operands, the texture-data unit busy 83 % of the cycles at 20 bytes per clock).  So A is
// staged 64 k at a time (whole lines, three stages), B 32 k at a time (four stages): 3 * BM * 128 + 4 * BN * 64 bytes,
// 160 KB for 256 x 256 tiles.  Phase p reads the half p % 2 of A tile p / 2 and B tile p, and issues half of the loads
// of A tile p / 2 + 2 and all loads of B tile p + 3; every wavefront issues the same number of loads LPP in every
// phase, so "my loads of everything that phase p + 1 reads have landed" is vmcnt(2 * LPP) at the end of phase p.
template <bool BF16, bool TRANS_B, int WM, int WN, int WCN>
constexpr int gemm_pp_lds_bytes() { return 3 * (2 * WM * 32) * 128 + 4 * (WCN * WN * 32) * 64; }

template <bool BF16, bool TRANS_B, int WM, int WN, int WCN>
__device__ __forceinline__ void gemm_tile_pp(const GemmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = 2 * WM * 32, BN = WCN * WN * 32, WAVES = 2 * WCN;
  constexpr int SA = 3, SB = 4;                       // stages of A (64 k each) and of B (32 k each)
  constexpr int A_STAGE = BM * 128, B_STAGE = BN * 64;
  constexpr int B_BASE = SA * A_STAGE;
  constexpr int A_INSTR = A_STAGE / 1024 / WAVES;     // direct loads per wavefront and A tile
  constexpr int B_INSTR = B_STAGE / 1024 / WAVES;     // ... and B tile
  constexpr int LPP = A_INSTR / 2 + B_INSTR;          // loads per wavefront and phase
  constexpr int CPRB = BN / 8;                        // (K,N) layout: chunks per k row
  constexpr int RPIB = 64 / (CPRB < 64 ? CPRB : 64);  // (K,N) layout: k rows per instruction
  static_assert(WAVES == 8, "two wavefronts per SIMD");
  static_assert(A_INSTR >= 2 && A_INSTR % 2 == 0 && B_INSTR >= 1 && A_STAGE % (1024 * WAVES) == 0 && B_STAGE % (1024 * WAVES) == 0,
                "every wavefront fetches whole kilobytes of A (in two halves) and of B");
  static_assert(TRANS_B || (CPRB >= 16 && CPRB <= 64), "(K,N) layout: 128 <= BN <= 512");
  static_assert(3 * LPP < 64, "loads in flight must fit the load counter");
  typedef unsigned short u16;
  typedef __attribute__((address_space(3))) unsigned char lds_u8;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WCN, wn = wave % WCN;
  const int group = wave / 4;   // wavefronts w and w + 4 share a SIMD (measured: pairing w with w ^ 1 instead loses 15 %)
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const u16* __restrict__ A = static_cast<const u16*>(p.A) + (size_t)z * p.stride_a;
  const u16* __restrict__ B = static_cast<const u16*>(p.B) + (size_t)z * p.stride_b;
  u16* __restrict__ C = static_cast<u16*>(p.C) + (size_t)z * p.stride_c;
  const unsigned lds0 = (unsigned)(size_t)(lds_u8*)smem;
  const int ld = p.ldk ? p.ldk : p.K;  // row stride of the K-contiguous operands

  // ---- what this lane fetches.  A: 8 rows of 128 bytes per instruction, LDS position (row, c) holds global chunk
  // c ^ ((row >> 1) & 7).  B as (N,K): 16 rows of 64 bytes, chunk c ^ ((row >> 2) & 3).  B as (K,N): k rows of BN
  // elements, chunk c ^ ((k & 3) << 2).
  const u16* a_ptr[A_INSTR];   // row pointer + chunk offset, advanced by 64 k per A tile
#pragma unroll
  for (int q = 0; q < A_INSTR; ++q) {
    const int row = (wave * A_INSTR + q) * 8 + lane / 8;
    const int sw = (row >> 1) & 7;
    a_ptr[q] = A + (size_t)min(m0 + row, p.M - 1) * ld + ((lane % 8) ^ sw) * 8;
  }
  int a_k8[A_INSTR];
#pragma unroll
  for (int q = 0; q < A_INSTR; ++q) {
    const int row = (wave * A_INSTR + q) * 8 + lane / 8;
    a_k8[q] = ((lane % 8) ^ ((row >> 1) & 7)) * 8;
  }
  const u16* b_row[B_INSTR];
  int b_k8[B_INSTR];
#pragma unroll
  for (int q = 0; q < B_INSTR; ++q) {
    if constexpr (TRANS_B) {
      const int row = (wave * B_INSTR + q) * 16 + lane / 4;
      const int sw = (row >> 2) & 3;
      b_row[q] = B + (size_t)min(n0 + row, p.N - 1) * ld;
      b_k8[q] = ((lane % 4) ^ sw) * 8;
    } else {
      const int kr = (wave * B_INSTR + q) * RPIB + lane / CPRB;
      const int c = (lane % CPRB) ^ ((kr & 3) << 2);
      b_row[q] = B + min(n0 + c * 8, p.N - 8);
      b_k8[q] = kr;
    }
  }
  const int last_k8 = p.K - 8;
  const int P = (p.K + 31) / 32;       // phases
  const int TA = (p.K + 63) / 64;      // A tiles

  // half h (instructions h * A_INSTR / 2 ...) of A tile t; past the end: the last tile again, into a stage nobody reads
  auto issue_a = [&](int t, auto half) {
    constexpr int h = decltype(half)::value;   // (compile-time: a_ptr stays in registers)
    const int k0 = min(t, TA - 1) * 64;
    const unsigned base = lds0 + (t % SA) * A_STAGE + wave * (A_INSTR * 1024);
#pragma unroll
    for (int q = h * (A_INSTR / 2); q < (h + 1) * (A_INSTR / 2); ++q) {
      const int over = max(k0 + a_k8[q] - last_k8, 0);   // a chunk past the last one of the row: that one instead
      lds_dma16(a_ptr[q] + (k0 - over), __builtin_amdgcn_readfirstlane(base + q * 1024));
    }
  };
  auto issue_b = [&](int t) {
    const int k0 = min(t, P - 1) * 32;
    const unsigned base = lds0 + B_BASE + (t % SB) * B_STAGE + wave * (B_INSTR * 1024);
#pragma unroll
    for (int q = 0; q < B_INSTR; ++q) {
      if constexpr (TRANS_B)
        lds_dma16(b_row[q] + min(k0 + b_k8[q], last_k8), __builtin_amdgcn_readfirstlane(base + q * 1024));
      else
        lds_dma16(b_row[q] + (size_t)min(k0 + b_k8[q], p.K - 1) * p.N, __builtin_amdgcn_readfirstlane(base + q * 1024));
    }
  };
  // entries at k >= K must be zero: clamped addresses delivered copies of real data.  Phase ph is the last one.
  auto zero_tail = [&](int ph) {
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const int ta = ph / 2;
    unsigned char* sa = smem + (ta % SA) * A_STAGE;
#pragma unroll
    for (int q = 0; q < A_INSTR; ++q)
      if (ta * 64 + a_k8[q] >= p.K) *reinterpret_cast<u32x4*>(sa + ((wave * A_INSTR + q) * 64 + lane) * 16) = zero;
    unsigned char* sb = smem + B_BASE + (ph % SB) * B_STAGE;
#pragma unroll
    for (int q = 0; q < B_INSTR; ++q)
      if (ph * 32 + b_k8[q] >= p.K) *reinterpret_cast<u32x4*>(sb + ((wave * B_INSTR + q) * 64 + lane) * 16) = zero;
  };

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- operand read addresses inside a stage (bytes), one per 16-wide sub-step
  const int frow = lane & 31, fkh = lane >> 5;
  int a_off[4];   // the four sub-steps of an A tile
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) a_off[ks] = (wm * WM * 32 + frow) * 128 + (((ks * 2 + fkh) ^ ((frow >> 1) & 7)) * 16);
  constexpr int NB = TRANS_B ? 2 : WN;
  int b_off[NB];
  if constexpr (TRANS_B) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) b_off[ks] = B_BASE + (wn * WN * 32 + frow) * 64 + (((ks * 2 + fkh) ^ ((frow >> 2) & 3)) * 16);
  } else {
    // lane group q = lane / 16 covers column half (q % 2) and k half (q / 2) of a sub-step; lane r of a
    // group points at k row r / 4 and columns 4 * (r % 4) .. + 3 of its half
    const int kr = fkh * 8 + ((lane & 15) >> 2);
    const int s = ((lane >> 2) & 3) << 2;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int c = ((wn * WN + j) * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1)) ^ s;
      b_off[j] = B_BASE + kr * (BN * 2) + c * 16 + (lane & 1) * 8;
    }
  }

  u32x4 fa[2][WM], fb[2][WN];  // the operand fragments of one phase (two sub-steps of 16)
  const std::integral_constant<int, 0> even;
  const std::integral_constant<int, 1> odd;
  // parity = ph % 2 at compile time: which half of the A tile
  auto mem_phase = [&](int ph, auto parity) {
    constexpr int h = decltype(parity)::value;
    const unsigned char* sa = smem + ((ph >> 1) % SA) * A_STAGE;
    const unsigned char* sb = smem + (ph % SB) * B_STAGE;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const int ao = a_off[2 * h + s];
#pragma unroll
      for (int i = 0; i < WM; ++i) fa[s][i] = *reinterpret_cast<const u32x4*>(sa + ao + i * 32 * 128);
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        if constexpr (TRANS_B) {
          fb[s][j] = *reinterpret_cast<const u32x4*>(sb + b_off[s] + j * 32 * 64);
        } else {
          typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
          const unsigned char* q0 = sb + b_off[j] + s * 16 * (BN * 2);
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0 + 4 * (BN * 2)));
          const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
          fb[s][j] = u32x4{l2.x, l2.y, h2.x, h2.y};
        }
      }
    }
    issue_a((ph >> 1) + 2, parity);
    issue_b(ph + 3);
  };
  auto compute_phase = [&]() {
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) acc[i][j] = mfma_32x32x16<BF16>(fb[s][j], fa[s][i], acc[i][j]);
    __builtin_amdgcn_s_setprio(0);
  };
  // at the end of phase ph: my loads of what phase ph + 1 reads have landed (two phases' worth may still fly)
  const bool tail = (p.K % 32) != 0;
  auto landed = [&](int ph) {
    wait_vmcnt<2 * LPP>();
    if (tail && ph + 2 == P) zero_tail(ph + 1);
  };
  auto interval_end = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };

  // prologue = the loads that phases -4 .. -1 would have issued
  issue_a(0, even);
  issue_a(0, odd); issue_b(0);
  issue_a(1, even); issue_b(1);
  issue_a(1, odd); issue_b(2);
  wait_vmcnt<2 * LPP>();  // A tile 0 and B tile 0 have landed
  if (tail && P == 1) zero_tail(0);
  __syncthreads();

  // (loops over pairs of phases with one exit each, the odd last phase after them: a loop with a second exit in its
  // middle makes the compiler keep two copies of the accumulators)
  int ph = 0;
  if (group == 0) {
    mem_phase(0, even);
    interval_end();
    for (; ph + 2 <= P; ph += 2) {
      compute_phase();
      landed(ph);
      interval_end();
      mem_phase(ph + 1, odd);
      interval_end();
      compute_phase();
      landed(ph + 1);
      interval_end();
      mem_phase(ph + 2, even);   // (past the last phase: read, never used)
      interval_end();
    }
    if (ph < P) {
      compute_phase();
      landed(ph);
      interval_end();
      mem_phase(ph + 1, odd);
      interval_end();
    }
  } else {
    interval_end();
    for (; ph + 2 <= P; ph += 2) {
      mem_phase(ph, even);
      landed(ph);
      interval_end();
      compute_phase();
      interval_end();
      mem_phase(ph + 1, odd);
      landed(ph + 1);
      interval_end();
      compute_phase();
      interval_end();
    }
    if (ph < P) {
      mem_phase(ph, even);
      landed(ph);
      interval_end();
      compute_phase();
      interval_end();
    }
  }
  wait_vmcnt<0>();  // the re-fetched last tiles: nothing may still be writing LDS when the stages are reused

  static_assert(WAVES * gemm_store_lds_bytes<WN>() <= SA * A_STAGE, "the epilogue fits the stages");
  if (!p.accumulate && p.N % 8 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0) {
    __syncthreads();  // everybody has read its last fragments and nobody's loads are in flight
    gemm_store_tile_lds<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, smem + wave * gemm_store_lds_bytes<WN>(), p.stream_out != 0, nullptr);
  } else {
    gemm_store_tile<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, nullptr);
  }
}

}  // namespace iex
