// Instrumented twin of the ping-pong GEMM tile (csrc/gemm_pp_device.cuh) for benchmarks/gemm_pingpong_ablation.hip:
// every operand in 32-k stages (the shipped tile keeps A in 64-k stages), the grouping of the wavefronts and the
// number of stages as template parameters, and DBG switches that leave one ingredient of the loop out at a time
// (1 = no direct loads after the prologue, 2 = operand fragments read once, 16 / 32 = no A / no B loads, 64 = loads
// issued but never waited for, 128 = every load from one L1-resident 16 KB).  Results of DBG builds are wrong on
// purpose; every address they use stays in bounds.  Not part of the library.
//
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
// Stage reuse: tile t sits in stage t % STAGES and is read in intervals 2 t P - 1 ... 2 (t + 1) P - 2
// (P = BK / 32 phases per tile); the loads of tile t + STAGES go out in M phases of tile t + 1, all of which
// come later.  A wavefront waits for its own loads of tile t + 1 at the end of the interval before that tile's
// first read (group 0: after the last C phase of tile t, group 1: after the last M phase of tile t) and the
// barrier publishes them.  LDS layout, chunk permutation and the hand-written load counts are those of
// gemm_dma_device.cuh; per accumulator the MFMAs run in the same k order, so results are bit-equal to that
// kernel's.
#pragma once
#include "../csrc/gemm_dma_device.cuh"

namespace iex {

// The direct load of the library, with a cache modifier when the program is built with -DIEX_DMA_MOD='" sc0"' and the like.
#ifndef IEX_DMA_MOD
#define IEX_DMA_MOD ""
#endif
__device__ __forceinline__ void lds_dma16_mod(const void* g, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" IEX_DMA_MOD ::"v"(g), "s"(lds_base_uniform) : "memory", "m0");
}

// GMODE: which wavefronts form group 1: 0 = wavefronts 4..7 (the second wavefront of every SIMD when a
// workgroup's wavefronts are dealt round-robin to the four SIMDs), 1 = odd wavefronts, 2 = no second group
// (every wavefront in phase: the control experiment).
template <bool BF16, bool TRANS_B, int WM, int WN, int WCN, int BK, int STAGES, int GMODE = 0, int DBG = 0>
__device__ __forceinline__ void gemm_tile_ppx(const GemmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = 2 * WM * 32, BN = WCN * WN * 32, WAVES = 2 * WCN;
  constexpr int CPR = BK / 8;          // 16-byte chunks per K-contiguous row
  constexpr int RB = BK * 2;           // bytes per K-contiguous row
  constexpr int RPI = 64 / CPR;        // rows one wavefront instruction fills
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_INSTR = A_BYTES / 1024 / WAVES, B_INSTR = B_BYTES / 1024 / WAVES;  // per wavefront and tile
  constexpr int LOADS = A_INSTR + B_INSTR;
  constexpr int CPRB = BN / 8;         // (K,N) layout: chunks per k row
  constexpr int RPIB = 64 / (CPRB < 64 ? CPRB : 64);  // (K,N) layout: k rows per instruction
  constexpr int PPT = BK / 32;         // phases per tile
  constexpr int KS = BK / 16;
  static_assert(BK == 32 || BK == 64, "K step");
  static_assert(WAVES == 8, "two wavefronts per SIMD");
  static_assert(A_INSTR >= 1 && B_INSTR >= 1 && A_BYTES % (1024 * WAVES) == 0 && B_BYTES % (1024 * WAVES) == 0,
                "every wavefront fetches whole kilobytes of A and of B");
  static_assert(LOADS % PPT == 0, "the loads of a tile are spread evenly over its phases");
  static_assert(TRANS_B || (CPRB >= 16 && CPRB <= 64), "(K,N) layout: 128 <= BN <= 512");
  static_assert(STAGES >= 2 && (STAGES - 1) * LOADS < 64, "stages in flight must fit the load counter");
  typedef unsigned short u16;
  typedef __attribute__((address_space(3))) unsigned char lds_u8;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WCN, wn = wave % WCN;
  const int group = GMODE == 0 ? wave / 4 : GMODE == 1 ? (wave & 1) : 0;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const u16* __restrict__ A = static_cast<const u16*>(p.A) + (size_t)z * p.stride_a;
  const u16* __restrict__ B = static_cast<const u16*>(p.B) + (size_t)z * p.stride_b;
  u16* __restrict__ C = static_cast<u16*>(p.C) + (size_t)z * p.stride_c;
  const unsigned lds0 = (unsigned)(size_t)(lds_u8*)smem;  // LDS byte address of stage 0
  const int ld = p.ldk ? p.ldk : p.K;

  // ---- what this lane fetches: per instruction a row pointer (or a column offset) and a chunk
  const u16* a_row[A_INSTR];
  int a_k8[A_INSTR];
#pragma unroll
  for (int q = 0; q < A_INSTR; ++q) {
    const int row = (wave * A_INSTR + q) * RPI + lane / CPR;
    const int sw = CPR == 4 ? (row >> 2) & 3 : (row >> 1) & 7;
    a_row[q] = A + (size_t)min(m0 + row, p.M - 1) * ld;
    a_k8[q] = ((lane % CPR) ^ sw) * 8;
  }
  const u16* b_row[B_INSTR];
  int b_k8[B_INSTR];
#pragma unroll
  for (int q = 0; q < B_INSTR; ++q) {
    if constexpr (TRANS_B) {
      const int row = (wave * B_INSTR + q) * RPI + lane / CPR;
      const int sw = CPR == 4 ? (row >> 2) & 3 : (row >> 1) & 7;
      b_row[q] = B + (size_t)min(n0 + row, p.N - 1) * ld;
      b_k8[q] = ((lane % CPR) ^ sw) * 8;
    } else {
      const int kr = (wave * B_INSTR + q) * RPIB + lane / CPRB;
      const int c = (lane % CPRB) ^ ((kr & 3) << 2);
      b_row[q] = B + min(n0 + c * 8, p.N - 8);
      b_k8[q] = kr;
    }
  }
  const int last_k8 = p.K - 8;
  const int KT = (p.K + BK - 1) / BK;

  auto issue_one = [&](int kt, int stage, int q) {
    const int k0 = (DBG & 128) ? 0 : min(kt, KT - 1) * BK;  // past the end: the last tile again, into a stage nobody reads
    if constexpr ((DBG & 128) != 0) {
      const unsigned base = lds0 + stage * STAGE_BYTES + (q < A_INSTR ? 0 : A_BYTES) + wave * (A_INSTR * 1024);
      lds_dma16_mod(a_row[q % A_INSTR] + a_k8[q % A_INSTR], __builtin_amdgcn_readfirstlane(base + (q % A_INSTR) * 1024));
      return;
    }
    if (q < A_INSTR) {
      const unsigned base = lds0 + stage * STAGE_BYTES + wave * (A_INSTR * 1024);
      lds_dma16_mod(a_row[q] + min(k0 + a_k8[q], last_k8), __builtin_amdgcn_readfirstlane(base + q * 1024));
    } else {
      const int qb = q - A_INSTR;
      const unsigned bbase = lds0 + stage * STAGE_BYTES + A_BYTES + wave * (B_INSTR * 1024);
      if constexpr (TRANS_B)
        lds_dma16_mod(b_row[qb] + min(k0 + b_k8[qb], last_k8), __builtin_amdgcn_readfirstlane(bbase + qb * 1024));
      else
        lds_dma16_mod(b_row[qb] + (size_t)min(k0 + b_k8[qb], p.K - 1) * p.N, __builtin_amdgcn_readfirstlane(bbase + qb * 1024));
    }
  };
  // entries at k >= K of the last tile must be zero: clamped addresses delivered copies of real data
  auto zero_tail = [&](int kt, int stage) {
    const int k0 = kt * BK;
    unsigned char* st = smem + stage * STAGE_BYTES;
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < A_INSTR; ++q)
      if (k0 + a_k8[q] >= p.K) *reinterpret_cast<u32x4*>(st + ((wave * A_INSTR + q) * 64 + lane) * 16) = zero;
#pragma unroll
    for (int q = 0; q < B_INSTR; ++q)
      if (k0 + b_k8[q] >= p.K) *reinterpret_cast<u32x4*>(st + A_BYTES + ((wave * B_INSTR + q) * 64 + lane) * 16) = zero;
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
  const int fsw = CPR == 4 ? (frow >> 2) & 3 : (frow >> 1) & 7;
  int a_off[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) a_off[ks] = (wm * WM * 32 + frow) * RB + (((ks * 2 + fkh) ^ fsw) * 16);
  constexpr int NB = TRANS_B ? KS : WN;
  int b_off[NB];
  if constexpr (TRANS_B) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) b_off[ks] = A_BYTES + (wn * WN * 32 + frow) * RB + (((ks * 2 + fkh) ^ fsw) * 16);
  } else {
    const int kr = fkh * 8 + ((lane & 15) >> 2);
    const int s = ((lane >> 2) & 3) << 2;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int c = ((wn * WN + j) * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1)) ^ s;
      b_off[j] = A_BYTES + kr * (BN * 2) + c * 16 + (lane & 1) * 8;
    }
  }

  u32x4 fa[2][WM], fb[2][WN];  // the operand fragments of one phase (two sub-steps of 16)
  // DBG & 256 / & 512: B / A of a later tile comes through registers (a plain load in one memory phase, written to LDS
  // at the start of the wavefront's next memory phase, to the bytes the direct load would have filled) - K a multiple of BK only
  u32x4 areg[A_INSTR], breg[B_INSTR];
  int reg_stage = -1;
  // memory phase h of tile kt
  bool have = false;
  auto mem_phase = [&](int kt, int h) {
    const unsigned char* st = smem + (kt % STAGES) * STAGE_BYTES;
    if constexpr ((DBG & (256 | 512)) != 0) {
      if (reg_stage >= 0) {
        unsigned char* dst = smem + reg_stage * STAGE_BYTES;
        if constexpr ((DBG & 512) != 0) {
#pragma unroll
          for (int q = 0; q < A_INSTR; ++q) *reinterpret_cast<u32x4*>(dst + ((wave * A_INSTR + q) * 64 + lane) * 16) = areg[q];
        }
        if constexpr ((DBG & 256) != 0) {
#pragma unroll
          for (int q = 0; q < B_INSTR; ++q) *reinterpret_cast<u32x4*>(dst + A_BYTES + ((wave * B_INSTR + q) * 64 + lane) * 16) = breg[q];
        }
      }
    }
    const bool skip = (DBG & 2) && have;
    have = true;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      if (skip) continue;
      const int ks = h * 2 + s;
#pragma unroll
      for (int i = 0; i < WM; ++i) fa[s][i] = *reinterpret_cast<const u32x4*>(st + a_off[ks] + i * 32 * RB);
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        if constexpr (TRANS_B) {
          fb[s][j] = *reinterpret_cast<const u32x4*>(st + b_off[ks] + j * 32 * RB);
        } else {
          typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
          const unsigned char* q0 = st + b_off[j] + ks * 16 * (BN * 2);
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0 + 4 * (BN * 2)));
          const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
          fb[s][j] = u32x4{l2.x, l2.y, h2.x, h2.y};
        }
      }
    }
    const int next = kt + STAGES - 1;
#pragma unroll
    for (int q = h * (LOADS / PPT); q < (h + 1) * (LOADS / PPT); ++q) {
      if constexpr ((DBG & 1) != 0) continue;
      if ((DBG & 16) && q < A_INSTR) continue;
      if ((DBG & 32) && q >= A_INSTR) continue;
      if ((DBG & 512) && q < A_INSTR) {
        areg[q] = *reinterpret_cast<const u32x4*>(a_row[q] + min(min(next, KT - 1) * BK + a_k8[q], last_k8));
        continue;
      }
      if ((DBG & 256) && q >= A_INSTR) {
        const int qb = q - A_INSTR;
        if constexpr (TRANS_B) breg[qb] = *reinterpret_cast<const u32x4*>(b_row[qb] + min(min(next, KT - 1) * BK + b_k8[qb], last_k8));
        else breg[qb] = *reinterpret_cast<const u32x4*>(b_row[qb] + (size_t)min(min(next, KT - 1) * BK + b_k8[qb], p.K - 1) * p.N);
        continue;
      }
      issue_one(next, next % STAGES, q);
    }
    if constexpr ((DBG & (256 | 512)) != 0) reg_stage = next % STAGES;
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
  // my loads of tile kt + 1 have landed (the tiles after it may still be in flight); zero its K tail
  const bool tail = (p.K % BK) != 0;
  auto landed = [&](int kt) {
    if constexpr ((DBG & (1|16|32|64)) == 0) wait_vmcnt<(STAGES - 2) * LOADS>(); else if constexpr ((DBG&(1|64))==0) wait_vmcnt<0>();
    if (tail && kt + 2 == KT) zero_tail(kt + 1, (kt + 1) % STAGES);
  };
  auto interval_end = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
#pragma unroll
    for (int q = 0; q < LOADS; ++q) issue_one(s, s, q);
  wait_vmcnt<(STAGES - 2) * LOADS>();  // my loads of tile 0 have landed
  if (tail && KT == 1) zero_tail(0, 0);
  __syncthreads();

  if (group == 0) {
    mem_phase(0, 0);
    interval_end();
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
      for (int h = 0; h < PPT; ++h) {
        compute_phase();
        if (h == PPT - 1) landed(kt);
        interval_end();
        if (h + 1 < PPT) mem_phase(kt, h + 1);
        else mem_phase(kt + 1, 0);   // (past the last tile: read, never used)
        interval_end();
      }
    }
  } else {
    interval_end();
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
      for (int h = 0; h < PPT; ++h) {
        mem_phase(kt, h);
        if (h == PPT - 1) landed(kt);
        interval_end();
        compute_phase();
        interval_end();
      }
    }
  }
  wait_vmcnt<0>();  // the re-fetched last tiles: nothing may still be writing LDS when the stages are reused

  static_assert(WAVES * gemm_store_lds_bytes<WN>() <= STAGES * STAGE_BYTES, "the epilogue fits the stages");
  if (!p.accumulate && p.N % 8 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0) {
    __syncthreads();  // everybody has read its last fragments and nobody's loads are in flight
    gemm_store_tile_lds<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, smem + wave * gemm_store_lds_bytes<WN>(), p.stream_out != 0, nullptr);
  } else {
    gemm_store_tile<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, nullptr);
  }
}

}  // namespace iex
