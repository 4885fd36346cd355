// The direct-load GEMM tile of csrc/gemm_dma_device.cuh with switches that leave one ingredient of its main loop out at a
// time, for benchmarks/gemm_loop_ablation.hip.  A copy of that routine as it was when the ablation was taken; results of
// DBG builds are wrong on purpose, every address they use stays in bounds.  Not part of the library.
#pragma once
#include "../csrc/gemm_dma_device.cuh"

namespace iex {

// (the address arithmetic of a direct load without the load)
__device__ __forceinline__ void lds_dma16_address_only(const void* g, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\t; no load of %0" ::"v"(g), "s"(lds_base_uniform) : "memory", "m0");
}

// DBG (for the loop-ablation benchmark, benchmarks/gemm_loop_ablation.hip; results are wrong on purpose): 1 = no direct
// loads after the prologue (the stages keep the first tiles' data), 2 = no barrier per K step, 4 = no fragment reads from LDS (the MFMAs multiply what the first read left),
// 8 = the address arithmetic of the direct loads without the loads.
template <bool BF16, bool TRANS_B, int WM, int WN, int WCN, int BK, int STAGES, bool SPLIT = false, int DBG = 0>
__device__ __forceinline__ void gemm_tile_dma_ablation(const GemmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = 2 * WM * 32, BN = WCN * WN * 32, WAVES = 2 * WCN;
  constexpr int CPR = BK / 8;          // 16-byte chunks per K-contiguous row
  constexpr int RB = BK * 2;           // bytes per K-contiguous row
  constexpr int RPI = 64 / CPR;        // rows one wavefront instruction fills
  constexpr int A_BYTES = BM * BK * 2, B_BYTES = BN * BK * 2, STAGE_BYTES = A_BYTES + B_BYTES;
  constexpr int A_INSTR = A_BYTES / 1024 / WAVES, B_INSTR = B_BYTES / 1024 / WAVES;  // per wavefront and tile
  constexpr int LOADS = A_INSTR + B_INSTR;
  constexpr int CPRB = BN / 8;         // (K,N) layout: chunks per k row
  constexpr int RPIB = 64 / (CPRB < 64 ? CPRB : 64);  // (K,N) layout: k rows per instruction
  static_assert(BK == 32 || BK == 64, "K step");
  static_assert(A_INSTR >= 1 && B_INSTR >= 1 && A_BYTES % (1024 * WAVES) == 0 && B_BYTES % (1024 * WAVES) == 0,
                "every wavefront fetches whole kilobytes of A and of B");
  static_assert(TRANS_B || (CPRB >= 16 && CPRB <= 64), "(K,N) layout: 128 <= BN <= 512");
  static_assert(STAGES >= 3 && (BK / 16) % 2 == 0 && (STAGES - 2) * LOADS < 64, "stages in flight must fit the load counter");
  typedef unsigned short u16;
  typedef __attribute__((address_space(3))) unsigned char lds_u8;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WCN, wn = wave % WCN;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const u16* __restrict__ A = static_cast<const u16*>(p.A) + (size_t)z * p.stride_a;
  const u16* __restrict__ B = static_cast<const u16*>(p.B) + (size_t)z * p.stride_b;
  u16* __restrict__ C = static_cast<u16*>(p.C) + (size_t)z * p.stride_c;
  const unsigned lds0 = (unsigned)(size_t)(lds_u8*)smem;  // LDS byte address of stage 0
  const int ld = p.ldk ? p.ldk : p.K;  // row stride of the K-contiguous operands

  // ---- what this lane fetches: per instruction a row pointer (or a column offset) and a chunk
  const u16* a_row[A_INSTR];
  int a_k8[A_INSTR];  // element offset of the chunk inside a K step
#pragma unroll
  for (int q = 0; q < A_INSTR; ++q) {
    const int row = (wave * A_INSTR + q) * RPI + lane / CPR;
    const int sw = CPR == 4 ? (row >> 2) & 3 : (row >> 1) & 7;
    a_row[q] = A + (size_t)min(m0 + row, p.M - 1) * ld;
    a_k8[q] = ((lane % CPR) ^ sw) * 8;
  }
  const u16* b_row[B_INSTR];  // (N,K): row pointer; (K,N): B + clamped column
  int b_k8[B_INSTR];          // (N,K): chunk offset inside a K step; (K,N): k row inside a K step
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

  // instruction q of a tile: A for q < A_INSTR, then B
  auto issue_one = [&](int kt, int stage, int q) {
    const int k0 = min(kt, KT - 1) * BK;  // past the end: the last tile again, into a stage nobody reads
    if (q < A_INSTR) {
      const unsigned base = lds0 + stage * STAGE_BYTES + wave * (A_INSTR * 1024);
      (DBG & 8 ? lds_dma16_address_only : lds_dma16)(a_row[q] + min(k0 + a_k8[q], last_k8), __builtin_amdgcn_readfirstlane(base + q * 1024));
    } else {
      const int qb = q - A_INSTR;
      const unsigned bbase = lds0 + stage * STAGE_BYTES + A_BYTES + wave * (B_INSTR * 1024);
      if constexpr (TRANS_B)
        (DBG & 8 ? lds_dma16_address_only : lds_dma16)(b_row[qb] + min(k0 + b_k8[qb], last_k8), __builtin_amdgcn_readfirstlane(bbase + qb * 1024));
      else
        (DBG & 8 ? lds_dma16_address_only : lds_dma16)(b_row[qb] + (size_t)min(k0 + b_k8[qb], p.K - 1) * p.N, __builtin_amdgcn_readfirstlane(bbase + qb * 1024));
    }
  };
  auto issue = [&](int kt, int stage) {
#pragma unroll
    for (int q = 0; q < LOADS; ++q) issue_one(kt, stage, q);
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

  // ---- operand read addresses inside a stage (bytes), one per 16-wide sub-step (and per column
  // block for the transpose reads): the chunk permutation makes them differ by more than a constant
  constexpr int KS = BK / 16;
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
    // lane group q = lane / 16 covers column half (q % 2) and k half (q / 2) of a sub-step; lane r of a
    // group points at k row r / 4 and columns 4 * (r % 4) .. + 3 of its half
    const int kr = fkh * 8 + ((lane & 15) >> 2);
    const int s = ((lane >> 2) & 3) << 2;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int c = ((wn * WN + j) * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1)) ^ s;
      b_off[j] = A_BYTES + kr * (BN * 2) + c * 16 + (lane & 1) * 8;
    }
  }

  u32x4 fa[2][WM], fb[2][WN];  // operand fragments of two consecutive sub-steps
  bool have_frags[2] = {false, false};
  auto read_frags = [&](const unsigned char* st, int ks, int buf) {
    if constexpr ((DBG & 4) != 0) {   // (each register set once, then never again)
      if (have_frags[buf]) return;
      have_frags[buf] = true;
    }
#pragma unroll
    for (int i = 0; i < WM; ++i) fa[buf][i] = *reinterpret_cast<const u32x4*>(st + a_off[ks] + i * 32 * RB);
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      if constexpr (TRANS_B) {
        fb[buf][j] = *reinterpret_cast<const u32x4*>(st + b_off[ks] + j * 32 * RB);
      } else {
        typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
        const unsigned char* q0 = st + b_off[j] + ks * 16 * (BN * 2);
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0 + 4 * (BN * 2)));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        fb[buf][j] = u32x4{l2.x, l2.y, h2.x, h2.y};
      }
    }
  };

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue(s, s);
  const bool tail = (p.K % BK) != 0;
  wait_vmcnt<(STAGES - 2) * LOADS>();  // my loads of tile 0 have landed
  if (tail && KT == 1) zero_tail(0, 0);
  __syncthreads();
  read_frags(smem, 0, 0);

  // Sub-step g multiplies the fragments read during sub-step g - 1 and reads those of g + 1, so
  // the LDS latency hides behind MFMAs.  Before the first read of the next tile (last sub-step of
  // a tile): wait for my loads of that tile, barrier (everybody's have landed and everybody has
  // read the previous tile for the last time), and then the next direct loads are issued between
  // the MFMAs of this sub-step, into the stage the previous tile just left.
  constexpr int NM = WM * WN;
  for (int kt = 0; kt < KT; ++kt) {
    const unsigned char* st = smem + (kt % STAGES) * STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = ks & 1;
      if (ks + 1 < KS) {
        read_frags(st, ks + 1, cur ^ 1);
        __builtin_amdgcn_sched_barrier(0);  // reads first: the compiler would sink them behind the MFMAs
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j) acc[i][j] = mfma_32x32x16<BF16>(fb[cur][j], fa[cur][i], acc[i][j]);
      } else {
        wait_vmcnt<(STAGES - 3) * LOADS>();  // my loads of tile kt + 1 have landed
        if (tail && kt + 2 == KT) zero_tail(kt + 1, (kt + 1) % STAGES);
        if constexpr ((DBG & 2) == 0) __syncthreads();
        read_frags(smem + ((kt + 1) % STAGES) * STAGE_BYTES, 0, cur ^ 1);  // (past the last tile: read, never used)
        __builtin_amdgcn_sched_barrier(0);
        const int next = kt + STAGES - 1;
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j) {
            acc[i][j] = mfma_32x32x16<BF16>(fb[cur][j], fa[cur][i], acc[i][j]);
            const int m = i * WN + j;
#pragma unroll
            for (int q = m * LOADS / NM; q < (m + 1) * LOADS / NM; ++q)
              if constexpr ((DBG & 1) == 0) issue_one(next, next % STAGES, q);
          }
      }
    }
  }
  wait_vmcnt<0>();  // the re-fetched last tiles: nothing may still be writing LDS when the workgroup ends

  const float* partial = nullptr;
  if constexpr (SPLIT) {
    // Two workgroups hold partial sums of this tile (one half of K each).  Whichever finishes first leaves its sums in
    // the workspace and is done; the other adds them to its own and stores the tile (a + b = b + a: the result does
    // not depend on who was first).  The second only ever waits for a workgroup that is past its K loop and waits for
    // nothing itself.
    constexpr int NMT = WM * WN;
    const int tile_id = (z * p.tiles_m + tile_m) * p.tiles_n + tile_n;
    int* tickets = p.split_flags;
    int* written = p.split_flags + (size_t)gridDim.y * p.tiles_m * p.tiles_n;
    float* mine = p.split_ws + (size_t)tile_id * (BM * BN) + (size_t)wave * (NMT * 16 * 64) + lane * 4;
    __syncthreads();  // everybody has read its last fragments: the stages are free
    if (tid == 0) *reinterpret_cast<int*>(smem) = atomicAdd(&tickets[tile_id], 1);
    __syncthreads();
    const int ticket = *reinterpret_cast<volatile int*>(smem);
    if (ticket == 0) {
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const f32x4 v = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
            *reinterpret_cast<f32x4*>(mine + ((i * WN + j) * 4 + q) * 256) = v;
            if (q == 3) __builtin_amdgcn_sched_barrier(0);
          }
      // The two workgroups of a tile run on one XCD (the launcher's numbering; one partition spanning the whole GPU,
      // ids dealt round-robin to the XCDs), whose L2 both see.  Every wavefront waits until L2 has acknowledged its own
      // stores (vmcnt counts stores until then), the barrier collects all of them, and only then the flag goes up.
      // Device-scope fences here would write back and invalidate that L2 under every workgroup still multiplying
      // (measured: 2.5 x slower).
      wait_vmcnt<0>();
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __syncthreads();
      if (tid == 0) __hip_atomic_store(&written[tile_id], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    // (bounded: about a tenth of a second, far beyond any epilogue; a kernel must end whatever happens.  A wait that gives
    // up says so in the tile's flag word -- the host-visible error mark -- and the tile is not stored: never stale sums.)
    if (tid == 0) {
      int seen = 0;
      for (int spins = 0; spins < (1 << 20) && (seen = __hip_atomic_load(&written[tile_id], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) == 0; ++spins)
        __builtin_amdgcn_s_sleep(4);
      if (seen == 0) __hip_atomic_store(&written[tile_id], -1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *reinterpret_cast<volatile int*>(smem + 4) = seen;   // (the word after the ticket's: slow threads may still be reading that one)
    }
    __syncthreads();
    if (*reinterpret_cast<volatile int*>(smem + 4) == 0) return;   // (uniform) the partner never published: leave the tile unwritten, flag = -1
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");   // (this CU has never read these lines: they come from L2)
    partial = mine;   // added where the sums are rounded and stored (adding them here would need all 256 sums in VGPRs at once)
  }
  // the stages are free now: row-contiguous stores through LDS where the shape allows
  static_assert(WAVES * gemm_store_lds_bytes<WN>() <= gemm_dma_lds_bytes<WM, WN, WCN, BK, STAGES>(), "the epilogue fits the stages");
  if (!p.accumulate && p.N % 8 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0) {
    __syncthreads();  // everybody has read its last fragments
    gemm_store_tile_lds<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, smem + wave * gemm_store_lds_bytes<WN>(), p.stream_out != 0, partial);
  } else {
    gemm_store_tile<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, partial);
  }
}

}  // namespace iex
