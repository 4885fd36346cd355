// Dense GEMM tile for gfx950 whose operands travel from global memory straight into LDS
// (global_load_lds_dwordx4): no staging registers and no ds_write in the main loop.
//
// Why: a ds_write_b128 stream runs at 64 bytes/clock/CU and, while it runs, takes a quarter of
// the LDS read rate away from the MFMA operand reads; with register staging the writes of one K
// step cost as many LDS cycles as all operand reads of that step, and LDS time equals MFMA time.
// A direct-to-LDS load costs the readers 6 % (measured with reader and writer wavefronts side by
// side).
//
// A direct load writes lane i's 16 bytes at M0 + 16 * i: one wavefront instruction fills 1 KB of
// LDS contiguously, so rows cannot be padded.  Bank conflicts are avoided by permuting WHICH 16-byte
// chunk of global memory each lane fetches instead:
//   K-contiguous operands (A, and B given as (N, K)): LDS row = BK elements; position (row, c)
//     holds global chunk c ^ sw(row), sw(row) = (row >> 2) & 3 for BK = 32 ((row >> 1) & 7 for 64):
//     the 16 lanes of a 128-bit operand read hit 16 different 4-bank groups.
//   B given as (K, N): LDS row = BN elements; position (k, c) holds global chunk c ^ ((k & 3) << 2):
//     the 32 lanes of a transpose read (4 k rows x 2 column halves x 32 bytes) hit 8 different
//     8-bank groups.
// Pipeline: STAGES LDS stages; the operand fragments of a 16-wide sub-step are read from LDS while
// the MFMAs of the sub-step before it run, and once per tile (before the first fragment read of
// tile t+1): wait for my loads of tile t+1 | barrier | issue tile t+STAGES-1, between MFMAs, into
// the stage that tile t-1 just left.
// The loads are inline assembly, invisible to the compiler's wait-count pass (told about them, it
// drains every load in flight before each LDS read); the waits are written by hand and rely on a
// fixed number of loads per step: past the last tile the last tile is fetched again.
// A K tail (K % BK != 0) is zeroed in LDS by the threads that fetched it, before the barrier.
#pragma once
#include "gemm_device.cuh"

namespace iex {

__device__ __forceinline__ void lds_dma16(const void* g, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_base_uniform) : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int WM, int WN, int WCN, int BK, int STAGES>
constexpr int gemm_dma_lds_bytes() {
  return STAGES * (2 * WM * 32 + WCN * WN * 32) * BK * 2;
}

constexpr int kXcds = 8;
constexpr int kGroupM = 4;

// Workgroup ids are dealt round-robin to the 8 XCDs (each with its own L2).  Give every
// XCD a contiguous band of C tiles (row-major over tiles) so that the A row panels a
// band needs are fetched into one L2 instead of eight.
__device__ __forceinline__ bool xcd_tile(int block, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + kXcds - 1) / kXcds;
  const int linear = (block % kXcds) * per_xcd + block / kXcds;
  if (linear >= total) return false;
  // inside the band, walk kGroupM tile rows column by column: the 32 tiles an XCD works on at one
  // time then share kGroupM row panels of A and 32 / kGroupM column panels of B in its L2
  const int per_group = kGroupM * tiles_n;
  const int first_row = (linear / per_group) * kGroupM;
  const int rows = min(tiles_m - first_row, kGroupM);
  const int in_group = linear % per_group;
  tile_m = first_row + in_group % rows;
  tile_n = in_group / rows;
  return true;
}

template <bool BF16, bool TRANS_B, int WM, int WN, int WCN, int BK, int STAGES, int SPLIT = 0>
__device__ __forceinline__ void gemm_tile_dma(const GemmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
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
      lds_dma16(a_row[q] + min(k0 + a_k8[q], last_k8), __builtin_amdgcn_readfirstlane(base + q * 1024));
    } else {
      const int qb = q - A_INSTR;
      const unsigned bbase = lds0 + stage * STAGE_BYTES + A_BYTES + wave * (B_INSTR * 1024);
      if constexpr (TRANS_B)
        lds_dma16(b_row[qb] + min(k0 + b_k8[qb], last_k8), __builtin_amdgcn_readfirstlane(bbase + qb * 1024));
      else
        lds_dma16(b_row[qb] + (size_t)min(k0 + b_k8[qb], p.K - 1) * p.N, __builtin_amdgcn_readfirstlane(bbase + qb * 1024));
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
  auto read_frags = [&](const unsigned char* st, int ks, int buf) {
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
        __syncthreads();
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
              issue_one(next, next % STAGES, q);
          }
      }
    }
  }
  wait_vmcnt<0>();  // the re-fetched last tiles: nothing may still be writing LDS when the workgroup ends

  const float* partial = nullptr;
  if constexpr (SPLIT == 1) {
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
  if constexpr (SPLIT == 2) {
    // split_parts workgroups hold partial sums of this tile (a stretch of K each).  Every one leaves its sums in the
    // workspace, waits until L2 has acknowledged them and draws a ticket; nobody waits for anybody.  The workgroup that
    // draws the last ticket finds all parts in L2 (the workgroups of a tile run on one XCD: the launcher's numbering),
    // adds them up in the order of the parts -- its own included, read back, so that the sum does not depend on who was
    // last -- and stores the tile.
    constexpr int NMT = WM * WN;
    const int parts = p.split_parts;
    const int tile_id = (z * p.tiles_m + tile_m) * p.tiles_n + tile_n;
    float* all = p.split_ws + (size_t)tile_id * parts * (BM * BN) + (size_t)wave * (NMT * 16 * 64) + lane * 4;
    float* mine = all + (size_t)p.split_part * (BM * BN);
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4 v = {acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
          *reinterpret_cast<f32x4*>(mine + ((i * WN + j) * 4 + q) * 256) = v;
        }
    wait_vmcnt<0>();   // (vmcnt counts a store until L2 has acknowledged it)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();   // everybody's sums are in L2, and everybody has read its last fragments: the stages are free
    if (tid == 0) *reinterpret_cast<int*>(smem) = atomicAdd(&p.split_flags[tile_id], 1);
    __syncthreads();
    if (*reinterpret_cast<volatile int*>(smem) != parts - 1) return;   // (uniform)
    // The other parts' sums come from L2: no workgroup of this launch has read a tile's parts before the tile's last
    // ticket is drawn, and that happens once, so no L1 holds a line of them (L1 starts empty at every launch).  Fences
    // stay at workgroup scope: a device-scope acquire here invalidates the XCD's L2 under every workgroup still
    // multiplying (measured: 4096 x 256 x 4096 21.8 -> 28.7 us), a device-scope release writes it back.
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int s = 0; s < parts; ++s) {
      const float* from = all + (size_t)s * (BM * BN);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(from + ((i * WN + j) * 4 + q) * 256);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[i][j][q * 4 + e] += v[e];
          }
    }
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
