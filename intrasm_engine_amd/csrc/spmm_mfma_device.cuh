// CSR SpMM on the matrix cores (gfx950, fp16 / bf16): the sparse operand is expanded to dense
// tiles in LDS on the fly and multiplied with v_mfma_f32_32x32x16.
//
// Why: the gather kernels move n * sizeof(T) bytes from L2 (or LDS) per nonzero and are bound
// by that gather bandwidth; the matrix cores of this part multiply a *dense* m x k block some
// ten times faster than the gather kernels process a 10 %-dense one.  So for moderately
// sparse operands (density from a few percent up) it is cheaper to treat zeros as zeros:
// HBM traffic stays that of CSR (the dense form of A exists only in LDS), the arithmetic
// runs at dense MFMA rate.
//
// Workgroup = 4 wavefronts (2 x 2), C tile = 128 rows (CSR rows in swizzled order) x 256
// columns, wave tile 64 x 128 = 2 x 4 MFMA tiles.  K is walked in chunks of 128 columns of A:
//   expansion   the workgroup zero-fills A_lds[128][128] and scatters the nonzeros of its rows
//               whose column lies in the chunk (column indices ascend inside a row, so these
//               are the next run after a per-row cursor).  A group of LPR lanes owns a row
//               and handles LPR nonzeros per pass; the next window of every row is loaded
//               right after the cursor moved, so it lands during the MFMA phase.
//   MFMA phase  4 steps of BK = 32: B (k x n, row-major) streams global -> registers -> LDS as
//               in the dense GEMM (3 register sets in flight, double-buffered LDS, transpose
//               reads ds_read_b64_tr_b16 form the operand), A fragments are 128-bit LDS reads.
// A_lds is single-buffered: two workgroups share a CU, so one expands while the other
// multiplies.  fp32 accumulation; deterministic; the epilogue scatters rows to
// row_indices[slot] and applies accumulate / bias / ReLU like the other SpMM kernels.
// Requirements (checked by the host): n % 8 == 0, 16-byte aligned dense operand and output.
#pragma once
#include "gemm_device.cuh"
#include "spmm_device.cuh"

namespace iex {

constexpr int kMfmaBM = 128;
constexpr int kMfmaBN = 256;
constexpr int kMfmaBKA = 128;                    // columns of A per expansion
constexpr int kMfmaLDA = kMfmaBKA + 8;           // LDS row stride of A, elements (272 bytes)
constexpr int kMfmaLDB = kMfmaBN + kGemmLdbPad;  // LDS row stride of B, elements
constexpr int kMfmaThreads = 256;
constexpr int kMfmaLdsBytes = (kMfmaBM * kMfmaLDA + 2 * kGemmBK * kMfmaLDB) * 2;

// The slice of B of one BK step that a thread carries from global memory to LDS.
struct SpmmMfmaBStage {
  static constexpr int CHUNKS = kMfmaBN * kGemmBK / 8 / kMfmaThreads;  // 128-bit chunks per thread
  typedef unsigned short u16;
  u32x4 rb[CHUNKS];
  __device__ __forceinline__ void load(const u16* __restrict__ B, int k, int n, int n0, int kt, int tid) {
    const int k0 = kt * kGemmBK;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int chunk = tid + c * kMfmaThreads;
      const int kr = chunk / (kMfmaBN / 8), nc = chunk % (kMfmaBN / 8);
      const int gk = k0 + kr, gn = n0 + nc * 8;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (gk < k && gn < n) v = *reinterpret_cast<const u32x4*>(B + (size_t)gk * n + gn);
      rb[c] = v;
    }
  }
  __device__ __forceinline__ void store(u16* b, int tid) const {
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int chunk = tid + c * kMfmaThreads;
      const int kr = chunk / (kMfmaBN / 8), nc = chunk % (kMfmaBN / 8);
      *reinterpret_cast<u32x4*>(b + kr * kMfmaLDB + nc * 8) = rb[c];
    }
  }
};

// Result of a wave (WM x WN MFMA tiles of 32 x 32, operands swapped) -> global memory, with
// the accumulate / bias / ReLU options; rows go to row_indices[slot].
template <bool BF16, int WM, int WN>
__device__ __forceinline__ void spmm_mfma_epilogue_direct(const SpmmParams& p, const f32x16 (&acc)[WM][WN],
                                                          unsigned short* __restrict__ C, int m0, int n0, int wm, int wn, int lane) {
  typedef unsigned short u16;
  // Swapped-operand result layout: lane holds row (lane % 32) of the 32x32 block and, in
  // accumulator quad q, columns q*8 + (lane / 32)*4 .. +3.  n % 8 == 0, so a quad is either
  // fully inside the matrix or fully outside.
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int slot = m0 + (wm * WM + i) * 32 + (lane & 31);
    if (slot >= p.m) continue;
    const int row = p.row_indices[slot];
    const float bias = p.bias ? p.bias[row] : 0.f;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int gn = n0 + (wn * WN + j) * 32 + q * 8 + (lane >> 5) * 4;
        if (gn >= p.n) continue;
        u16* dst = C + (size_t)row * p.n + gn;
        float x[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = acc[i][j][q * 4 + e];
        if (p.accumulate) {
          const u32x2 prev = *reinterpret_cast<const u32x2*>(dst);
          const unsigned w[2] = {prev.x, prev.y};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const u16 h = (u16)(w[e >> 1] >> ((e & 1) * 16));
            x[e] += BF16 ? __builtin_bit_cast(float, (unsigned)h << 16)
                         : (float)__builtin_bit_cast(_Float16, h);
          }
        }
        u16 h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float y = x[e] + bias;
          if (p.relu) y = fmaxf(y, 0.f);
          h[e] = f32_to_16(y, BF16);
        }
        u32x2 w;
        w.x = (unsigned)h[0] | ((unsigned)h[1] << 16);
        w.y = (unsigned)h[2] | ((unsigned)h[3] << 16);
        *reinterpret_cast<u32x2*>(dst) = w;
      }
    }
  }
}

// The same through LDS, as gemm_store_tile_lds does for the GEMM: every 32-row block of the wavefront's
// tile is laid out in the wavefront's own slice of LDS and read back 16 lanes per row, so a store
// instruction writes WN * 64 contiguous bytes of 64 / (WN * 4) output rows instead of 32 pieces of 16
// bytes (output rate of these kernels 1.2 -> 3 TB/s).  Rows still go where row_indices sends them.
// No accumulation; 16-byte aligned C; `lds`: gemm_store_lds_bytes<WN>() bytes that only this wavefront touches.
template <bool BF16, int WM, int WN>
__device__ __forceinline__ void spmm_mfma_epilogue_lds(const SpmmParams& p, const f32x16 (&acc)[WM][WN],
                                                       unsigned short* __restrict__ C, int m0, int n0, int wm, int wn, int lane,
                                                       unsigned char* lds) {
  typedef unsigned short u16;
  constexpr int ROWB = WN * 64 + 16, CPR = WN * 4, RPI = kWave / CPR;
  static_assert(kWave % CPR == 0 && 32 % RPI == 0, "whole rows per instruction");
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int slot0 = m0 + (wm * WM + i) * 32;
    if (slot0 >= p.m) break;  // (uniform)
    const float bias = p.bias ? p.bias[p.row_indices[min(slot0 + (lane & 31), p.m - 1)]] : 0.f;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        u16 h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float y = acc[i][j][q * 4 + e] + bias;
          if (p.relu) y = fmaxf(y, 0.f);
          h[e] = f32_to_16(y, BF16);
        }
        u32x2 w;
        w.x = (unsigned)h[0] | ((unsigned)h[1] << 16);
        w.y = (unsigned)h[2] | ((unsigned)h[3] << 16);
        *reinterpret_cast<u32x2*>(lds + (lane & 31) * ROWB + (j * 32 + q * 8 + (lane >> 5) * 4) * 2) = w;
      }
    }
    const int chunk = lane % CPR;
    const int gn = n0 + wn * WN * 32 + chunk * 8;
#pragma unroll
    for (int t = 0; t < 32 / RPI; ++t) {
      const int r = t * RPI + lane / CPR;
      const u32x4 v = *reinterpret_cast<const u32x4*>(lds + r * ROWB + chunk * 16);
      if (slot0 + r < p.m && gn < p.n) {
        const int row = p.row_indices[slot0 + r];
        u16* dst = C + (size_t)row * p.n + gn;
        if (p.stream_out) {
          asm volatile("" : "+v"(dst));  // (or the compiler merges this store with the plain one and drops the hint)
          __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));
        } else {
          *reinterpret_cast<u32x4*>(dst) = v;
        }
      }
    }
  }
}

// Every thread of the workgroup must call this (it may contain a barrier); `smem` = the workgroup's LDS,
// free from here on, at least waves * gemm_store_lds_bytes<WN>() bytes.
template <bool BF16, int WM, int WN>
__device__ __forceinline__ void spmm_mfma_epilogue(const SpmmParams& p, const f32x16 (&acc)[WM][WN],
                                                   unsigned short* __restrict__ C, int m0, int n0, int wm, int wn, int lane,
                                                   unsigned char* smem) {
  if (!p.accumulate && (reinterpret_cast<uintptr_t>(C) & 15) == 0) {
    __syncthreads();  // everybody has read its last operands
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    spmm_mfma_epilogue_lds<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, smem + wave * gemm_store_lds_bytes<WN>());
  } else {
    spmm_mfma_epilogue_direct<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane);
  }
}

template <bool BF16, typename IT, int LPR>
__device__ __forceinline__ void spmm_mfma_block(const SpmmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = kMfmaBM, BN = kMfmaBN, BK = kGemmBK, BKA = kMfmaBKA, LDA = kMfmaLDA, LDB = kMfmaLDB;
  constexpr int WM = 2, WN = 4;
  constexpr int SETS = kGemmSets;
  constexpr int GROUPS = kMfmaThreads / LPR;  // row groups per workgroup
  constexpr int R = BM / GROUPS;              // rows per group
  constexpr int kNoCol = 0x7fffffff;
  constexpr unsigned long long kGroupMask = LPR == 64 ? ~0ull : ((1ull << (LPR & 63)) - 1ull);
  typedef unsigned short u16;

  u16* sA = reinterpret_cast<u16*>(smem);  // [BM][LDA]
  u16* sB = sA + BM * LDA;                 // [2][BK][LDB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const u16* __restrict__ values = static_cast<const u16*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
  const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
  const u16* __restrict__ B = static_cast<const u16*>(p.dense) + (size_t)z * p.k * p.n;
  u16* __restrict__ C = static_cast<u16*>(p.out) + (size_t)z * p.m * p.n;

  // ---- expansion state: group g = tid / LPR owns local rows g, g + GROUPS, ... -------------
  const int sub = tid % LPR;
  const int group = tid / LPR;
  const int gshift = lane & ~(LPR - 1);
  int pos[R], end[R], wc[R];
  u16 wv[R];
  auto load_window = [&](int j) {
    const int idx = pos[j] + sub;
    wc[j] = kNoCol;
    wv[j] = 0;
    if (idx < end[j]) {
      wc[j] = (int)cols[idx];
      wv[j] = values[idx];
    }
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
    load_window(j);
  }

  auto expand = [&](int ka0) {
    const int kend = ka0 + BKA;
    // zero the rows of this group (same wavefront as the scatter below: LDS keeps the order)
#pragma unroll
    for (int j = 0; j < R; ++j) {
      u16* rowp = sA + (group + j * GROUPS) * LDA;
      constexpr int kRowVecs = BKA / 8;  // 128-bit stores per row
#pragma unroll
      for (int q = 0; q < (kRowVecs + LPR - 1) / LPR; ++q) {
        const int v = q * LPR + sub;
        if (kRowVecs % LPR == 0 || v < kRowVecs) *reinterpret_cast<u32x4*>(rowp + v * 8) = u32x4{0u, 0u, 0u, 0u};
      }
    }
    bool again = false;
    bool full[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
      const bool in = wc[j] < kend;
      if (in) sA[(group + j * GROUPS) * LDA + (wc[j] - ka0)] = wv[j];
      const unsigned long long b = __ballot(in);
      const int cnt = __popcll((b >> gshift) & kGroupMask);
      pos[j] += cnt;
      full[j] = cnt == LPR;
      again |= full[j];
    }
    // rows with more than LPR nonzeros in this chunk: keep going (loads are exposed here)
    while (__any(again)) {
      again = false;
#pragma unroll
      for (int j = 0; j < R; ++j) {
        int c = kNoCol;
        u16 v = 0;
        const int idx = pos[j] + sub;
        if (full[j] && idx < end[j]) {
          c = (int)cols[idx];
          v = values[idx];
        }
        const bool in = c < kend;
        if (in) sA[(group + j * GROUPS) * LDA + (c - ka0)] = v;
        const unsigned long long b = __ballot(in);
        const int cnt = __popcll((b >> gshift) & kGroupMask);
        pos[j] += cnt;
        full[j] = cnt == LPR;
        again |= full[j];
      }
    }
    // the window of the next chunk starts at the cursor; it lands during the MFMA phase
#pragma unroll
    for (int j = 0; j < R; ++j) load_window(j);
  };

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  SpmmMfmaBStage regs[SETS];
  const int KT = (p.k + BK - 1) / BK;
#pragma unroll
  for (int s = 0; s < SETS; ++s)
    if (s < KT) regs[s].load(B, p.k, p.n, n0, s, tid);
  regs[0].store(sB, tid);
  if (SETS < KT) regs[0].load(B, p.k, p.n, n0, SETS, tid);
  // (the barrier after the first expansion also publishes B tile 0)

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;

  auto step = [&](int kt, auto phase) {
    constexpr int PH = decltype(phase)::value;
    constexpr int buf = PH & 1;
    constexpr int set = (PH + 1) % SETS;
    if ((kt & (BKA / BK - 1)) == 0) {
      expand(kt * BK);
      __syncthreads();
    }
    const u16* a = sA + (wm * WM * 32 + frag_row) * LDA + (kt & (BKA / BK - 1)) * BK + frag_k;
    const u16* b = sB + buf * BK * LDB + ((lane >> 5) * 8 + ((lane & 15) >> 2)) * LDB + wn * WN * 32 +
                   ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      u32x4 fa[WM], fb[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i) fa[i] = *reinterpret_cast<const u32x4*>(a + i * 32 * LDA + ks * 16);
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
        const u16* q0 = b + (ks * 16) * LDB + j * 32;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0 + 4 * LDB));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        fb[j] = u32x4{l2.x, l2.y, h2.x, h2.y};
      }
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) acc[i][j] = mfma_32x32x16<BF16>(fb[j], fa[i], acc[i][j]);
    }
    if (kt + 1 < KT) {
      regs[set].store(sB + (buf ^ 1) * BK * LDB, tid);
      if (kt + 1 + SETS < KT) regs[set].load(B, p.k, p.n, n0, kt + 1 + SETS, tid);
    }
    __syncthreads();
  };

  static_assert(SETS == 3, "the step loop below is unrolled for 3 register sets (period 6)");
  int kt = 0;
  for (; kt + 6 <= KT; kt += 6) {
    step(kt + 0, std::integral_constant<int, 0>{});
    step(kt + 1, std::integral_constant<int, 1>{});
    step(kt + 2, std::integral_constant<int, 2>{});
    step(kt + 3, std::integral_constant<int, 3>{});
    step(kt + 4, std::integral_constant<int, 4>{});
    step(kt + 5, std::integral_constant<int, 5>{});
  }
  if (kt < KT) step(kt++, std::integral_constant<int, 0>{});
  if (kt < KT) step(kt++, std::integral_constant<int, 1>{});
  if (kt < KT) step(kt++, std::integral_constant<int, 2>{});
  if (kt < KT) step(kt++, std::integral_constant<int, 3>{});
  if (kt < KT) step(kt++, std::integral_constant<int, 4>{});

  spmm_mfma_epilogue<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, smem);
}

}  // namespace iex
