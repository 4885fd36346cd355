// CSR SpMM on the matrix cores, second arrangement: 8 wavefronts (2 x 4), C tile 128 x 512,
// the expanded A chunk double-buffered in LDS so that the expansion of chunk c+1 is spread
// over the four MFMA steps of chunk c (one row per lane group and step) and runs in the
// shadow of the matrix cores.  See spmm_mfma_device.cuh for the idea.
//
// Expansion state per lane group (16 lanes own 4 rows): cursor, row end and W windows of 16
// nonzeros each, packed (column << 16 | 16-bit value) so that one unsigned compare against
// (chunk end << 16) tells whether a nonzero belongs to the chunk.  After a row-visit the
// windows are reloaded at the new cursor; they land during the next four steps.
// BKA = columns of A per chunk.  With 128 (what the library launches) a row-visit happens once
// per four steps and W windows may not hold a dense row's run: a loop with exposed loads picks up
// the rest, and because of that loop the compiler drains every load in flight at each wait.
// 64 with W = 4 always holds the whole run and needs no loop, but doubles the row-visits and
// spills 150 bytes: measured 2-2.6x slower, so it is not instantiated.
// Requirements (checked by the host): n % 8 == 0, 16-byte aligned dense operand and output,
// k < 65535 (packed columns), ascending column indices without duplicates inside a row.
#pragma once
#include "spmm_mfma_device.cuh"

namespace iex {

constexpr int kMfma2BN = 512;
constexpr int kMfma2LDB = kMfma2BN + kGemmLdbPad;
constexpr int kMfma2Threads = 512;
template <int BKA>
constexpr int spmm_mfma2_lds_bytes() { return (2 * kMfmaBM * (BKA + 8) + 2 * kGemmBK * kMfma2LDB) * 2; }

struct SpmmMfma2BStage {
  static constexpr int CHUNKS = kMfma2BN * kGemmBK / 8 / kMfma2Threads;  // 128-bit chunks per thread
  typedef unsigned short u16;
  u32x4 rb[CHUNKS];
  __device__ __forceinline__ void load(const u16* __restrict__ B, int k, int n, int n0, int kt, int tid) {
    const int k0 = kt * kGemmBK;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int chunk = tid + c * kMfma2Threads;
      const int kr = chunk / (kMfma2BN / 8), nc = chunk % (kMfma2BN / 8);
      const int gk = k0 + kr, gn = n0 + nc * 8;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (gk < k && gn < n) v = *reinterpret_cast<const u32x4*>(B + (size_t)gk * n + gn);
      rb[c] = v;
    }
  }
  __device__ __forceinline__ void store(u16* b, int tid) const {
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int chunk = tid + c * kMfma2Threads;
      const int kr = chunk / (kMfma2BN / 8), nc = chunk % (kMfma2BN / 8);
      *reinterpret_cast<u32x4*>(b + kr * kMfma2LDB + nc * 8) = rb[c];
    }
  }
};

template <bool BF16, typename IT, int W, int BKA>
__device__ __forceinline__ void spmm_mfma2_block(const SpmmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = kMfmaBM, BN = kMfma2BN, BK = kGemmBK, LDA = BKA + 8, LDB = kMfma2LDB;
  constexpr int WM = 2, WN = 4;
  constexpr int LPR = 16;
  constexpr int GROUPS = kMfma2Threads / LPR;  // 32 lane groups
  constexpr int R = BM / GROUPS;               // 4 rows per group
  constexpr int SPC = BKA / BK;                // steps per chunk (4 or 2)
  constexpr int RPS = R / SPC;                 // rows a lane group expands per step (1 or 2)
  static_assert(BKA == 128 || BKA == 64, "chunk width");
  static_assert(BK / 16 >= RPS, "one row-visit per 16-wide MFMA sub-step at most");
  constexpr unsigned kNone = 0xffffffffu;
  typedef unsigned short u16;

  u16* sA = reinterpret_cast<u16*>(smem);  // [2][BM][LDA]
  u16* sB = sA + 2 * BM * LDA;             // [2][BK][LDB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const u16* __restrict__ values = static_cast<const u16*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
  const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
  const u16* __restrict__ B = static_cast<const u16*>(p.dense) + (size_t)z * p.k * p.n;
  u16* __restrict__ C = static_cast<u16*>(p.out) + (size_t)z * p.m * p.n;

  const int sub = tid % LPR;
  const int group = tid / LPR;
  const int gshift = lane & ~(LPR - 1);
  int pos[R], end[R];
  // A window entry is the pair (value, column) as two 16-bit halves of one register, filled by
  // two 16-bit loads with a clamped index and no arithmetic on the result: nothing here waits
  // for the loads, so they overlap the MFMAs.  Whether the entry belongs to the row (index
  // below the row end) is decided when it is used.  The host guarantees nnz > 0.
  u16 wval[R][W];
  IT wcol[R][W];
  const int last_nz = p.nnz - 1;
  auto load_windows = [&](int j) {
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const int safe = min(pos[j] + w * LPR + sub, last_nz);
      wval[j][w] = values[safe];
      wcol[j][w] = cols[safe];
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
    load_windows(j);
  }

  // Row j of this lane group, columns [ka0, ka0 + BKA) -> abuf.  The zero fill and the scatter
  // come from the same wavefront, and LDS keeps the order of a wavefront's accesses.
  auto expand_row = [&](int j, int ka0, u16* abuf) {
    u16* rowp = abuf + (group + j * GROUPS) * LDA;
    if constexpr (BKA == 128) *reinterpret_cast<u32x4*>(rowp + sub * 8) = u32x4{0u, 0u, 0u, 0u};
    else *reinterpret_cast<u32x2*>(rowp + sub * 4) = u32x2{0u, 0u};
    const int kend = ka0 + BKA;
    const unsigned lim = (unsigned)kend << 16;
    int consumed = 0;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const int c = (int)wcol[j][w];
      const bool in = pos[j] + w * LPR + sub < end[j] && c < kend;
      if (in) rowp[c - ka0] = wval[j][w];
      consumed += __popcll((__ballot(in) >> gshift) & 0xffffull);
    }
    pos[j] += consumed;
    if constexpr (W * LPR < BKA) {
      bool more = consumed == W * LPR;
      // A run longer than the windows held in registers: the loads of these passes are exposed.
      // (Unrolling this loop into forward branches, so that the compiler could keep counting the
      // loads in flight across it, was measured: the extra register pressure costs far more.)
      while (__any(more)) {
        unsigned e = kNone;
        const int idx = pos[j] + sub;
        if (more && idx < end[j]) e = ((unsigned)(u16)cols[idx] << 16) | (unsigned)values[idx];
        const bool in = e < lim;
        if (in) rowp[(int)(e >> 16) - ka0] = (u16)e;
        const int cnt = __popcll((__ballot(in) >> gshift) & 0xffffull);
        pos[j] += cnt;
        more = cnt == LPR;
      }
    }
    load_windows(j);
  };

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  SpmmMfma2BStage regs[2];  // regs[t % 2] carries B tile t
  const int KT = (p.k + BK - 1) / BK;
  regs[0].load(B, p.k, p.n, n0, 0, tid);
  if (1 < KT) regs[1].load(B, p.k, p.n, n0, 1, tid);
#pragma unroll
  for (int j = 0; j < R; ++j) expand_row(j, 0, sA);
  regs[0].store(sB, tid);
  if (2 < KT) regs[0].load(B, p.k, p.n, n0, 2, tid);
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;

  // One BK step; J = kt % 4 is static (row of the lane groups to expand, LDS buffer and
  // register set of B alternate with its parity).
  auto step = [&](int kt, auto jc) {
    constexpr int J = decltype(jc)::value;
    constexpr int buf = J & 1;
    constexpr int set = (J + 1) & 1;
    const int chunk = kt / SPC;
    const u16* a = sA + (chunk & 1) * BM * LDA + (wm * WM * 32 + frag_row) * LDA + (J % SPC) * BK + frag_k;
    const u16* b = sB + buf * BK * LDB + ((lane >> 5) * 8 + ((lane & 15) >> 2)) * LDB + wn * WN * 32 +
                   ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    const bool next_chunk = (chunk + 1) * BKA < p.k;
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
      if (ks < RPS && next_chunk) expand_row((J % SPC) * RPS + ks, (chunk + 1) * BKA, sA + ((chunk + 1) & 1) * BM * LDA);
    }
    if (kt + 1 < KT) {
      regs[set].store(sB + (buf ^ 1) * BK * LDB, tid);
      if (kt + 3 < KT) regs[set].load(B, p.k, p.n, n0, kt + 3, tid);
    }
    __syncthreads();
  };

  int kt = 0;
  for (; kt + 4 <= KT; kt += 4) {
    step(kt + 0, std::integral_constant<int, 0>{});
    step(kt + 1, std::integral_constant<int, 1>{});
    step(kt + 2, std::integral_constant<int, 2>{});
    step(kt + 3, std::integral_constant<int, 3>{});
  }
  if (kt < KT) step(kt++, std::integral_constant<int, 0>{});
  if (kt < KT) step(kt++, std::integral_constant<int, 1>{});
  if (kt < KT) step(kt++, std::integral_constant<int, 2>{});

  spmm_mfma_epilogue<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane);
}

}  // namespace iex
