// CSR SpMM on the matrix cores, second arrangement: 8 wavefronts (2 x 4), C tile 128 x 512,
// the expanded A chunk double-buffered in LDS so that the expansion of chunk c+1 is spread
// over the four MFMA steps of chunk c (one row per lane group and step) and runs in the
// shadow of the matrix cores.  See spmm_mfma_device.cuh for the idea.
//
// Expansion state per lane group (16 lanes own 4 rows): cursor, row end and W windows of 16
// nonzeros each (value and column, as loaded).  After a row-visit the windows are reloaded at
// the new cursor; they land during the next four steps.
// BKA = columns of A per chunk (128: a row-visit once per four steps).  W windows may not hold a
// dense row's run inside a chunk.  Then the workgroup multiplies the same chunk once more with
// what the windows left behind (the products add up to the same sum), instead of a loop over
// exposed loads inside the row-visit: every load of the main loop is unconditional and outside
// any inner loop, so the compiler counts the loads in flight and each wait names exactly the
// ones it needs.  The host picks W so that such a second pass is rare (W * 16 above the mean
// run by a margin); a matrix with a few much denser rows pays one extra pass per chunk they touch.
// Requirements (checked by the host): n % 8 == 0, 16-byte aligned dense operand and output,
// k < 65535 (packed columns), ascending column indices without duplicates inside a row.
#pragma once
#include "spmm_mfma_device.cuh"

namespace iex {

constexpr int kMfma2BN = 512;
constexpr int kMfma2LDB = kMfma2BN + kGemmLdbPad;
constexpr int kMfma2Threads = 512;
template <int BKA>
constexpr int spmm_mfma2_lds_bytes() { return (2 * kMfmaBM * (BKA + 8) + 2 * kGemmBK * kMfma2LDB) * 2 + 16 + kMfma2Threads * 4; }

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
      // unconditional, clamped into the matrix: a guarded load is a branch, and behind a branch the
      // compiler waits for every load in flight wherever one is needed.  A k row beyond the matrix
      // meets zeros of A, a column beyond n feeds columns of C that are never stored.
      const int gk = min(k0 + kr, k - 1), gn = min(n0 + nc * 8, n - 8);
      rb[c] = *reinterpret_cast<const u32x4*>(B + (size_t)gk * n + gn);
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
  static_assert(BKA == 128 && R == SPC, "one row of every lane group is expanded per step");
  typedef unsigned short u16;

  u16* sA = reinterpret_cast<u16*>(smem);  // [2][BM][LDA]
  u16* sB = sA + 2 * BM * LDA;             // [2][BK][LDB]
  int* again = reinterpret_cast<int*>(sB + 2 * BK * LDB);  // [2], one per A buffer
  // One word per lane that absorbs the writes of lanes with nothing to write: a predicated store is
  // a branch around it, and branches cut the step into blocks across which the compiler cannot
  // interleave the expansion with the MFMAs.
  int* sink = again + 4 + threadIdx.x;

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
  // come from the same wavefront, and LDS keeps the order of a wavefront's accesses.  A run that
  // fills every window may continue beyond them: the row raises *again, and the workgroup gives
  // the same chunk another pass with what is left (no loop over loads here: inside one, the
  // compiler could no longer count the loads in flight and would drain them all at every wait).
  auto expand_row = [&](int j, int ka0, u16* abuf, int* again) {
    u16* rowp = abuf + (group + j * GROUPS) * LDA;
    *reinterpret_cast<u32x4*>(rowp + sub * 8) = u32x4{0u, 0u, 0u, 0u};
    const int kend = ka0 + BKA;
    int consumed = 0;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      const int c = (int)wcol[j][w];
      const bool in = pos[j] + w * LPR + sub < end[j] && c < kend;
      if constexpr (W < 5) {
        *(in ? rowp + (c - ka0) : reinterpret_cast<u16*>(sink)) = wval[j][w];
      } else {  // five windows: the unpredicated form keeps more registers live and spills
        if (in) rowp[c - ka0] = wval[j][w];
      }
      consumed += __popcll((__ballot(in) >> gshift) & 0xffffull);
    }
    pos[j] += consumed;
    *(consumed == W * LPR ? again : sink) = 1;
    load_windows(j);
  };

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  if (tid < 2) again[tid] = 0;
  __syncthreads();
  SpmmMfma2BStage regs[2];  // regs[s % 2] carries the B tile of step s
  const int chunks = (p.k + BKA - 1) / BKA;
  regs[0].load(B, p.k, p.n, n0, 0, tid);
  regs[1].load(B, p.k, p.n, n0, 1, tid);
#pragma unroll
  for (int j = 0; j < R; ++j) expand_row(j, 0, sA, again);
  regs[0].store(sB, tid);
  regs[0].load(B, p.k, p.n, n0, 2, tid);
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;

  // Step J of a pass: multiply B tile J of chunk `cur` (LDS buffer J % 2) with columns
  // [J * BK, J * BK + BK) of the expanded chunk in A buffer `ab`; expand row J of every lane group
  // for chunk `nxt` into the other A buffer; hand the B tile of the next step to LDS and request
  // the one three steps ahead (`ahead`; beyond the matrix it is clamped and meets zeros of A).
  auto step = [&](int ab, int nxt, int ahead, auto jc) {
    constexpr int J = decltype(jc)::value;
    constexpr int buf = J & 1;
    constexpr int set = (J + 1) & 1;
    const u16* a = sA + ab * BM * LDA + (wm * WM * 32 + frag_row) * LDA + J * BK + frag_k;
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
      if (ks == 0) expand_row(J, nxt * BKA, sA + (ab ^ 1) * BM * LDA, again + (ab ^ 1));
    }
    if (J == 1 && tid == 0) again[ab] = 0;  // read before this pass, raised again in the next one
    regs[set].store(sB + (buf ^ 1) * BK * LDB, tid);
    regs[set].load(B, p.k, p.n, n0, ahead, tid);
    __syncthreads();
  };

  int cur = 0, ab = 0;
  bool repeat = __builtin_amdgcn_readfirstlane(again[0]) != 0;
  while (cur < chunks) {
    const int nxt = repeat ? cur : cur + 1;
    step(ab, nxt, cur * SPC + 3, std::integral_constant<int, 0>{});
    step(ab, nxt, nxt * SPC + 0, std::integral_constant<int, 1>{});
    step(ab, nxt, nxt * SPC + 1, std::integral_constant<int, 2>{});
    step(ab, nxt, nxt * SPC + 2, std::integral_constant<int, 3>{});
    ab ^= 1;
    repeat = __builtin_amdgcn_readfirstlane(again[ab]) != 0;
    cur = nxt;
  }

  spmm_mfma_epilogue<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane, smem);
}

}  // namespace iex
