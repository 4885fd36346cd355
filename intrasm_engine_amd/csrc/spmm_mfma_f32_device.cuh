// CSR SpMM in fp32 on the matrix cores (gfx950, v_mfma_f32_32x32x2_f32 or 16x16x4_f32).  The
// sparse operand is expanded to dense MT x 128 blocks in LDS (MT = 32 or 16 rows, the MFMA
// tile height) and multiplied at the dense fp32 MFMA rate (64 FMA-flops per clock and SIMD),
// which beats the gather kernels from roughly 25 % density up: those move n * 4 bytes from L2
// per nonzero.  (The text below says 32 rows and 8 k rows per group; with MT = 16 read 16 rows
// and 16 k rows per group: a wave then has four k slots of 16 lanes instead of two of 32.)
//
// Workgroup = 4 multiplying wavefronts, C tile = MT rows (CSR rows in swizzled order) x BN columns.
//   A   chunks of 128 columns, double-buffered [32][132] floats in LDS.  A group of 8 lanes
//       owns one row: cursor, row end and W windows of 8 nonzeros in registers; chunk c+1 is
//       expanded before the MFMAs of chunk c are issued and the windows are reloaded right
//       after, so those loads land during the MFMAs.  One barrier per chunk.
//   B   (k x n row-major) never touches LDS: with a 32-row tile every element of B feeds
//       exactly one MFMA of the workgroup, and the MFMA operand layout (lane = column, half
//       wave = k) is a coalesced global load already.  A lane loads NJ adjacent columns
//       (NJ*4 bytes) of one k row; element j feeds MFMA j, whose 32 "columns" are therefore
//       the strided set {NJ*i + j}.  At the end a lane holds NJ adjacent columns per
//       accumulator slot and stores them with one NJ*4-byte store.
//   k   a wave covers 32 x 32*NJ columns; the BN / (32*NJ) waves along n times WAVES_K waves
//       along k make up the workgroup.  The k slices interleave by groups of 8 k rows (one
//       128-bit LDS read of A per lane and group: lanes 0-31 take k .. k+3, lanes 32-63
//       k+4 .. k+7, the B loads follow the same assignment); partial tiles are added through
//       LDS at the end in a fixed order (deterministic).
// Loads of B run four groups (4 x 4 loads per lane) ahead of the MFMAs.
// SPLIT: the workgroup has 8 wavefronts with two roles.  Waves 0-3 only multiply, waves 4-7
// only expand the next chunk; one of each shares a SIMD, so the vector-ALU work of the
// expansion runs beside the other wave's MFMAs instead of in front of them, and the
// multiplying waves carry no loop around loads (the compiler can then count their loads in
// flight exactly).  Without SPLIT all 4 waves do both, one after the other.
// Requirements (checked by the host): n % 4 == 0, 16-byte aligned dense operand and output,
// strictly ascending column indices inside a row.
#pragma once
#include "spmm_device.cuh"

namespace iex {

typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// columns of A per chunk: at most 128 nonzeros of a row fall into one, which 16 windows of 8 hold
template <int MT>
constexpr int spmm_mfma_f32_bka() { return 128; }
constexpr int kF32Threads = 256;       // per role

template <int MT, int NJ, int WAVES_N>
constexpr int spmm_mfma_f32_lds_bytes() {
  constexpr int a_bytes = 2 * MT * (spmm_mfma_f32_bka<MT>() + 4) * 4;
  constexpr int red_bytes = (4 / WAVES_N - 1) * WAVES_N * NJ * (MT * MT / 64) * 64 * 4;  // partial tiles of the k slices
  return a_bytes > red_bytes ? a_bytes : red_bytes;
}

template <int NJ>
struct F32Frag {
  float v[NJ];
};

template <int MT, int NJ, int WAVES_N, int W, bool SPLIT>
__device__ __forceinline__ void spmm_mfma_f32_block(const SpmmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = MT, BKA = spmm_mfma_f32_bka<MT>();
  constexpr int LDA = BKA + 4;            // floats: 16 consecutive rows start in distinct 4-bank groups
  constexpr int KSLOTS = 64 / MT;         // k rows one MFMA consumes = lane groups of MT lanes (2 or 4)
  constexpr int GK = 4 * KSLOTS;          // k rows of a group (one 128-bit A read per lane = 4 MFMA steps)
  constexpr int ACC = MT * MT / 64;       // accumulator registers of one MFMA tile (16 or 4)
  constexpr int WAVES_K = 4 / WAVES_N;
  constexpr int WCOLS = MT * NJ;          // columns of a wave
  constexpr int BN = WCOLS * WAVES_N;     // columns of the workgroup
  constexpr int GROUPS = BKA / GK;        // groups per chunk (16 or 8)
  constexpr int GPW = GROUPS / WAVES_K;   // groups per wave and chunk
  constexpr int LPR = 8;                  // lanes per row of the expansion
  constexpr int EXP_THREADS = MT * LPR;   // threads that expand (256 or 128)
  typedef float acc_t __attribute__((ext_vector_type(ACC)));
  static_assert(MT == 32 || MT == 16, "MFMA tile height");
  constexpr int AHEAD = GPW < 4 ? GPW : 4;  // groups of B loads in flight
  constexpr int kNoCol = 0x7fffffff;
  static_assert(NJ == 2 || NJ == 4, "a lane loads 2 or 4 adjacent columns");
  static_assert(GPW % AHEAD == 0, "the prefetch ring is unrolled over the groups of a chunk");

  float* sA = reinterpret_cast<float*>(smem);  // [2][BM][LDA]

  const int lane = threadIdx.x & 63;
  const bool is_mma = threadIdx.x < kF32Threads;                                   // wave-uniform roles
  const bool is_exp = SPLIT ? threadIdx.x >= kF32Threads : threadIdx.x < EXP_THREADS;
  const int tid = threadIdx.x % kF32Threads;                // index inside the role
  const int wave = tid >> 6;
  const int wn = wave % WAVES_N, wk = wave / WAVES_N;
  const int half = lane / MT;  // k slot: which 4 of the GK k rows of a group this lane feeds
  const int l32 = lane % MT;   // row (A fragment) / column slot (B fragment) of this lane
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const float* __restrict__ values = static_cast<const float*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
  const int* __restrict__ cols = static_cast<const int*>(p.cols);
  const float* __restrict__ B = static_cast<const float*>(p.dense) + (size_t)z * p.k * p.n;
  float* __restrict__ C = static_cast<float*>(p.out) + (size_t)z * p.m * p.n;

  // ---- expansion: lane group tid / 8 owns local row tid / 8 -------------------------------
  const int sub = tid % LPR;
  const int erow = tid / LPR;
  const int gshift = lane & ~(LPR - 1);
  int pos = 0, end = 0;
  if (is_exp) {
    const int slot = m0 + erow;
    if (slot < p.m) {
      const int row = p.row_indices[slot];
      pos = p.row_offsets[row];
      end = p.row_offsets[row + 1];
    }
  }
  // W register windows of 8 nonzeros per row; the first wcnt of them are used (wave-uniform:
  // enough for 1.3 x the run a row of this wave would have per chunk if its nonzeros were
  // spread evenly, plus one).  A denser stretch than that falls back to the loop in expand().
  int wc[W];
  float wv[W];
  int wcnt = W;
  if (W > 8) {
    int need = (int)(((long long)(end - pos) * BKA * 13 / 10 / (p.k > 0 ? p.k : 1) + LPR - 1) / LPR) + 1;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) need = max(need, __shfl_xor(need, o));
    wcnt = min(W, need);
  }
  // (loads are unconditional with a clamped index and no arithmetic on the result: no branches
  // and no wait at the load, so they overlap the MFMAs; the host guarantees nnz > 0)
  const int last_nz = p.nnz - 1;
  auto load_windows = [&]() {
#pragma unroll
    for (int w = 0; w < W; ++w) {
      if (w >= wcnt) break;  // wave-uniform
      const int idx = pos + w * LPR + sub;
      const int safe = min(idx, last_nz);
      wc[w] = cols[safe];   // raw: whether idx < end is decided at use, so that nothing
      wv[w] = values[safe]; // here waits for the loads
    }
  };
  if (is_exp) load_windows();
  // Columns [ka0, ka0 + BKA) of the row -> abuf.  Zero fill and scatter come from the same
  // wavefront, and LDS keeps the order of a wavefront's accesses.
  auto expand = [&](int ka0, float* abuf) {
    float* rowp = abuf + erow * LDA;
#pragma unroll
    for (int q = 0; q < BKA / 4 / LPR; ++q) *reinterpret_cast<f32x4_t*>(rowp + (q * LPR + sub) * 4) = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int kend = ka0 + BKA;
    int consumed = 0;
#pragma unroll
    for (int w = 0; w < W; ++w) {
      if (w >= wcnt) break;  // wave-uniform
      const bool in = pos + w * LPR + sub < end && wc[w] < kend;
      if (in) rowp[wc[w] - ka0] = wv[w];
      consumed += __popcll((__ballot(in) >> gshift) & 0xffull);
    }
    pos += consumed;
    // every window consumed: the run may go on -- unless the windows already span a whole chunk
    bool more = consumed == wcnt * LPR && wcnt * LPR < BKA;
    while (__any(more)) {  // a run longer than the windows held in registers: loads are exposed here
      int c = kNoCol;
      float v = 0.f;
      const int idx = pos + sub;
      if (more && idx < end) {
        c = cols[idx];
        v = values[idx];
      }
      const bool in = c < kend;
      if (in) rowp[c - ka0] = v;
      const int cnt = __popcll((__ballot(in) >> gshift) & 0xffull);
      pos += cnt;
      more = cnt == LPR;
    }
    load_windows();
  };

  // ---- B: the 4 k rows of group g (chunk-relative) that this lane feeds ----------------------
  const int col = n0 + wn * WCOLS + l32 * NJ;  // first of the NJ columns of this lane
  const bool col_ok = col < p.n;               // n % 4 == 0: the NJ columns are in or out together
  // Loads are clamped to valid addresses instead of masked: a k row beyond the matrix meets
  // zeros of A, a column beyond n is computed and never stored.
  const float* __restrict__ bsafe = B + (col_ok ? col : 0);
  const int last_k = p.k - 1;
  auto load_b = [&](F32Frag<NJ> (&f)[4], int kbase) {  // kbase = first k row of the group
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float* src = bsafe + (size_t)min(kbase + half * 4 + i, last_k) * p.n;
      if constexpr (NJ == 4) {
        const f32x4_t v = *reinterpret_cast<const f32x4_t*>(src);
#pragma unroll
        for (int j = 0; j < 4; ++j) f[i].v[j] = v[j];
      } else {
        const float2 v = *reinterpret_cast<const float2*>(src);
        f[i].v[0] = v.x;
        f[i].v[1] = v.y;
      }
    }
  };

  acc_t acc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int r = 0; r < ACC; ++r) acc[j][r] = 0.f;

  // group index of this wave, global over chunks: gi -> k row (gi / GPW) * BKA + ((gi % GPW) * WAVES_K + wk) * 8
  auto group_k = [&](int gi) { return (gi / GPW) * BKA + ((gi % GPW) * WAVES_K + wk) * GK; };
  const int n_chunks = (p.k + BKA - 1) / BKA;

  F32Frag<NJ> ring[AHEAD][4];
  if (is_mma) {
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) load_b(ring[a], group_k(a));
  }
  if (is_exp) expand(0, sA);
  __syncthreads();

  // The scheduling barriers pin the order "MFMAs of group g, then the loads that refill its
  // ring slot": left alone, the compiler sinks all loads of a chunk behind its last MFMA and
  // the next chunk starts by waiting for them.
  for (int c = 0; c < n_chunks; ++c) {
    if (is_exp && c + 1 < n_chunks) expand((c + 1) * BKA, sA + ((c + 1) & 1) * BM * LDA);
    __builtin_amdgcn_sched_barrier(0);
    if (is_mma) {
      const float* a = sA + (c & 1) * BM * LDA + l32 * LDA + half * 4 + wk * GK;
#pragma unroll
      for (int g = 0; g < GPW; ++g) {
        const f32x4_t fa = *reinterpret_cast<const f32x4_t*>(a + g * WAVES_K * GK);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < NJ; ++j) {
            if constexpr (MT == 32) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(ring[g % AHEAD][i].v[j], fa[i], acc[j], 0, 0, 0);
            else acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(ring[g % AHEAD][i].v[j], fa[i], acc[j], 0, 0, 0);
          }
        __builtin_amdgcn_sched_barrier(0);
        load_b(ring[g % AHEAD], group_k(c * GPW + g + AHEAD));  // (past the end: clamped, unused)
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
  }

  if constexpr (WAVES_K > 1) {
    // partial tiles of the k slices -> LDS (the A buffers are free after the last barrier),
    // added by the wavefront of slice 0 in slice order
    constexpr int Q = ACC / 4;  // 128-bit pieces of an accumulator tile per lane
    f32x4_t* red = reinterpret_cast<f32x4_t*>(smem);  // [WAVES_K - 1][WAVES_N][NJ * Q][64]
    if (is_mma && wk > 0) {
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int q = 0; q < Q; ++q)
          red[(((wk - 1) * WAVES_N + wn) * NJ * Q + j * Q + q) * 64 + lane] =
              f32x4_t{acc[j][q * 4], acc[j][q * 4 + 1], acc[j][q * 4 + 2], acc[j][q * 4 + 3]};
    }
    __syncthreads();
    if (!is_mma || wk > 0) return;
#pragma unroll
    for (int s = 1; s < WAVES_K; ++s)
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int q = 0; q < Q; ++q) {
          const f32x4_t v = red[(((s - 1) * WAVES_N + wn) * NJ * Q + j * Q + q) * 64 + lane];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[j][q * 4 + e] += v[e];
        }
  }

  // Swapped operands: lane holds row (lane % MT) of the tile; accumulator slot v of MFMA j is
  // column NJ * ((v / 4) * 4 * KSLOTS + (lane / MT) * 4 + v % 4) + j of the wave's column range.
  const int slot = m0 + l32;
  if (!is_mma || slot >= p.m) return;
  const int row = p.row_indices[slot];
  const float bias = p.bias ? p.bias[row] : 0.f;
#pragma unroll
  for (int v = 0; v < ACC; ++v) {
    const int gn = n0 + wn * WCOLS + NJ * ((v / 4) * 4 * KSLOTS + half * 4 + (v % 4));
    if (gn >= p.n) continue;
    float* dst = C + (size_t)row * p.n + gn;
    float x[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) x[j] = acc[j][v];
    if (p.accumulate) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) x[j] += dst[j];
    }
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      x[j] += bias;
      if (p.relu) x[j] = fmaxf(x[j], 0.f);
    }
    if constexpr (NJ == 4) *reinterpret_cast<f32x4_t*>(dst) = f32x4_t{x[0], x[1], x[2], x[3]};
    else *reinterpret_cast<float2*>(dst) = make_float2(x[0], x[1]);
  }
}

}  // namespace iex
