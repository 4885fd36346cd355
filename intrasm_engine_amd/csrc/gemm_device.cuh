// Dense companion GEMM for gfx950: C = A * B (or A * B^T), fp16 / bf16 in, fp32
// accumulate on the matrix cores (v_mfma_f32_32x32x16_{f16,bf16}), LDS double-buffered.
//
// Tiling: a workgroup of 2 x WCN wavefronts (WCN = 2, or 4 for the 512-thread workgroups of
// the fused launch) owns a (2*WM*32) x (WCN*WN*32) tile of C; a wavefront owns WM x WN MFMA
// tiles of 32 x 32.  The K loop advances BK = 32 per step.
// Software pipeline: global loads run kGemmSets steps ahead of the MFMAs (one register set
// per step in flight, 128-bit loads), a set is written to the idle LDS buffer one step
// before it is consumed, one barrier per step:
//   step t:  MFMA on LDS[t%2] | registers(tile t+1) -> LDS[(t+1)%2] | issue loads of tile t+1+SETS
// so a global load has kGemmSets MFMA steps to complete (L2 / MALL latency is several steps).
// A (and B given as (N, K)) sit in LDS K-contiguous ([row][k], rows padded by 8 elements so
// that the 128-bit operand reads of 8 consecutive lanes fall in distinct banks).  B given as
// (K, N) is kept in LDS as it is in memory ([k][n], rows padded by 32 elements) and the MFMA
// operand is formed by the LDS transpose read of gfx950 (ds_read_b64_tr_b16): the 16 lanes
// of a group each point at 4 adjacent n of one k row, and lane i receives column n0+i of 4
// consecutive k rows, so no register transposes and full 128-bit global loads for both
// layouts.
// The MFMA is issued with the operands swapped (B fragment as the "A" operand): a lane
// then holds 4 adjacent columns of one row of C per accumulator quad and stores them
// with one 64-bit store.
#pragma once
#include "iex_common.h"

namespace iex {

struct GemmParams {
  int M, N, K;
  const void* A;
  const void* B;
  void* C;
  long long stride_a, stride_b, stride_c;
  int tiles_m, tiles_n;
  // epilogue beyond C = A * B, for the SpMM path that hands its product to this kernel:
  // C = relu?((accumulate ? C : 0) + A * B + row_bias[row])
  const float* row_bias = nullptr;
  int relu = 0, accumulate = 0;
  int stream_out = 0;  // C is far larger than the caches: store it with the streaming hint
  // K split over two workgroups per tile (gemm.hip): the row stride of A and of an (N, K) B when K above is only a
  // part of it (0: K is the stride), where the first workgroup to finish a tile leaves its fp32 partial sums, and
  // per tile a ticket counter and a "partial sums written" flag (both zero at launch)
  int ldk = 0;
  float* split_ws = nullptr;
  int* split_flags = nullptr;
  // K split over split_parts workgroups per tile, every one of which leaves its partial sums in the workspace and draws
  // a ticket (zero at launch); the one that draws the last adds all parts up in the order of the parts and stores
  int split_parts = 0, split_part = 0;
};

// iex_gemm with the epilogue options above (gemm.hip).
int gemm_dispatch(int dtype, int trans_b_and_shape, int M, int N, int K, const void* A, const void* B, void* C, int batch,
                  long long stride_a, long long stride_b, long long stride_c, void* stream, const float* row_bias, int relu,
                  int accumulate, void* workspace = nullptr, size_t workspace_bytes = 0, bool workspace_flags_are_zero = false);
// Bytes of workspace with which gemm_dispatch, left to choose, splits K over two workgroups per tile (0: this shape is
// not split), and where in such a workspace the words sit that must be zero at launch (gemm_dispatch zeroes them with a
// launch of its own unless the caller says it has: workspace_flags_are_zero).
size_t gemm_auto_split_bytes(int M, int N, int K, int batch);
int gemm_auto_split_parts(int M, int N, int K, int batch);   // parts of K that gemm_dispatch would use with that workspace (1: no split)
void gemm_auto_split_flags(int M, int N, int K, int batch, size_t* offset_bytes, int* words);

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kGemmBK = 32;
constexpr int kGemmPad = 8;
constexpr int kGemmLd = kGemmBK + kGemmPad;  // LDS row stride in elements (80 bytes)
constexpr int kGemmSets = 3;                 // register sets = K steps of global loads in flight

constexpr int kGemmLdbPad = 32;  // padding of a [k][n] row of B in LDS, elements

template <bool TRANS_B, int WM, int WN, int WCN = 2, int BK = kGemmBK>
constexpr int gemm_lds_bytes() {
  constexpr int a_elems = 2 * WM * 32 * (BK + kGemmPad);
  constexpr int b_elems = TRANS_B ? WCN * WN * 32 * (BK + kGemmPad) : BK * (WCN * WN * 32 + kGemmLdbPad);
  return 2 /*buffers*/ * (a_elems + b_elems) * 2 /*bytes*/;
}

typedef short s16x4 __attribute__((ext_vector_type(4)));

template <bool BF16>
__device__ __forceinline__ f32x16 mfma_32x32x16(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                   0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                  0);
  }
}

__device__ __forceinline__ float f16_to_32(unsigned short h, bool bf16) {
  if (bf16) return __uint_as_float((unsigned)h << 16);
  return (float)__builtin_bit_cast(_Float16, h);
}

__device__ __forceinline__ unsigned short f32_to_16(float v, bool bf16) {
  if (bf16) {
    __hip_bfloat16 h = __float2bfloat16(v);
    return __builtin_bit_cast(unsigned short, h);
  }
  __half h = __float2half_rn(v);
  return __builtin_bit_cast(unsigned short, h);
}

// The slice of one K step that a thread carries from global memory to LDS.
template <bool TRANS_B, int BM, int BN, int THREADS = 256, int BK_ = kGemmBK>
struct GemmStage {
  static constexpr int BK = BK_;
  static constexpr int LD = BK_ + kGemmPad;
  static constexpr int A_CHUNKS = BM * (BK / 8) / THREADS;   // 128-bit chunks per thread (A, and B^T layout)
  static constexpr int B_CHUNKS = BN * (BK / 8) / THREADS;
  static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1, "a stage must give every thread a chunk of A and of B");
  static constexpr int LDB = BN + kGemmLdbPad;               // LDS row stride of B kept as [k][n]
  static constexpr int B_ELEMS = TRANS_B ? BN * LD : BK * LDB;  // one LDS buffer of B, elements
  typedef unsigned short u16;

  u32x4 ra[A_CHUNKS];
  u32x4 rb[B_CHUNKS];  // (N,K): chunk = 8 k of one n row; (K,N): chunk = 8 n of one k row

  // Loads are unconditional, from addresses clamped into the matrices, and nothing is computed
  // on their results here: guarded loads are branches, and behind a branch the compiler can no
  // longer count the loads in flight and waits for all of them wherever one is needed.  Rows of A
  // (columns of B) beyond the matrix only feed rows (columns) of C that are never stored; the K
  // tail is zeroed when the set is written to LDS.
  __device__ __forceinline__ void load(const GemmParams& p, const u16* __restrict__ A, const u16* __restrict__ B, int m0,
                                       int n0, int kt, int tid) {
    const int k0 = kt * BK;
    const int last_k8 = p.K - 8;  // K % 8 == 0: the last whole chunk of a row
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int chunk = tid + c * THREADS;
      const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
      const int gm = min(m0 + row, p.M - 1), gk = min(k0 + kc * 8, last_k8);
      ra[c] = *reinterpret_cast<const u32x4*>(A + (size_t)gm * p.K + gk);
    }
    if constexpr (TRANS_B) {
#pragma unroll
      for (int c = 0; c < B_CHUNKS; ++c) {
        const int chunk = tid + c * THREADS;
        const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
        const int gn = min(n0 + row, p.N - 1), gk = min(k0 + kc * 8, last_k8);
        rb[c] = *reinterpret_cast<const u32x4*>(B + (size_t)gn * p.K + gk);
      }
    } else {
      const int last_n8 = p.N - 8;  // N % 8 == 0 in this layout
#pragma unroll
      for (int c = 0; c < B_CHUNKS; ++c) {
        const int chunk = tid + c * THREADS;
        const int kr = chunk / (BN / 8), nc = chunk % (BN / 8);
        const int gk = min(k0 + kr, p.K - 1), gn = min(n0 + nc * 8, last_n8);
        rb[c] = *reinterpret_cast<const u32x4*>(B + (size_t)gk * p.N + gn);
      }
    }
  }

  // kt = the K step the set carries (for the K tail: entries at k >= K are written as zeros)
  __device__ __forceinline__ void store(const GemmParams& p, u16* a, u16* b, int kt, int tid) const {
    const int k0 = kt * BK;
    const bool tail = k0 + BK > p.K;  // uniform
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int chunk = tid + c * THREADS;
      const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
      *reinterpret_cast<u32x4*>(a + row * LD + kc * 8) = (tail && k0 + kc * 8 >= p.K) ? zero : ra[c];
    }
    if constexpr (TRANS_B) {
#pragma unroll
      for (int c = 0; c < B_CHUNKS; ++c) {
        const int chunk = tid + c * THREADS;
        const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
        *reinterpret_cast<u32x4*>(b + row * LD + kc * 8) = (tail && k0 + kc * 8 >= p.K) ? zero : rb[c];
      }
    } else {
#pragma unroll
      for (int c = 0; c < B_CHUNKS; ++c) {
        const int chunk = tid + c * THREADS;
        const int kr = chunk / (BN / 8), nc = chunk % (BN / 8);
        *reinterpret_cast<u32x4*>(b + kr * LDB + nc * 8) = (tail && k0 + kr >= p.K) ? zero : rb[c];
      }
    }
  }
};

// Writes the WM x WN accumulator blocks of one wavefront to C (rounded to the 16-bit type).
template <bool BF16, int WM, int WN>
__device__ __forceinline__ void gemm_store_tile(const GemmParams& p, const f32x16 (&acc)[WM][WN], unsigned short* __restrict__ C,
                                                int m0, int n0, int wm, int wn, int lane, const float* partial = nullptr) {
  typedef unsigned short u16;
  // Swapped-operand result layout: lane holds row (lane % 32) of the 32x32 block and, in
  // accumulator quad q, columns q*8 + (lane / 32)*4 .. +3.
  const bool vec_ok = (p.N % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7) == 0);
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int gm = m0 + (wm * WM + i) * 32 + (lane & 31);
    if (gm >= p.M) continue;
    const float bias = p.row_bias ? p.row_bias[gm] : 0.f;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int gn = n0 + (wn * WN + j) * 32 + q * 8 + (lane >> 5) * 4;
        if (gn >= p.N) continue;
        u16* dst = C + (size_t)gm * p.N + gn;
        float x[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = acc[i][j][q * 4 + e];
        if (partial) {   // the other half of K: this lane's sums in the same order, 256 floats per (block, quad)
          const f32x4 o = *reinterpret_cast<const f32x4*>(partial + ((i * WN + j) * 4 + q) * 256);
          x[0] += o.x, x[1] += o.y, x[2] += o.z, x[3] += o.w;
        }
        if (p.accumulate) {
          if (vec_ok) {
            const u32x2 w = *reinterpret_cast<const u32x2*>(dst);
            x[0] += f16_to_32((u16)(w.x & 0xffffu), BF16);
            x[1] += f16_to_32((u16)(w.x >> 16), BF16);
            x[2] += f16_to_32((u16)(w.y & 0xffffu), BF16);
            x[3] += f16_to_32((u16)(w.y >> 16), BF16);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (gn + e < p.N) x[e] += f16_to_32(dst[e], BF16);
          }
        }
        u16 h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float y = x[e] + bias;
          if (p.relu) y = fmaxf(y, 0.f);
          h[e] = f32_to_16(y, BF16);
        }
        if (vec_ok) {
          u32x2 w;
          w.x = (unsigned)h[0] | ((unsigned)h[1] << 16);
          w.y = (unsigned)h[2] | ((unsigned)h[3] << 16);
          *reinterpret_cast<u32x2*>(dst) = w;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (gn + e < p.N) dst[e] = h[e];
        }
      }
    }
  }
}

// The same, through LDS: a lane's accumulators are 4 adjacent columns of 32 different rows, so the
// direct store writes 32 pieces of 16 bytes per instruction; here each 32-row block of the wavefront's
// tile is laid out in the wavefront's own slice of LDS (rows padded by 16 bytes) and read back 16 lanes
// per row, so a store instruction writes 4 rows of WN * 64 contiguous bytes.  A GEMM with a short K is a
// writer of its output: 16 x 4096 x 4096 outputs with K = 64 went from 1.7 TB/s to the rate of a fill.
// `lds` = this wavefront's slice, gemm_store_lds_bytes<WN>() bytes, nobody else touches it (no barrier
// needed: the LDS operations of one wavefront execute in order).  Needs N % 8 == 0, a 16-byte aligned
// C and no accumulation; `stream`: store with the streaming hint.
template <int WN>
constexpr int gemm_store_lds_bytes() { return 32 * (WN * 64 + 16); }

template <bool BF16, int WM, int WN>
__device__ __forceinline__ void gemm_store_tile_lds(const GemmParams& p, const f32x16 (&acc)[WM][WN], unsigned short* __restrict__ C,
                                                    int m0, int n0, int wm, int wn, int lane, unsigned char* lds, bool stream,
                                                    const float* partial = nullptr) {
  typedef unsigned short u16;
  constexpr int ROWB = WN * 64 + 16;   // bytes of a padded row
  constexpr int CPR = WN * 4;          // 16-byte chunks per row
  constexpr int RPI = kWave / CPR;     // rows a store instruction covers
  static_assert(kWave % CPR == 0 && 32 % RPI == 0, "whole rows per instruction");
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int row0 = m0 + (wm * WM + i) * 32;
    if (row0 >= p.M) break;  // (uniform)
    const int gm_w = min(row0 + (lane & 31), p.M - 1);
    const float bias = p.row_bias ? p.row_bias[gm_w] : 0.f;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        u16 h[4];
        f32x4 o = {0.f, 0.f, 0.f, 0.f};
        if (partial) o = *reinterpret_cast<const f32x4*>(partial + ((i * WN + j) * 4 + q) * 256);   // the other half of K
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float y = acc[i][j][q * 4 + e] + o[e] + bias;
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
      if (row0 + r < p.M && gn < p.N) {
        u16* dst = C + (size_t)(row0 + r) * p.N + gn;
        if (stream) {
          asm volatile("" : "+v"(dst));  // (keeps the compiler from merging this store with the plain one and dropping the hint)
          __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst));
        } else {
          *reinterpret_cast<u32x4*>(dst) = v;
        }
      }
    }
  }
}

// One C tile.  `smem` must hold gemm_lds_bytes<WM,WN>() bytes, 16-byte aligned.
// All 2 * WCN * 64 threads of the workgroup must call this (it contains barriers).
template <bool BF16, bool TRANS_B, int WM, int WN, int SETS = kGemmSets, int WCN = 2, int BK = kGemmBK>
__device__ __forceinline__ void gemm_tile(const GemmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = 2 * WM * 32;
  constexpr int BN = WCN * WN * 32;
  constexpr int LD = BK + kGemmPad;
  static_assert(SETS == 2 || SETS == 3, "register sets in flight");
  constexpr int PERIOD = SETS == 2 ? 2 : 6;  // steps after which LDS buffer and register set repeat
  typedef unsigned short u16;

  typedef GemmStage<TRANS_B, BM, BN, 2 * WCN * 64, BK> Stage;
  constexpr int LDB = Stage::LDB;
  constexpr int B_ELEMS = Stage::B_ELEMS;
  u16* sA = reinterpret_cast<u16*>(smem);  // [2][BM][LD]
  u16* sB = sA + 2 * BM * LD;              // [2][BN][LD]  or  [2][BK][LDB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WCN, wn = wave % WCN;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const u16* __restrict__ A = static_cast<const u16*>(p.A) + (size_t)z * p.stride_a;
  const u16* __restrict__ B = static_cast<const u16*>(p.B) + (size_t)z * p.stride_b;
  u16* __restrict__ C = static_cast<u16*>(p.C) + (size_t)z * p.stride_c;

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  Stage regs[SETS];  // regs[t % SETS] carries tile t (statically indexed below)

  const int KT = (p.K + BK - 1) / BK;
  // prologue: tiles 0 .. SETS-1 in flight, tile 0 into LDS[0], then tile SETS replaces it
#pragma unroll
  for (int s = 0; s < SETS; ++s)
    regs[s].load(p, A, B, m0, n0, s, tid);  // (a tile beyond the last one loads clamped addresses and is never used)
  regs[0].store(p, sA, sB, 0, tid);
  regs[0].load(p, A, B, m0, n0, SETS, tid);
  __syncthreads();

  const int frag_row = lane & 31;      // row of the 32-row operand block this lane feeds
  const int frag_k = (lane >> 5) * 8;  // which 8 of the 16 k entries of a sub-step

  // One step; PH = t % (2*SETS) is a compile-time phase so that both the register set
  // ((t+1) % SETS) and the LDS buffer (t % 2) are static.
  auto step = [&](int kt, auto phase) {
    constexpr int PH = decltype(phase)::value;
    constexpr int buf = PH & 1;
    constexpr int set = (PH + 1) % SETS;
    const u16* a = sA + buf * BM * LD + (wm * WM * 32 + frag_row) * LD + frag_k;
    // (N,K) layout: 128-bit read of 8 k of row n.  (K,N) layout: two transpose reads; the lane
    // group q = lane/16 covers n-half (q%2) and k-half (q/2) of the sub-step, lane r of the
    // group points at k row r/4 and n columns 4*(r%4).., and receives column n0 + r of 4 k rows.
    const u16* b = TRANS_B ? sB + buf * B_ELEMS + (wn * WN * 32 + frag_row) * LD + frag_k
                           : sB + buf * B_ELEMS + ((lane >> 5) * 8 + ((lane & 15) >> 2)) * LDB + wn * WN * 32 +
                                 ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    // the operand fragments of two 16-wide sub-steps are requested before their MFMAs: the reads
    // of the second land while the MFMAs of the first run
#pragma unroll
    for (int kp = 0; kp < BK / 32; ++kp) {
      u32x4 fa[2][WM], fb[2][WN];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int ks = kp * 2 + h;
#pragma unroll
        for (int i = 0; i < WM; ++i) fa[h][i] = *reinterpret_cast<const u32x4*>(a + i * 32 * LD + ks * 16);
#pragma unroll
        for (int j = 0; j < WN; ++j) {
          if constexpr (TRANS_B) {
            fb[h][j] = *reinterpret_cast<const u32x4*>(b + j * 32 * LD + ks * 16);
          } else {
            typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
            const u16* q0 = b + (ks * 16) * LDB + j * 32;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q0 + 4 * LDB));
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            fb[h][j] = u32x4{l2.x, l2.y, h2.x, h2.y};
          }
        }
      }
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j) acc[i][j] = mfma_32x32x16<BF16>(fb[h][j], fa[h][i], acc[i][j]);
    }
    // unconditional on purpose (see GemmStage::load): past the last tile this writes zeros to the
    // idle buffer and fetches clamped addresses
    regs[set].store(p, sA + (buf ^ 1) * BM * LD, sB + (buf ^ 1) * B_ELEMS, kt + 1, tid);
    regs[set].load(p, A, B, m0, n0, kt + 1 + SETS, tid);
    __syncthreads();
  };

  int kt = 0;
  if constexpr (PERIOD == 6) {
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
  } else {
    for (; kt + 2 <= KT; kt += 2) {
      step(kt + 0, std::integral_constant<int, 0>{});
      step(kt + 1, std::integral_constant<int, 1>{});
    }
    if (kt < KT) step(kt++, std::integral_constant<int, 0>{});
  }

  gemm_store_tile<BF16, WM, WN>(p, acc, C, m0, n0, wm, wn, lane);
}

}  // namespace iex
