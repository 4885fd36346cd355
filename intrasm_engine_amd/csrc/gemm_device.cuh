// Dense companion GEMM for gfx950: C = A * B (or A * B^T), fp16 / bf16 in, fp32
// accumulate on the matrix cores (v_mfma_f32_32x32x16_{f16,bf16}), LDS double-buffered.
//
// Tiling: a workgroup of 4 wavefronts (2 x 2) owns a (2*WM*32) x (2*WN*32) tile of C;
// a wavefront owns WM x WN MFMA tiles of 32 x 32.  The K loop advances BK = 32 per step:
//   global -> registers (next step, 128-bit loads) | MFMA on the current LDS buffer |
//   registers -> the other LDS buffer | one barrier.
// Both operands sit in LDS K-contiguous ([row][k], rows padded by 8 elements so that the
// 128-bit operand reads of 8 consecutive lanes fall in distinct banks).  When B is given
// as (K, N) a thread transposes 4 x 4 blocks in registers (v_perm_b32) on the way in, so
// the MFMA operand reads are identical for both layouts.
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
};

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kGemmBK = 32;
constexpr int kGemmPad = 8;
constexpr int kGemmLd = kGemmBK + kGemmPad;  // LDS row stride in elements (80 bytes)

template <int WM, int WN>
constexpr int gemm_lds_bytes() {
  return 2 /*buffers*/ * (2 * WM * 32 + 2 * WN * 32) * kGemmLd * 2 /*bytes*/;
}

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

__device__ __forceinline__ unsigned short f32_to_16(float v, bool bf16) {
  if (bf16) {
    __hip_bfloat16 h = __float2bfloat16(v);
    return __builtin_bit_cast(unsigned short, h);
  }
  __half h = __float2half_rn(v);
  return __builtin_bit_cast(unsigned short, h);
}

// One C tile.  `smem` must hold gemm_lds_bytes<WM,WN>() bytes, 16-byte aligned.
// All 256 threads of the workgroup must call this (it contains barriers).
template <bool BF16, bool TRANS_B, int WM, int WN>
__device__ __forceinline__ void gemm_tile(const GemmParams& p, int tile_m, int tile_n, int z, unsigned char* smem) {
  constexpr int BM = 2 * WM * 32;
  constexpr int BN = 2 * WN * 32;
  constexpr int BK = kGemmBK;
  constexpr int LD = kGemmLd;
  constexpr int A_CHUNKS = BM * (BK / 8) / 256;        // 128-bit chunks per thread (A, and B^T layout)
  constexpr int B_CHUNKS = BN * (BK / 8) / 256;
  constexpr int B_TASKS = (BK / 4) * (BN / 4) / 256;   // 4x4 blocks per thread (B as (K,N))
  typedef unsigned short u16;

  u16* sA = reinterpret_cast<u16*>(smem);               // [2][BM][LD]
  u16* sB = sA + 2 * BM * LD;                           // [2][BN][LD]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
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

  u32x4 ra[A_CHUNKS];
  u32x4 rb[B_CHUNKS];      // trans_b layout
  u32x2 rbt[B_TASKS][4];   // (K,N) layout: 4 k-rows x 4 n-columns per task

  auto load_global = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int chunk = tid + c * 256;
      const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
      const int gm = m0 + row, gk = k0 + kc * 8;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (gm < p.M && gk < p.K) v = *reinterpret_cast<const u32x4*>(A + (size_t)gm * p.K + gk);
      ra[c] = v;
    }
    if constexpr (TRANS_B) {
#pragma unroll
      for (int c = 0; c < B_CHUNKS; ++c) {
        const int chunk = tid + c * 256;
        const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
        const int gn = n0 + row, gk = k0 + kc * 8;
        u32x4 v = {0u, 0u, 0u, 0u};
        if (gn < p.N && gk < p.K) v = *reinterpret_cast<const u32x4*>(B + (size_t)gn * p.K + gk);
        rb[c] = v;
      }
    } else {
#pragma unroll
      for (int t = 0; t < B_TASKS; ++t) {
        const int task = tid + t * 256;
        const int kg = task / (BN / 4), nc = task % (BN / 4);
        const int gn = n0 + nc * 4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int gk = k0 + kg * 4 + r;
          u32x2 v = {0u, 0u};
          if (gn < p.N && gk < p.K) v = *reinterpret_cast<const u32x2*>(B + (size_t)gk * p.N + gn);
          rbt[t][r] = v;
        }
      }
    }
  };

  auto store_lds = [&](int buf) {
    u16* a = sA + buf * BM * LD;
    u16* b = sB + buf * BN * LD;
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c) {
      const int chunk = tid + c * 256;
      const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
      *reinterpret_cast<u32x4*>(a + row * LD + kc * 8) = ra[c];
    }
    if constexpr (TRANS_B) {
#pragma unroll
      for (int c = 0; c < B_CHUNKS; ++c) {
        const int chunk = tid + c * 256;
        const int row = chunk / (BK / 8), kc = chunk % (BK / 8);
        *reinterpret_cast<u32x4*>(b + row * LD + kc * 8) = rb[c];
      }
    } else {
#pragma unroll
      for (int t = 0; t < B_TASKS; ++t) {
        const int task = tid + t * 256;
        const int kg = task / (BN / 4), nc = task % (BN / 4);
        // rbt[t][r] = {B[k+r][n], B[k+r][n+1] | B[k+r][n+2], B[k+r][n+3]}; column e of the 4x4
        // block becomes the 4 consecutive k entries of LDS row n+e.
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const unsigned sel = (e & 1) ? 0x07060302u : 0x05040100u;  // high or low halves of (src1, src0)
          u32x2 w;
          w.x = __builtin_amdgcn_perm(rbt[t][1][e >> 1], rbt[t][0][e >> 1], sel);
          w.y = __builtin_amdgcn_perm(rbt[t][3][e >> 1], rbt[t][2][e >> 1], sel);
          *reinterpret_cast<u32x2*>(b + (nc * 4 + e) * LD + kg * 4) = w;
        }
      }
    }
  };

  const int KT = (p.K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  const int frag_row = lane & 31;        // row of the 32-row operand block this lane feeds
  const int frag_k = (lane >> 5) * 8;    // which 8 of the 16 k entries of a sub-step

  for (int kt = 0; kt < KT; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < KT) load_global(kt + 1);
    const u16* a = sA + buf * BM * LD + (wm * WM * 32 + frag_row) * LD + frag_k;
    const u16* b = sB + buf * BN * LD + (wn * WN * 32 + frag_row) * LD + frag_k;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      u32x4 fa[WM], fb[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i) fa[i] = *reinterpret_cast<const u32x4*>(a + i * 32 * LD + ks * 16);
#pragma unroll
      for (int j = 0; j < WN; ++j) fb[j] = *reinterpret_cast<const u32x4*>(b + j * 32 * LD + ks * 16);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) acc[i][j] = mfma_32x32x16<BF16>(fb[j], fa[i], acc[i][j]);
    }
    if (kt + 1 < KT) store_lds(buf ^ 1);
    __syncthreads();
  }

  // Swapped-operand result layout: lane holds row (lane % 32) of the 32x32 block and, in
  // accumulator quad q, columns q*8 + (lane / 32)*4 .. +3.
  const bool vec_ok = (p.N % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 7) == 0);
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int gm = m0 + (wm * WM + i) * 32 + (lane & 31);
    if (gm >= p.M) continue;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int gn = n0 + (wn * WN + j) * 32 + q * 8 + (lane >> 5) * 4;
        if (gn >= p.N) continue;
        u16 h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) h[e] = f32_to_16(acc[i][j][q * 4 + e], BF16);
        u16* dst = C + (size_t)gm * p.N + gn;
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

}  // namespace iex
