// CSR SpMM with a slice of the dense operand resident in LDS and k split over workgroups (gfx950, wave64).
//
// The row kernel (spmm_device.cuh) gathers every dense row it needs from L2: nnz * tile bytes through the
// 64 B/clk/CU vector-memory path, which is what bounds it.  An LDS gather runs at three times that rate, but a
// workgroup that stages the dense operand must share each staged row among many CSR rows or the staging itself
// costs as much as the gathers did; and a matrix with a few thousand rows has too few blocks of many rows to
// fill 256 CUs.  Hence three decisions:
//   * a workgroup owns R = WAVES * RPW CSR rows x one k slice x one tile of 64 * VEC columns; the k slices of
//     one row block run on different CUs and their fp32 partial sums meet in a second, small kernel (fixed
//     order over the slices: deterministic, no float atomics);
//   * rows are dealt to workgroups by rank in the swizzle (row_indices lists rows by decreasing length):
//     workgroup b takes ranks b, b + B, b + 2B, ... and inside it the wavefronts take them in snake order, so
//     every workgroup and every wavefront gets the same mix of long and short rows;
//   * the slice is walked in stages of KB dense rows, double-buffered, fetched by direct-to-LDS loads (one
//     wavefront instruction = 1 KB of contiguous LDS = 1, 2 or 4 dense row segments, exactly the layout the
//     gather reads), the loads of stage s + 1 in flight while stage s is gathered from; one barrier per stage.
// A wavefront keeps, per row, 64 (column, value) pairs from the row's cursor in two VGPRs; columns ascend, so
// the nonzeros that fall into a stage are the run [p0, cnt) found with one ballot.  When fewer than KB lanes
// of the window are left, the window is re-read at the cursor one stage ahead (its latency hides behind the
// stage's gathers).  Each nonzero is a v_readlane broadcast of (column, value), one LDS read of VEC elements
// and VEC FMAs; four are in flight.  Where a slice does not start at column 0, a row's cursor is found by a
// 64-way search over its column indices (three rounds cover rows of 262144 entries).
// All loads have landed at every stage boundary (s_waitcnt vmcnt(0) by hand: the direct loads are inline
// assembly the compiler cannot count), so compiler-made waits for the window loads are never too weak.
// DBG (0 in the library) switches single ingredients off for benchmarks/spmm_ksplit_ablation.hip: 1 = no gathers,
// 2 = no direct loads, 4 = no cursor search, 8 = no barrier, 16 = (column, value) from arithmetic instead of
// v_readlane, 32 = no LDS read per nonzero.  Such builds compute wrong results; every address stays in bounds.
// Requirements (checked by the host): canonical CSR (strictly ascending columns inside a row), row bytes of the
// dense operand and both dense pointers multiples of 16, n at least one 128-bit vector, k <= 262144.
#pragma once
#include "../csrc/gemm_dma_device.cuh"
#include "../csrc/spmm_device.cuh"

namespace iex {

struct KsplitParams {
  SpmmParams p;
  int row_blocks;   // ceil(m / R)
  int slices;       // k slices (S); 1 = results go straight to the output
  int slice_rows;   // dense rows per slice, a multiple of KB
  float* partial;   // [S][batch][m][n] fp32 partial sums when S > 1
};

template <int VEC, typename T, int KB>
constexpr int spmm_ksplit_lds_bytes() { return 2 * KB * kWave * VEC * (int)sizeof(T); }

template <typename T, typename IT, int VEC, int RPW, int WAVES, int KB, int DBG = 0>
__device__ __forceinline__ void spmm_ksplit_block(const KsplitParams& q, int rb, int s, int by, int z, unsigned char* smem) {
  constexpr int TW = kWave * VEC;                 // columns of a tile
  constexpr int RB = TW * (int)sizeof(T);         // bytes of a staged dense row: 256, 512 or 1024
  constexpr int STAGE = KB * RB;
  constexpr int Q = STAGE / 1024 / WAVES;         // direct loads per wavefront and stage
  constexpr int RPI = 1024 / RB;                  // dense rows per direct load
  constexpr int EPC = 16 / (int)sizeof(T);        // elements per 16-byte chunk
  constexpr int kNoCol = 0x7fffffff;
  static_assert(KB <= kWave, "a stage holds at most one window of a row's nonzeros");
  static_assert(RB == 256 || RB == 512 || RB == 1024, "tile rows of 256, 512 or 1024 bytes");
  static_assert(Q >= 1 && STAGE % (1024 * WAVES) == 0, "every wavefront fetches whole kilobytes of a stage");
  typedef vec_t<T, VEC> V;
  typedef __attribute__((address_space(3))) unsigned char lds_u8;
  typedef typename stream_word<sizeof(V)>::type W;   // the same bytes as a builtin vector: one ds_read
  typedef __attribute__((address_space(3))) const W lds_W;
  const SpmmParams& p = q.p;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = uniform(tid >> 6);
  const unsigned lds0 = (unsigned)(size_t)(lds_u8*)smem;
  const int col0 = by * TW + lane * VEC;
  const bool lane_live = col0 < p.n;

  const T* __restrict__ values = static_cast<const T*>(p.values) + (p.per_batch_values ? (size_t)z * p.nnz : (size_t)0);
  const IT* __restrict__ cols = static_cast<const IT*>(p.cols);
  const unsigned char* dense = reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.dense) + (size_t)z * p.k * p.n);

  const int k0 = s * q.slice_rows;
  const int k1 = min(p.k, k0 + q.slice_rows);
  const int stages = (k1 - k0 + KB - 1) / KB;

  // ---- what this lane fetches of every stage: row r_in of the instruction's RPI rows, 16 bytes at column cb
  const int r_in = (lane * 16) / RB;
  int fc = by * TW + ((lane * 16) % RB) / (int)sizeof(T);
  if (fc + EPC > p.n) fc = p.n - EPC;             // beyond the last column: a valid chunk nobody gathers
  const unsigned char* gcol = dense + (size_t)fc * sizeof(T);
  const size_t row_bytes = (size_t)p.n * sizeof(T);
  auto issue = [&](int st) {
    const int kb0 = k0 + st * KB;
    const unsigned base = lds0 + (st & 1) * STAGE + wave * (Q * 1024);
#pragma unroll
    for (int i = 0; i < Q; ++i) {
      const int kr = min(kb0 + (wave * Q + i) * RPI + r_in, p.k - 1);   // past the end: a valid row nobody gathers
      if (!(DBG & 2)) lds_dma16(gcol + (size_t)kr * row_bytes, __builtin_amdgcn_readfirstlane(base + i * 1024));
    }
  };
  if (stages > 0) issue(0);

  // ---- this wavefront's rows: ranks i * WAVES + (w or WAVES - 1 - w) of the workgroup's R ranks
  int row[RPW], pos[RPW], rend[RPW];
  float acc[RPW][VEC];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const int j = i * WAVES + ((i & 1) ? (WAVES - 1 - wave) : wave);
    const long long slot = (long long)j * q.row_blocks + rb;
    row[i] = -1;
    pos[i] = rend[i] = 0;
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[i][e] = 0.f;
    if (slot < p.m) {
      row[i] = uniform(p.row_indices[slot]);
      pos[i] = uniform(p.row_offsets[row[i]]);
      rend[i] = uniform(p.row_offsets[row[i] + 1]);
    }
  }
  if (k0 > 0 && !(DBG & 4)) {
    // cursor = first nonzero with column >= k0: 64-way search, the rows' rounds side by side
    int hi[RPW];
#pragma unroll
    for (int i = 0; i < RPW; ++i) hi[i] = rend[i];
#pragma unroll 1
    for (int round = 0; round < 3; ++round) {
      int probe[RPW], step[RPW];
#pragma unroll
      for (int i = 0; i < RPW; ++i) {
        const int span = hi[i] - pos[i];
        step[i] = max(1, (span + kWave - 1) / kWave);
        const int idx = pos[i] + lane * step[i];
        probe[i] = idx < hi[i] ? (int)cols[idx] : kNoCol;
      }
#pragma unroll
      for (int i = 0; i < RPW; ++i) {
        const int below = __popcll(__ballot(probe[i] < k0));   // probes ascend: the first `below` lie before the slice
        if (below == 0) {
          hi[i] = pos[i];
        } else {
          hi[i] = min(hi[i], pos[i] + below * step[i]);
          pos[i] += (below - 1) * step[i] + 1;
        }
      }
    }
  }

  // ---- windows: lane l holds nonzero wbase + l of the row (column kNoCol past the row's end)
  int c[RPW], p0[RPW];
  float v[RPW];
  auto load_window = [&](int i) {
    c[i] = kNoCol;
    v[i] = 0.f;
    p0[i] = 0;
    if (pos[i] + lane < rend[i]) {
      c[i] = (int)cols[pos[i] + lane];
      v[i] = elem<T>::to_float(values[pos[i] + lane]);
    }
  };
#pragma unroll
  for (int i = 0; i < RPW; ++i) load_window(i);

  const unsigned lane_b = lane * (unsigned)sizeof(V);
  for (int st = 0; st < stages; ++st) {
    const int kb0 = k0 + st * KB;
    const int kb_end = min(kb0 + KB, k1);
    wait_vmcnt<0>();   // my direct loads of stage st and my window loads have landed
    // The compiler counts only the loads it can see.  Left alone it waits for a window load where the window is
    // first used, with a count that takes the direct loads issued in between (younger, invisible to it) for
    // window loads, and so drains the stage that was meant to land behind this stage's gathers.  Passing the
    // windows through an empty statement here puts its wait at this point, where everything has landed.
#pragma unroll
    for (int i = 0; i < RPW; ++i) asm volatile("" : "+v"(c[i]), "+v"(v[i]));
    if (!(DBG & 8)) __syncthreads();   // everybody's have, and everybody is done gathering from stage st - 1
    if (st + 1 < stages) issue(st + 1);
    const unsigned sb = lds0 + (st & 1) * STAGE - (unsigned)kb0 * RB;   // LDS address of dense row 0, were it staged
    auto gather = [&](int i, int t) {
      const unsigned a = lane_b + (sb + (unsigned)((DBG & 16) ? kb0 + ((t * 5) & (KB - 1)) : bcast_i(c[i], t)) * RB);
      if (DBG & 32) { V r; for (int e = 0; e < VEC; ++e) r.v[e] = elem<T>::from_float(__int_as_float(a)); return r; }
      return __builtin_bit_cast(V, *reinterpret_cast<lds_W*>(a));
    };
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
      if (DBG & 1) continue;
      const int te = __popcll(__ballot(c[i] < kb_end));   // lanes [p0, te) are this stage's run
      int t = p0[i];
      pos[i] += te - t;
      for (; t + 8 <= te; t += 8) {
        V bv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) bv[u] = gather(i, t + u);
#pragma unroll
        for (int u = 0; u < 8; ++u) fma_vec<T, VEC>(acc[i], (DBG & 16) ? __int_as_float(0x3f800000 + t + u) : bcast_f(v[i], t + u), bv[u]);
      }
      if (t + 4 <= te) {
        V bv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) bv[u] = gather(i, t + u);
#pragma unroll
        for (int u = 0; u < 4; ++u) fma_vec<T, VEC>(acc[i], (DBG & 16) ? __int_as_float(0x3f800000 + t + u) : bcast_f(v[i], t + u), bv[u]);
        t += 4;
      }
      if (t < te) {
        // one to three left: the reads first, clamped to the run's last lane, then as many FMAs as there are
        const int l1 = min(t + 1, te - 1), l2 = min(t + 2, te - 1);
        const V b0 = gather(i, t), b1 = gather(i, l1), b2 = gather(i, l2);
        fma_vec<T, VEC>(acc[i], bcast_f(v[i], t), b0);
        if (t + 1 < te) fma_vec<T, VEC>(acc[i], bcast_f(v[i], t + 1), b1);
        if (t + 2 < te) fma_vec<T, VEC>(acc[i], bcast_f(v[i], t + 2), b2);
      }
      p0[i] = te;
      // fewer than KB lanes left: the next stage's run may not fit.  Re-read the window at the cursor now, straight
      // into the registers this stage no longer needs; the loads land behind the other rows' gathers.
      if (te + KB > kWave && pos[i] < rend[i] && st + 1 < stages) load_window(i);
    }
  }
  wait_vmcnt<0>();   // (a slice without stages issued nothing; otherwise everything landed at the last boundary)

  if (!lane_live) return;
  if (q.slices > 1) {
    // fp32 partial sums of this slice; the second kernel adds the slices in order
    float* __restrict__ part = q.partial + ((size_t)s * gridDim.z + z) * p.m * p.n;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {
      if (row[i] < 0) continue;
      float* o = part + (size_t)row[i] * p.n + col0;
      if constexpr (VEC % 4 == 0) {
#pragma unroll
        for (int e = 0; e < VEC; e += 4) *reinterpret_cast<float4*>(o + e) = float4{acc[i][e], acc[i][e + 1], acc[i][e + 2], acc[i][e + 3]};
      } else if constexpr (VEC == 2) {
        *reinterpret_cast<float2*>(o) = float2{acc[i][0], acc[i][1]};
      } else {
        o[0] = acc[i][0];
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    if (row[i] < 0) continue;
    const float bias = p.bias ? p.bias[row[i]] : 0.f;
    T* __restrict__ out = static_cast<T*>(p.out) + ((size_t)z * p.m + row[i]) * p.n + col0;
    if (p.accumulate) {
      const V prev = load_vec<T, VEC>(out);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[i][e] += elem<T>::to_float(prev.v[e]);
    }
    V o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float x = acc[i][e] + bias;
      if (p.relu) x = fmaxf(x, 0.f);
      o.v[e] = elem<T>::from_float(x);
    }
    store_vec<T, VEC>(out, o);
  }
}

// out[z, r, c .. c + 3] = sum over the slices, in order, of the partial sums (+ bias, ReLU, previous output).
// One thread per four adjacent columns (n % 4 == 0).
template <typename T>
__global__ __launch_bounds__(256) void spmm_ksplit_reduce_kernel(SpmmParams p, const float* __restrict__ partial, int slices, int batch) {
  const size_t quads = (size_t)batch * p.m * p.n / 4;
  const size_t per_slice = (size_t)batch * p.m * p.n;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < quads; i += (size_t)gridDim.x * 256) {
    const float4* src = reinterpret_cast<const float4*>(partial) + i;
    float4 sum = *src;
    for (int s = 1; s < slices; ++s) {
      const float4 x = *(src + s * (per_slice / 4));
      sum.x += x.x;
      sum.y += x.y;
      sum.z += x.z;
      sum.w += x.w;
    }
    float r[4] = {sum.x, sum.y, sum.z, sum.w};
    T* __restrict__ out = static_cast<T*>(p.out) + i * 4;
    if (p.accumulate) {
      const vec_t<T, 4> prev = load_vec<T, 4>(out);
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] += elem<T>::to_float(prev.v[e]);
    }
    const float bias = p.bias ? p.bias[(i * 4 / p.n) % p.m] : 0.f;
    vec_t<T, 4> o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float x = r[e] + bias;
      if (p.relu) x = fmaxf(x, 0.f);
      o.v[e] = elem<T>::from_float(x);
    }
    store_vec<T, 4>(out, o);
  }
}

}  // namespace iex
