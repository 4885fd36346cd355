// CSR SDDMM for gfx950 (wave64): out[j] = <lhs[row(j), :], rhs[col(j), :]>.
//
// Work decomposition
//   * a wavefront owns one CSR row (swizzled order) or, for long rows, every WPR-th
//     chunk of 64 nonzeros of it; outputs are independent, so no reduction crosses
//     wavefronts and nothing is atomic;
//   * a group of LPN adjacent lanes handles one nonzero: the LPN lanes read one rhs row
//     as a single contiguous LPN*VEC*sizeof(T) segment (128-bit per lane when the shape
//     allows), so G = 64/LPN nonzeros are in flight per instruction;
//   * the lhs row fragment that a lane needs is the same for every nonzero of the row
//     and is held in registers when k <= 2*LPN*VEC (the attention shapes); otherwise it
//     is re-read (it hits L1: every group reads the same bytes);
//   * column indices are read 64 at a time (one per lane, the next 64 prefetched) and a
//     full chunk issues all its gathers before the first reduction;
//   * the LPN partial dot products are summed with DPP row operations (quad_perm,
//     row_half_mirror, row_mirror): no LDS, no bpermute in the reduction.
// Accumulation is fp32; with SUM_OVER_BATCH the batch loop runs inside the kernel so
// the (nnz) output is a deterministic sum.
#include <algorithm>
#include <cmath>
#include "iex_common.h"
#include "sddmm_mfma_device.cuh"

namespace iex {
namespace {

struct SddmmParams {
  int m, k, n, nnz, batch;
  const int* row_indices;
  const int* row_offsets;
  const int* cols;
  const void* lhs;
  const void* rhs;
  void* out;
  int sum_over_batch, accumulate;
  int deep = 0;  // generic-k path: keep four slices of both rows in flight (set by the launcher)
};

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <typename T, int VEC>
__device__ __forceinline__ float dot_vec(const vec_t<T, VEC>& a, const vec_t<T, VEC>& b, float acc) {
  if constexpr (sizeof(T) == 2 && VEC >= 2 && __is_same(T, __half)) {
#pragma unroll
    for (int i = 0; i < VEC / 2; ++i) {
      f16x2 x = __builtin_bit_cast(f16x2, *reinterpret_cast<const uint32_t*>(&a.v[2 * i]));
      f16x2 y = __builtin_bit_cast(f16x2, *reinterpret_cast<const uint32_t*>(&b.v[2 * i]));
      acc = __builtin_amdgcn_fdot2(x, y, acc, false);
    }
    return acc;
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      acc = fmaf(elem<T>::to_float(a.v[i]), elem<T>::to_float(b.v[i]), acc);
    return acc;
  }
}

// PASSES > 0: k <= PASSES*LPN*VEC (EXACT: k equals it, so no load needs a predicate): the lhs
//             fragment of a (row, batch entry) is one register load per pass; a chunk of 64
//             nonzeros takes LPN steps of G nonzeros: all column indices are shuffled out and
//             all gathers issued first, then step s reduces and leaves its result in lane s of
//             every group, so each lane ends up with exactly one output (nonzero lane%LPN*G +
//             lane/LPN) and the chunk is written with ONE store instruction that covers 64
//             consecutive outputs.  Plain stores only (no accumulate mode).
// PASSES == 0: generic k and accumulate mode, operands streamed in LPN*VEC slices.
// A block serves kSddmmZb batch entries (grid.z = ceil(batch / kSddmmZb)) in per-entry output
// mode, so the row's column indices are fetched once and reused.
constexpr int kSddmmZb = 4;

template <typename T, int VEC, int LPN, int PASSES, int WPR, bool EXACT>
__global__ __launch_bounds__(256) void sddmm_kernel(SddmmParams p) {
  constexpr int G = kWave / LPN;
  constexpr int KT = LPN * VEC;
  constexpr int kRowsPerBlock = 4 / WPR;
  const int lane = lane_id();
  const int wave = uniform(threadIdx.x >> 6);
  const int sub = lane / LPN;
  const int sl = lane % LPN;
  const int row_slot = blockIdx.x * kRowsPerBlock + wave / WPR;
  const int part = wave % WPR;
  if (row_slot >= p.m) return;

  const int row = uniform(p.row_indices[row_slot]);
  const int start = uniform(p.row_offsets[row]);
  const int end = uniform(p.row_offsets[row + 1]);
  // per-entry output: this block's slice of the batch; batch-summed output: one pass that
  // loops over the whole batch inside the dot product
  const int zbeg = p.sum_over_batch ? 0 : (int)blockIdx.z * kSddmmZb;
  const int zend = p.sum_over_batch ? 1 : min(p.batch, zbeg + kSddmmZb);
  const int zn = p.sum_over_batch ? p.batch : 1;
  const size_t lhs_zstride = (size_t)p.m * p.k;
  const size_t rhs_zstride = (size_t)p.n * p.k;
  const T* __restrict__ lhs_row = static_cast<const T*>(p.lhs) + (size_t)row * p.k;
  const T* __restrict__ rhs_all = static_cast<const T*>(p.rhs);
  T* __restrict__ out_all = static_cast<T*>(p.out);

  // column index of nonzero base+lane; the next chunk's indices are fetched while the
  // current chunk is processed
  int base = start + part * kWave;
  int c = (base + lane < end) ? p.cols[base + lane] : 0;
  for (; base < end; base += kWave * WPR) {
    const int next = base + kWave * WPR;
    const int c_next = (next + lane < end) ? p.cols[next + lane] : 0;
    const int cnt = min(kWave, end - base);
    if constexpr (PASSES > 0) {
      // slots past cnt carry column 0: they gather a valid row and their result is dropped
      int cc[LPN];
#pragma unroll
      for (int st = 0; st < LPN; ++st) cc[st] = __shfl(c, st * G + sub, kWave);
      const int my_t = sl * G + sub;  // the nonzero whose result this lane will hold
      for (int z = zbeg; z < zend; ++z) {
        const T* __restrict__ lhs = lhs_row + (size_t)z * lhs_zstride;
        const T* __restrict__ rhs = rhs_all + (size_t)z * rhs_zstride;
        vec_t<T, VEC> lfrag[PASSES];
        vec_t<T, VEC> rv[LPN][PASSES];
#pragma unroll
        for (int ps = 0; ps < PASSES; ++ps) {
          const int kk = ps * KT + sl * VEC;
          if (EXACT || kk < p.k) lfrag[ps] = load_vec<T, VEC>(lhs + kk);
        }
#pragma unroll
        for (int st = 0; st < LPN; ++st) {
          const T* r = rhs + (size_t)cc[st] * p.k;
#pragma unroll
          for (int ps = 0; ps < PASSES; ++ps) {
            const int kk = ps * KT + sl * VEC;
            if (EXACT || kk < p.k) rv[st][ps] = load_vec<T, VEC>(r + kk);
          }
        }
        float res = 0.f;
#pragma unroll
        for (int st = 0; st < LPN; ++st) {
          float acc = 0.f;
#pragma unroll
          for (int ps = 0; ps < PASSES; ++ps)
            if (EXACT || ps * KT + sl * VEC < p.k) acc = dot_vec<T, VEC>(lfrag[ps], rv[st][ps], acc);
          acc = group_sum<LPN>(acc);
          res = (sl == st) ? acc : res;
        }
        if (my_t < cnt) out_all[(p.sum_over_batch ? (size_t)0 : (size_t)z * p.nnz) + base + my_t] = elem<T>::from_float(res);
      }
    } else {
      for (int z = zbeg; z < zend; ++z) {
        const T* __restrict__ lhs = lhs_row + (size_t)z * lhs_zstride;
        const T* __restrict__ rhs = rhs_all + (size_t)z * rhs_zstride;
        T* __restrict__ out = out_all + (p.sum_over_batch ? (size_t)0 : (size_t)z * p.nnz);
        const int steps = (cnt + G - 1) / G;
        for (int st = 0; st < steps; ++st) {
          const int t = st * G + sub;           // nonzero of this chunk handled by my lane group
          const int col = __shfl(c, t, kWave);  // t < 64 always; slots past cnt carry column 0
          float acc = 0.f;
          for (int zz = 0; zz < zn; ++zz) {
            const T* l = lhs + (size_t)zz * lhs_zstride;
            const T* r = rhs + (size_t)zz * rhs_zstride + (size_t)col * p.k;
            int kk = sl * VEC;
            if (p.deep) {
              // few wavefronts on the chip: a long k is a chain of load -> multiply -> load with one
              // memory latency per slice unless several slices are in flight.  (With the chip full,
              // other wavefronts hide that latency and the extra rows in flight only cost cache hits:
              // 4096 x 4096 at 90 %, k = 2048, fp32: 1.16 ms plain, 1.67 ms this way; 1024 x 1024 at
              // 95 %, k = 4096: 0.36 ms plain, 0.13 ms this way.)
              for (; kk + 3 * KT < p.k; kk += 4 * KT) {
                vec_t<T, VEC> lv[4], rv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                  lv[u] = load_vec<T, VEC>(l + kk + u * KT);
                  rv[u] = load_vec<T, VEC>(r + kk + u * KT);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) acc = dot_vec<T, VEC>(lv[u], rv[u], acc);
              }
            }
            for (; kk < p.k; kk += KT)
              acc = dot_vec<T, VEC>(load_vec<T, VEC>(l + kk), load_vec<T, VEC>(r + kk), acc);
          }
          acc = group_sum<LPN>(acc);
          if (sl == 0 && t < cnt) {
            const size_t o = (size_t)base + t;
            if (p.accumulate) acc += elem<T>::to_float(out[o]);
            out[o] = elem<T>::from_float(acc);
          }
        }
      }
    }
    c = c_next;
  }
}

template <typename T, int VEC, int LPN, int PASSES, int WPR, bool EXACT>
int launch_one(const SddmmParams& p0, hipStream_t stream) {
  SddmmParams p = p0;
  dim3 grid(ceil_div(p.m, 4 / WPR), 1, p.sum_over_batch ? 1 : ceil_div(p.batch, kSddmmZb));
  p.deep = (long long)grid.x * grid.z * 4 <= 2048;  // at most two wavefronts per SIMD of the chip
  note_kernel("sddmm_kernel<%s, %d, %d, %d, %d, %s>", type_name<T>(), VEC, LPN, PASSES, WPR, EXACT ? "true" : "false");
  hipLaunchKernelGGL((sddmm_kernel<T, VEC, LPN, PASSES, WPR, EXACT>), grid, dim3(256), 0, stream, p);
  return check_hip(hipGetLastError(), "sddmm launch");
}

template <typename T, int VEC, int LPN, int PASSES, bool EXACT>
int launch_wpr(const SddmmParams& p, int wpr, hipStream_t stream) {
  if (wpr == 4) return launch_one<T, VEC, LPN, PASSES, 4, EXACT>(p, stream);
  return launch_one<T, VEC, LPN, PASSES, 1, EXACT>(p, stream);
}

template <typename T, int VEC, int LPN>
int launch_passes(const SddmmParams& p, int wpr, hipStream_t stream) {
  // register-resident lhs needs one batch entry per dot product and plain stores
  const bool fast = !(p.sum_over_batch && p.batch > 1) && !p.accumulate;
  constexpr int kt = LPN * VEC;
  if (fast && p.k == kt) return launch_wpr<T, VEC, LPN, 1, true>(p, wpr, stream);
  if (fast && p.k == 2 * kt) return launch_wpr<T, VEC, LPN, 2, true>(p, wpr, stream);
  if (fast && p.k < kt) return launch_wpr<T, VEC, LPN, 1, false>(p, wpr, stream);
  if (fast && p.k < 2 * kt) return launch_wpr<T, VEC, LPN, 2, false>(p, wpr, stream);
  return launch_wpr<T, VEC, LPN, 0, false>(p, wpr, stream);
}

template <typename T>
int launch_typed(const SddmmParams& p, int wpr, hipStream_t stream) {
  constexpr int kMax = 16 / (int)sizeof(T);
  int vec = kMax;
  while (vec > 1 && (p.k % vec != 0 || !aligned(p.lhs, sizeof(T) * vec) || !aligned(p.rhs, sizeof(T) * vec)))
    vec >>= 1;
  // lanes per nonzero: enough to cover k in one or two passes, at most 16 (one DPP row)
  if (vec == kMax) {
    if (p.k <= 8 * vec) return launch_passes<T, kMax, 8>(p, wpr, stream);
    return launch_passes<T, kMax, 16>(p, wpr, stream);
  }
  if (vec >= 2) return launch_passes<T, 2, 16>(p, wpr, stream);
  return launch_passes<T, 1, 16>(p, wpr, stream);
}

// ---- dense product, then sampling (16-bit types, caller's workspace of m * n * 2 bytes) ----
// A long k makes the gather kernel read k * 2 bytes of rhs per nonzero through the L2 -> CU path;
// the dense GEMM computes all m * n dot products on the matrix cores in less time than that takes
// once the mask is not very sparse, and a small kernel then picks the nonzeros' entries.
// Same arithmetic per output (fp32 accumulation over k, one rounding to the 16-bit type).
__global__ __launch_bounds__(256) void sample_dense_kernel(int m, int n, const int* __restrict__ row_offsets,
                                                           const int* __restrict__ cols,
                                                           const uint16_t* __restrict__ dense,
                                                           uint16_t* __restrict__ out) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= m) return;
  const int start = row_offsets[row], end = row_offsets[row + 1];
  const uint16_t* drow = dense + (size_t)row * n;
  for (int j = start + lane_id(); j < end; j += kWave) out[j] = drow[cols[j]];
}

inline bool sddmm_dense_fits(int dtype, const SddmmParams& p) {
  return (dtype == IEX_F16 || dtype == IEX_BF16) && !p.accumulate && !(p.sum_over_batch && p.batch > 1) &&
         p.k > 0 && p.k % 8 == 0 && p.n % 8 == 0 && (long long)p.m * p.n < (1ll << 31) && aligned(p.lhs, 16) &&
         aligned(p.rhs, 16);
}

inline size_t sddmm_dense_bytes(const SddmmParams& p) { return (size_t)p.m * p.n * 2; }

// Time model fitted on MI355X (fp16).  Dense product per batch entry: three launches, the GEMM at
// 1000 TFLOP/s or, with few tiles, 0.23 us per K step of 32 per round of 512 tiles of 128 x 128,
// m * n * 2 bytes written and nnz entries picked at 4 TB/s.  Gather kernel: nnz * k * 2 bytes at
// 15 TB/s (16 heads of 4096 x 4096 at 93 % sparsity, k = 64: 125 us; 2048 x 1024 at 80 %, k = 2048:
// 117 us), and with a k beyond the register-resident fragments no less than one wave's chain of
// loads (0.12 us per 128 elements of k and step of 4 nonzeros with four slices in flight:
// 1024 x 1024 at 95 %, k = 4096: 50 us).  Measured: 11008 x 4096 at 80 %, k = 8192 (weight gradient of an MLP
// projection) 16.5 -> 0.77 ms; 4096 x 4096 at 50 %, k = 8192 9.7 -> 0.32 ms; 4096 x 4096 at 90 %,
// k = 512 120 -> 55 us.  The dense product has to win by 15 %.
inline bool sddmm_dense_wins(const SddmmParams& p) {
  const double flops = 2.0 * p.m * p.n * p.k;
  const double tiles = (double)ceil_div(p.m, 128) * ceil_div(p.n, 128);
  const double product = std::max(flops / 1000e12, std::ceil(tiles / 512.0) * (p.k / 32.0) * 0.23e-6);
  const double dense = p.batch * (16e-6 + product + ((double)p.m * p.n * 2 + (double)p.nnz * 8) / 4e12);
  const double row_nnz = (double)p.nnz / p.m;
  const double chain = p.k > 256 ? std::ceil(row_nnz / (row_nnz >= 64.0 ? 16.0 : 4.0)) * (p.k / 128.0) * 0.12e-6 : 0.0;
  const double gather = std::max(8e-6 + (double)p.batch * p.nnz * p.k * 2 / 15e12, chain);
  return 1.15 * dense < gather;
}

int launch_sddmm_dense(int dtype, const SddmmParams& p, void* ws, hipStream_t stream) {
  for (int z = 0; z < p.batch; ++z) {
    const uint16_t* lhs = static_cast<const uint16_t*>(p.lhs) + (size_t)z * p.m * p.k;
    const uint16_t* rhs = static_cast<const uint16_t*>(p.rhs) + (size_t)z * p.n * p.k;
    // (the dispatcher, not the public entry point: that one starts a new trail of kernel names)
    if (int rc = gemm_dispatch(dtype, 1, p.m, p.n, p.k, lhs, rhs, ws, 1, 0, 0, 0, stream, nullptr, 0, 0)) return rc;
    note_kernel("sample_dense_kernel");
    hipLaunchKernelGGL(sample_dense_kernel, dim3(ceil_div(p.m, 4)), dim3(256), 0, stream, p.m, p.n, p.row_offsets, p.cols,
                       static_cast<const uint16_t*>(ws), static_cast<uint16_t*>(p.out) + (size_t)z * p.nnz);
    if (int rc = check_hip(hipGetLastError(), "sddmm sampling launch")) return rc;
  }
  return 0;
}

// ---- score tiles on the matrix cores, sampled inside the workgroup (sddmm_mfma_device.cuh) ----
// 16-bit types, k = 32, 64 or 128, plain store, one output per batch entry, canonical CSR (columns ascending and
// distinct inside a row), n <= 128 * kSdMaxTiles; the workspace holds (6 ceil(n / 128) + 1) * m words (per row and
// column tile: a 128-bit mask, a cursor, a packed word).
inline bool sddmm_mfma_fits(int dtype, const SddmmParams& p) {
  return (dtype == IEX_F16 || dtype == IEX_BF16) && !p.accumulate && !(p.sum_over_batch && p.batch > 1) &&
         (p.k == 32 || p.k == 64 || p.k == 128) && aligned(p.lhs, 16) && aligned(p.rhs, 16) &&
         ceil_div(p.n, kSdBN) <= kSdMaxTiles && (long long)(ceil_div(p.n, kSdBN) + 1) * p.m < (1ll << 28);
}

inline size_t sddmm_mfma_bytes(const SddmmParams& p) { return sb_words(p.m, ceil_div(p.n, kSdBN), p.nnz) * sizeof(int); }

// The host does not look at the pattern, so the choice goes by the mask's overall density.  Measured on MI355X
// (fp16, 16 heads of 4096 x 4096, k = 64, microseconds, gather kernel / this kernel with its two setup kernels;
// bench.py, extras.sddmm_fp16_16heads_by_mask):
//   band of 256 + 32 scattered per row (7 %)  114 /  54      band of 512 + 32 (13 %)      213 /  70
//   band of 128 + 16 scattered (3.5 %)          73 /  45      block diagonal 256 (6 %)      98 /  34
//   causal window of 512 (12 %)                173 /  55
//   equal rows, columns at random:  1 %  29 (stays on the gather kernel)   5 %  89 / 100    10 %  155 / 177
//                                  20 % 287 / 175
// (a caller that keeps tables and lists saves 15 of these microseconds per call).  Masks with structure (what per-entry
// SDDMM is used for: attention) gain 1.6x to 3x from 3 % up; a mask without any loses 1.1x to 1.2x below 15 %.
// IEX_SDDMM_FORCE_VARIANT(1) keeps the gather kernel.
inline bool sddmm_mfma_wins(const SddmmParams& p) {
  const double density = (double)p.nnz / ((double)p.m * p.n);
  return density >= 0.03 && (double)p.batch * p.m * p.n >= 32.0 * 1024 * 1024;
}

template <bool BF16, int KS>
int launch_sddmm_mfma_ks(const SddmmMfmaParams& q, int batch, hipStream_t stream) {
  constexpr int lds = sddmm_mfma_lds_bytes<KS>();
  auto kernel = sddmm_mfma_kernel<BF16, KS>;
  static thread_local bool raised = false;   // per instantiation: more than 64 KB of dynamic LDS
  if (!raised) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "hipFuncSetAttribute(LDS size)"))
      return rc;
    raised = true;
  }
  note_kernel("sddmm_mfma_kernel<%s, %d>", BF16 ? "true" : "false", KS);
  hipLaunchKernelGGL(kernel, dim3(ceil_div(q.m, kSdBM), batch), dim3(kSdThreads), lds, stream, q);
  return check_hip(hipGetLastError(), "sddmm (matrix-core) launch");
}

// ready: bit 0 = the caller vouches that an earlier call on this pattern left the tables in the workspace, bit 1 = that the
// lists are there too, from a call with the same dense_code (this kernel's, or the SpMM's for such patterns: same lists).
int launch_sddmm_mfma(int dtype, const SddmmParams& p, void* ws, int dense_code, int ready, hipStream_t stream) {
  const int tiles_n = ceil_div(p.n, kSdBN);
  const SdTables t = sd_tables(ws, p.m, tiles_n);
  const SbLists l = sb_lists(ws, p.m, tiles_n, p.nnz);
  // dense_code (for tests and tuning): 0 = the built-in threshold, 1 = every tile on the matrix cores, 255 = none,
  // else 64 * code nonzeros per 128 x 128 block
  if (int rc = sb_setup(t, l, p.m, tiles_n, dense_code, ready, p.row_offsets, p.cols, stream)) return rc;
  SddmmMfmaParams q{p.m, p.k, p.n, p.nnz, p.cols, p.lhs, p.rhs, p.out, t.mask, t.tile_ptr, t.brief, tiles_n,
                    p.row_offsets, l.thin_ent, l.thin_cnt, l.dense_list};
  const bool bf16 = dtype == IEX_BF16;
  switch (p.k) {
    case 32: return bf16 ? launch_sddmm_mfma_ks<true, 2>(q, p.batch, stream) : launch_sddmm_mfma_ks<false, 2>(q, p.batch, stream);
    case 64: return bf16 ? launch_sddmm_mfma_ks<true, 4>(q, p.batch, stream) : launch_sddmm_mfma_ks<false, 4>(q, p.batch, stream);
    default: return bf16 ? launch_sddmm_mfma_ks<true, 8>(q, p.batch, stream) : launch_sddmm_mfma_ks<false, 8>(q, p.batch, stream);
  }
}

}  // namespace

// Bytes of workspace with which iex_sddmm_ws would compute the dense product and sample it (0: it
// would not, whatever the workspace).  Pointers are taken to be 16-byte aligned.
// What iex_sddmm_ws would do with a workspace of the size that sddmm_workspace_bytes names: 0 = not use it, 3 = keep the
// tables of the kernel for masks with structure in it, 7 = the dense product.
int sddmm_workspace_kind(int dtype, int flags, int m, int k, int n, int nonzeros, int batch) {
  if (m <= 0 || k <= 0 || n <= 0 || nonzeros <= 0 || batch <= 0) return 0;
  const int variant = (flags >> 16) & 0xf;
  if (variant != 0 && variant != 7 && variant != 3) return 0;
  void* const some_aligned = reinterpret_cast<void*>(size_t(256));
  SddmmParams p{m, k, n, nonzeros, batch, nullptr, nullptr, nullptr, some_aligned, some_aligned, nullptr,
                (flags & IEX_SDDMM_SUM_OVER_BATCH) != 0, (flags & IEX_SDDMM_ACCUMULATE) != 0};
  const bool any_order = (flags & IEX_SDDMM_ANY_COLUMN_ORDER) != 0;
  if (variant != 7 && sddmm_mfma_fits(dtype, p) && (variant == 3 || (!any_order && sddmm_mfma_wins(p)))) return 3;
  if (variant == 3 || !sddmm_dense_fits(dtype, p)) return 0;
  return (variant == 7 || sddmm_dense_wins(p)) ? 7 : 0;
}

size_t sddmm_workspace_bytes(int dtype, int flags, int m, int k, int n, int nonzeros, int batch) {
  if (m <= 0 || k <= 0 || n <= 0 || nonzeros <= 0 || batch <= 0) return 0;
  const int variant = (flags >> 16) & 0xf;
  if (variant != 0 && variant != 7 && variant != 3) return 0;
  void* const some_aligned = reinterpret_cast<void*>(size_t(256));
  SddmmParams p{m, k, n, nonzeros, batch, nullptr, nullptr, nullptr, some_aligned, some_aligned, nullptr,
                (flags & IEX_SDDMM_SUM_OVER_BATCH) != 0, (flags & IEX_SDDMM_ACCUMULATE) != 0};
  const bool any_order = (flags & IEX_SDDMM_ANY_COLUMN_ORDER) != 0;
  if (variant != 7 && sddmm_mfma_fits(dtype, p) && (variant == 3 || (!any_order && sddmm_mfma_wins(p)))) return sddmm_mfma_bytes(p);
  if (variant == 3) return 0;
  if (!sddmm_dense_fits(dtype, p)) return 0;
  if (variant == 0 && !sddmm_dense_wins(p)) return 0;
  return sddmm_dense_bytes(p);
}

int sddmm_dispatch(int dtype, int flags, int m, int k, int n, int nonzeros, const int* row_indices,
                   const int* row_offsets, const int* column_indices, const void* lhs, const void* rhs,
                   void* out, void* stream, int batch, void* workspace, size_t workspace_bytes) {
  IEX_REQUIRE(m >= 0 && k >= 0 && n >= 0 && nonzeros >= 0 && batch >= 0, IEX_ERR_BAD_ARGUMENT,
              "sddmm: negative dimension (m=%d k=%d n=%d nnz=%d batch=%d)", m, k, n, nonzeros, batch);
  trail_reset();
  if (m == 0 || nonzeros == 0 || batch == 0) return 0;
  IEX_REQUIRE(row_indices && row_offsets && column_indices && out, IEX_ERR_BAD_ARGUMENT,
              "sddmm: null pointer argument");
  IEX_REQUIRE(k == 0 || (lhs && rhs), IEX_ERR_BAD_ARGUMENT, "sddmm: null dense operand");
  IEX_REQUIRE(batch <= 65535, IEX_ERR_TOO_LARGE, "sddmm: batch %d exceeds 65535", batch);
  IEX_REQUIRE((long long)m * k < (1ll << 31) && (long long)n * k < (1ll << 31), IEX_ERR_TOO_LARGE,
              "sddmm: a dense operand exceeds 2^31 elements per batch entry");
  SddmmParams p{m, k, n, nonzeros, batch, row_indices, row_offsets, column_indices, lhs, rhs, out,
                (flags & IEX_SDDMM_SUM_OVER_BATCH) != 0, (flags & IEX_SDDMM_ACCUMULATE) != 0};
  int wpr = (flags >> 8) & 0xff;  // forced (1 or 4), else from the mean row length
  if (wpr != 1 && wpr != 4) wpr = ((double)nonzeros / m >= 64.0) ? 4 : 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int variant = (flags >> 16) & 0xf;  // 0 = choose, 1 = gather kernel, 3 = score tiles on the matrix cores, 7 = dense product then sampling
  const bool any_order = (flags & IEX_SDDMM_ANY_COLUMN_ORDER) != 0;   // (the tables of variant 3 assume ascending, distinct columns)
  if ((variant == 0 && !any_order) || variant == 3) {
    const bool fits = sddmm_mfma_fits(dtype, p);
    const bool room = workspace && aligned(workspace, 16) && workspace_bytes >= sddmm_mfma_bytes(p);
    if (variant == 3) {
      IEX_REQUIRE(fits, IEX_ERR_UNSUPPORTED, "sddmm: the matrix-core kernel needs fp16 / bf16, k = 32, 64 or 128, plain store, one output per batch entry and 16-byte aligned operands");
      IEX_REQUIRE(room, IEX_ERR_BAD_ARGUMENT, "sddmm: the matrix-core kernel needs a 16-byte aligned workspace of %zu bytes (iex_sddmm_ws)", sddmm_mfma_bytes(p));
    }
    if (fits && room && (variant == 3 || sddmm_mfma_wins(p))) return launch_sddmm_mfma(dtype, p, workspace, variant == 3 ? (flags >> 8) & 0xff : 0,
                                                                                 ((flags & IEX_SDDMM_TABLES_READY) ? 1 : 0) | ((flags & IEX_SDDMM_LISTS_READY) ? 2 : 0), s);
  }
  if (variant == 0 || variant == 7) {
    const bool fits = sddmm_dense_fits(dtype, p);
    const bool room = workspace && aligned(workspace, 16) && workspace_bytes >= sddmm_dense_bytes(p);
    if (variant == 7) {
      IEX_REQUIRE(fits, IEX_ERR_UNSUPPORTED, "sddmm: the dense-product path needs fp16 / bf16, plain store, one batch entry per output, k and n multiples of 8 and 16-byte aligned operands");
      IEX_REQUIRE(room, IEX_ERR_BAD_ARGUMENT, "sddmm: the dense-product path needs a 16-byte aligned workspace of %zu bytes (iex_sddmm_ws)", sddmm_dense_bytes(p));
    }
    if (fits && room && (variant == 7 || sddmm_dense_wins(p))) return launch_sddmm_dense(dtype, p, workspace, s);
  }
  switch (dtype) {
    case IEX_F32: return launch_typed<float>(p, wpr, s);
    case IEX_F16: return launch_typed<__half>(p, wpr, s);
    case IEX_BF16: return launch_typed<__hip_bfloat16>(p, wpr, s);
  }
  return fail(IEX_ERR_UNSUPPORTED, "sddmm: no kernel for dtype=%d", dtype);
}

}  // namespace iex

extern "C" {

int iex_sddmm_ex(int dtype, int flags, int m, int k, int n, int nonzeros, const int* row_indices,
                 const int* row_offsets, const int* column_indices, const void* lhs_matrix,
                 const void* rhs_matrix, void* output_values, void* stream, int batch) {
  return iex::sddmm_dispatch(dtype, flags, m, k, n, nonzeros, row_indices, row_offsets, column_indices,
                             lhs_matrix, rhs_matrix, output_values, stream, batch, nullptr, 0);
}

int iex_sddmm_ws(int dtype, int flags, int m, int k, int n, int nonzeros, const int* row_indices,
                 const int* row_offsets, const int* column_indices, const void* lhs_matrix,
                 const void* rhs_matrix, void* output_values, void* stream, int batch, void* workspace,
                 size_t workspace_bytes) {
  return iex::sddmm_dispatch(dtype, flags, m, k, n, nonzeros, row_indices, row_offsets, column_indices,
                             lhs_matrix, rhs_matrix, output_values, stream, batch, workspace, workspace_bytes);
}

size_t iex_sddmm_workspace_bytes(int dtype, int flags, int m, int k, int n, int nonzeros, int batch) {
  return iex::sddmm_workspace_bytes(dtype, flags, m, k, n, nonzeros, batch);
}

size_t iex_pattern_tables_bytes(int m, int n, int nonzeros) {
  using namespace iex;
  if (m <= 0 || n <= 0 || nonzeros <= 0) return 0;
  const int tiles = ceil_div(n, kSdBN);
  if (tiles > kSdMaxTiles || (long long)(tiles + 1) * m >= (1ll << 28)) return 0;
  return sb_words(m, tiles, nonzeros) * sizeof(int);
}

int iex_pattern_tables(int m, int n, int nonzeros, const int* row_offsets, const int* column_indices, void* workspace,
                       size_t workspace_bytes, void* stream) {
  using namespace iex;
  const size_t need = iex_pattern_tables_bytes(m, n, nonzeros);
  IEX_REQUIRE(need > 0, IEX_ERR_UNSUPPORTED, "pattern tables: needs m, n, nonzeros > 0 and n <= %d", kSdMaxTiles * kSdBN);
  IEX_REQUIRE(row_offsets && column_indices && workspace && aligned(workspace, 16) && workspace_bytes >= need, IEX_ERR_BAD_ARGUMENT,
              "pattern tables: null pointer, or the workspace is not 16-byte aligned or shorter than %zu bytes", need);
  trail_reset();
  const int tiles = ceil_div(n, kSdBN);
  return sb_setup(sd_tables(workspace, m, tiles), sb_lists(workspace, m, tiles, nonzeros), m, tiles, 0, 0, row_offsets, column_indices,
                  static_cast<hipStream_t>(stream));
}

int iex_sddmm_workspace_kind(int dtype, int flags, int m, int k, int n, int nonzeros, int batch) {
  return iex::sddmm_workspace_kind(dtype, flags, m, k, n, nonzeros, batch);
}

int iex_CudaSddmm2(int m, int k, int n, int nonzeros, const int* row_indices, const int* row_offsets,
                   const int* column_indices, const float* lhs_matrix, const float* rhs_matrix,
                   float* output_values, void* stream, int batch_size) {
  return iex::sddmm_dispatch(IEX_F32, IEX_SDDMM_SUM_OVER_BATCH | IEX_SDDMM_ANY_COLUMN_ORDER, m, k, n, nonzeros, row_indices,
                             row_offsets, column_indices, lhs_matrix, rhs_matrix, output_values, stream,
                             batch_size, nullptr, 0);
}

}  // extern "C"
