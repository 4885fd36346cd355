// Host side of the SpMM for attention-like sparse operands (spmm_blocks_device.cuh): what it serves, how much
// workspace it needs, the launch.
#include "spmm_blocks_device.cuh"
#include "spmm_device.cuh"

namespace iex {

// fp16 / bf16, int32 indices, output columns a multiple of 64 (served in slices of 64), plain store without bias or ReLU.
bool spmm_blocks_fits(int dtype, int itype, const SpmmParams& p) {
  return (dtype == IEX_F16 || dtype == IEX_BF16) && itype == IEX_I32 && p.n >= kSbN && p.n % kSbN == 0 && p.n <= 1024 && !p.accumulate && !p.relu && !p.bias &&
         aligned(p.dense, 16) && aligned(p.out, 16) && ceil_div(p.k, kSdBN) <= kSdMaxTiles &&
         (long long)(ceil_div(p.k, kSdBN) + 1) * p.m < (1ll << 28);
}

// The host does not look at the pattern, so where nothing is forced the choice goes by the overall density, and only
// for values per batch entry (attention probabilities: masks with structure).  Measured on MI355X (fp16, 16 batch
// entries of 4096 x 4096, n = 64, microseconds, row kernel / this kernel with its two setup kernels / with tables
// and lists kept; bench.py, extras.spmm_fp16_16heads_by_mask):
//   band of 256 + 32 scattered per row (7 %)   94 /  48 /  35     band of 512 + 32 (13 %)        175 /  65 /  48
//   band of 128 + 16 scattered (3.5 %)          62 /  41 /  31     block diagonal 256 (6 %)        83 /  32 /  20
//   causal window of 512 (12 %)                149 /  47 /  32
//   equal rows, columns at random:  1 %  40 (stays on the row kernel)    5 %  78 / 106 / 93
//                                  10 % 142 / 154 / 141                 20 % 265 / 149 / 134
// Masks with structure gain 1.5x to 3x from 3 % up; a mask without any loses up to 1.4x between 3 and 10 %.
// IEX_SPMM_FORCE_VARIANT(1) keeps the row kernel.
bool spmm_blocks_wins(const SpmmParams& p, int batch) {
  const double density = (double)p.nnz / ((double)p.m * p.k);
  return p.per_batch_values && p.nnz >= 8 && density >= 0.03 && (double)batch * p.m * p.k >= 32.0 * 1024 * 1024;
}

size_t spmm_blocks_bytes(const SpmmParams& p) { return sb_words(p.m, ceil_div(p.k, kSdBN), p.nnz) * sizeof(int); }

template <bool BF16>
static int launch_blocks(const SpmmBlocksParams& q, int batch, hipStream_t stream) {
  constexpr int lds = spmm_blocks_lds_bytes();
  auto kernel = spmm_blocks_kernel<BF16>;
  static thread_local bool raised = false;   // per instantiation: more than 64 KB of dynamic LDS
  if (!raised) {
    if (int rc = check_hip(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds),
                           "hipFuncSetAttribute(LDS size)"))
      return rc;
    raised = true;
  }
  note_kernel("spmm_blocks_kernel<%s>", BF16 ? "true" : "false");
  hipLaunchKernelGGL(kernel, dim3(ceil_div(q.m, kSdBM), batch * (q.n / kSbN)), dim3(kSdThreads), lds, stream, q);
  return check_hip(hipGetLastError(), "spmm (dense blocks) launch");
}

// dense_code (for tests and tuning): 0 = the built-in threshold, 1 = every tile on the matrix cores, 255 = none,
// else 64 * code nonzeros per 128 x 128 block.  ready: bit 0 = the caller vouches that an earlier call on this
// pattern (this kernel's or the SDDMM's for masks with structure: same tables) left the tables in the workspace,
// bit 1 = that an earlier call of this kernel with the same dense_code left its lists there too.
int launch_spmm_blocks(int dtype, const SpmmParams& p, int batch, void* ws, int dense_code, int ready, hipStream_t stream) {
  IEX_REQUIRE((long long)batch * (p.n / kSbN) <= 65535, IEX_ERR_TOO_LARGE, "spmm: batch %d x %d column slices exceed 65535", batch, p.n / kSbN);
  const int tiles_k = ceil_div(p.k, kSdBN);
  const SdTables t = sd_tables(ws, p.m, tiles_k);
  const SbLists l = sb_lists(ws, p.m, tiles_k, p.nnz);
  const int* cols = static_cast<const int*>(p.cols);
  if (int rc = sb_setup(t, l, p.m, tiles_k, dense_code, ready, p.row_offsets, cols, stream)) return rc;
  SpmmBlocksParams q{p.m, p.k, p.nnz, p.row_offsets, p.values, p.per_batch_values ? (size_t)p.nnz : 0, p.dense, p.out, p.n,
                     t.mask, t.tile_ptr, t.brief, tiles_k, l.zeros, l.thin_ent, l.thin_cnt, l.dense_list};
  return dtype == IEX_BF16 ? launch_blocks<true>(q, batch, stream) : launch_blocks<false>(q, batch, stream);
}

}  // namespace iex
