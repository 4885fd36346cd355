// Error reporting, version and handle round-trip entry points of libiex_hip.so.
#include "iex_common.h"

#include <cstring>

namespace iex {

char* last_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(last_error_buffer(), 512, fmt, ap);
  va_end(ap);
  return code;
}

static char* trail_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

void trail_reset() { trail_buffer()[0] = 0; }

void note_kernel(const char* fmt, ...) {
  char* buf = trail_buffer();
  size_t used = std::strlen(buf);
  if (used > 0 && used + 4 < 512) {
    std::memcpy(buf + used, " + ", 4);
    used += 3;
  }
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf + used, 512 - used, fmt, ap);
  va_end(ap);
}

int check_hip(hipError_t err, const char* what) {
  if (err == hipSuccess) return 0;
  snprintf(last_error_buffer(), 512, "%s: %s (hipError_t %d)", what, hipGetErrorString(err), (int)err);
  return (int)err;
}

}  // namespace iex

namespace {
// Plain streaming copy, 128 bits per lane per step, grid-stride.
__global__ __launch_bounds__(256) void copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

// What is wrong with a CSR pattern, as bits ORed into *status: one wavefront per row.
template <typename IT>
__global__ __launch_bounds__(256) void csr_check_kernel(int m, int k, int nnz, const int* __restrict__ row_offsets, const IT* __restrict__ cols,
                                                        int* status) {
  const int lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= m) return;
  const int s = row_offsets[r], e = row_offsets[r + 1];
  int bad = 0;
  if (s < 0 || e < s || e > nnz || (r == 0 && s != 0) || (r == m - 1 && e != nnz)) bad |= IEX_CSR_BAD_OFFSETS;
  if (!bad) {
    // 256 columns per step (four loads in flight); a column's left neighbour comes from the lane before, the last
    // lane of the chunk before, or -- across steps -- the carried last column of the step before
    int carry = 0;
    for (int base = s; base < e; base += 256) {
      int c[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = base + u * 64 + lane;
        c[u] = j < e ? (int)cols[j] : 0;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (base + u * 64 >= e) break;   // (uniform)
        const int j = base + u * 64 + lane;
        int before = __shfl_up(c[u], 1, 64);
        const int chunk_before = u == 0 ? carry : __builtin_amdgcn_readlane(c[u > 0 ? u - 1 : 0], 63);
        if (lane == 0) before = chunk_before;
        if (j < e) {
          if (c[u] < 0 || c[u] >= k) bad |= IEX_CSR_COLUMN_OUT_OF_RANGE;
          if (j > s && before >= c[u]) bad |= IEX_CSR_NOT_ASCENDING;
        }
      }
      carry = __builtin_amdgcn_readlane(c[3], 63);
    }
  }
  if (bad) atomicOr(status, bad);
}

// histogram[j] += rows with more than 64 << j nonzeros, j = 0 .. 15 (counts: integer additions commute, so the result
// does not depend on the order of the atomics); a thread per row, a workgroup adds up in LDS first.
__global__ __launch_bounds__(256) void csr_row_histogram_kernel(int m, const int* __restrict__ row_offsets, int* histogram) {
  __shared__ int local[16];
  if (threadIdx.x < 16) local[threadIdx.x] = 0;
  __syncthreads();
  const int r = blockIdx.x * 256 + threadIdx.x;
  if (r < m) {
    const long long len = (long long)row_offsets[r + 1] - row_offsets[r];
    for (int j = 0; j < 16 && len > (64ll << j); ++j) atomicAdd(&local[j], 1);
  }
  __syncthreads();
  if (threadIdx.x < 16 && local[threadIdx.x]) atomicAdd(&histogram[threadIdx.x], local[threadIdx.x]);
}

// *dense_nonzeros += the nonzeros of this block of 128 rows that sit in 128 x 128 blocks holding at least dense_min of
// them.  `parts` workgroups (16 wavefronts each) per 128 rows; the counters of the row block's column blocks live in
// LDS.  Which row a nonzero belongs to does not matter inside a row block, so the block's nonzeros -- one contiguous
// stretch of the column array -- are dealt to the workgroups and their wavefronts in equal contiguous shares, whatever
// the row lengths; a wavefront takes 512 of them per step (eight loads in flight, the next step's loads issued before
// this step's are counted).  Neighbours that fall into the same column block (in runs, when the columns ascend) are
// counted by the first lane of their run, so a run costs one LDS atomic, not one per nonzero.  Any column order gives
// the same counts.  With parts > 1 the workgroups of a row block add their counters into block_counts[row block][tile]
// (zero at launch) and take a ticket from done[row block] (zero at launch); the one that draws the last ticket finds
// every sum complete and compares them with dense_min.
constexpr int kShareMaxTiles = 512;   // k <= 65536
constexpr int kShareThreads = 1024;
constexpr int kShareLoads = 8;
constexpr int kShareMaxParts = 32;
template <typename IT>
__global__ __launch_bounds__(kShareThreads) void csr_dense_share_kernel(int m, int k, int nnz, const int* __restrict__ row_offsets, const IT* __restrict__ cols,
                                                                        int dense_min, int* dense_nonzeros, int parts, int* block_counts, int* done) {
  __shared__ int count[kShareMaxTiles];
  __shared__ int total;
  __shared__ int ticket;
  const int tiles = (k + 127) / 128;
  for (int t = threadIdx.x; t < tiles; t += kShareThreads) count[t] = 0;
  if (threadIdx.x == 0) total = 0;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row_block = (int)blockIdx.x / parts, part = (int)blockIdx.x % parts;
  const int row0 = row_block * 128;
  // (offsets that point outside the arrays are cut to them: the kernel may run before anybody has checked the pattern)
  const int first = min(max(row_offsets[row0], 0), nnz);
  const int last = min(max(row_offsets[min(m, row0 + 128)], first), nnz);
  const int share = ((last - first + kShareThreads * parts - 1) / (kShareThreads * parts)) * 64;   // whole chunks of 64 per wavefront
  const int begin = min(first + (part * (kShareThreads / 64) + wave) * share, last), end = min(begin + share, last);
  auto fetch = [&](int base, int (&t)[kShareLoads]) {
#pragma unroll
    for (int u = 0; u < kShareLoads; ++u) {
      const int j = base + u * 64 + lane;
      t[u] = -1;   // (no nonzero here, or a column outside the matrix: counted nowhere)
      if (j < end) {
        const int c = (int)cols[j];
        if (c >= 0 && c < k) t[u] = c >> 7;
      }
    }
  };
  int cur[kShareLoads], next[kShareLoads];
  if (begin < end) fetch(begin, cur);
  for (int base = begin; base < end; base += 64 * kShareLoads) {
    if (base + 64 * kShareLoads < end) fetch(base + 64 * kShareLoads, next);   // (uniform)
#pragma unroll
    for (int u = 0; u < kShareLoads; ++u) {
      if (base + u * 64 >= end) break;   // (uniform)
      const int t = cur[u];
      const int before = __shfl_up(t, 1, 64);
      const unsigned long long heads = __ballot(lane == 0 || t != before);
      if ((heads >> lane) & 1ull) {
        const unsigned long long later = lane == 63 ? 0ull : heads >> (lane + 1);
        const int run = later ? __builtin_ctzll(later) + 1 : 64 - lane;
        if (t >= 0) atomicAdd(&count[t], run);
      }
    }
#pragma unroll
    for (int u = 0; u < kShareLoads; ++u) cur[u] = next[u];
  }
  __syncthreads();
  int mine = 0;
  if (parts == 1) {
    for (int t = threadIdx.x; t < tiles; t += kShareThreads) mine += count[t] >= dense_min ? count[t] : 0;
  } else {
    int* sums = block_counts + (size_t)row_block * tiles;
    // Device-scope atomics are carried out where all XCDs see them, and one that returns the old value has been carried
    // out when that value is back: once every wavefront has waited for its own and the barrier has collected them, the
    // ticket may be drawn.  (A device-scope fence here instead writes back the L2 of the XCD under everybody else:
    // measured 150 us for the kernel whatever the pattern.)
    int seen = 0;
    for (int t = threadIdx.x; t < tiles; t += kShareThreads)
      if (count[t]) seen ^= atomicAdd(&sums[t], count[t]);
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(seen) : : "memory");
    __syncthreads();
    if (threadIdx.x == 0) ticket = atomicAdd(&done[row_block], 1);
    __syncthreads();
    if (ticket != parts - 1) return;   // (uniform)
    for (int t = threadIdx.x; t < tiles; t += kShareThreads) {
      const int sum = __hip_atomic_load(&sums[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      mine += sum >= dense_min ? sum : 0;
    }
  }
  if (mine) atomicAdd(&total, mine);
  __syncthreads();
  if (threadIdx.x == 0 && total) atomicAdd(dense_nonzeros, total);
}

// Workgroups per block of 128 rows: enough for two per CU, as far as the scratch memory reaches.
inline int dense_share_parts(int m, int k, const void* scratch, size_t scratch_bytes) {
  const int row_blocks = (m + 127) / 128, tiles = (k + 127) / 128;
  if (!scratch || row_blocks == 0 || scratch_bytes < (size_t)row_blocks * (tiles + 1) * sizeof(int)) return 1;
  return std::min(kShareMaxParts, std::max(1, 512 / row_blocks));
}
}  // namespace

extern "C" {

int iex_csr_dense_share(int itype, int m, int k, int nonzeros, const int* row_offsets, const void* column_indices, int dense_min,
                        int* dense_nonzeros, void* scratch, size_t scratch_bytes, void* stream) {
  IEX_REQUIRE(m >= 0 && k >= 0 && nonzeros >= 0 && dense_min >= 0, IEX_ERR_BAD_ARGUMENT, "csr_dense_share: negative argument");
  IEX_REQUIRE(dense_nonzeros && (m == 0 || (row_offsets && column_indices)), IEX_ERR_BAD_ARGUMENT, "csr_dense_share: null pointer argument");
  IEX_REQUIRE(itype == IEX_I32 || itype == IEX_I16, IEX_ERR_UNSUPPORTED, "csr_dense_share: column indices must be int32 or int16");
  IEX_REQUIRE(k <= 128 * kShareMaxTiles, IEX_ERR_TOO_LARGE, "csr_dense_share: more than %d columns", 128 * kShareMaxTiles);
  IEX_REQUIRE(!scratch || iex::aligned(scratch, 4), IEX_ERR_BAD_ARGUMENT, "csr_dense_share: scratch memory must be 4-byte aligned");
  if (m == 0 || k == 0 || nonzeros == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int row_blocks = (m + 127) / 128, tiles = (k + 127) / 128;
  const int parts = dense_share_parts(m, k, scratch, scratch_bytes);
  int* block_counts = static_cast<int*>(scratch);
  int* done = block_counts ? block_counts + (size_t)row_blocks * tiles : nullptr;
  if (itype == IEX_I32)
    hipLaunchKernelGGL(csr_dense_share_kernel<int>, dim3(row_blocks * parts), dim3(kShareThreads), 0, s, m, k, nonzeros, row_offsets, static_cast<const int*>(column_indices), dense_min, dense_nonzeros, parts, block_counts, done);
  else
    hipLaunchKernelGGL(csr_dense_share_kernel<short>, dim3(row_blocks * parts), dim3(kShareThreads), 0, s, m, k, nonzeros, row_offsets, static_cast<const short*>(column_indices), dense_min, dense_nonzeros, parts, block_counts, done);
  return iex::check_hip(hipGetLastError(), "csr_dense_share launch");
}

size_t iex_csr_dense_share_scratch_bytes(int m, int k) {
  if (m <= 0 || k <= 0) return 0;
  const size_t row_blocks = ((size_t)m + 127) / 128, tiles = ((size_t)k + 127) / 128;
  return row_blocks >= 512 ? 0 : row_blocks * (tiles + 1) * sizeof(int);   // (512 row blocks fill the chip by themselves)
}

int iex_csr_check(int itype, int m, int k, int nonzeros, const int* row_offsets, const void* column_indices, int* status, void* stream) {
  IEX_REQUIRE(m >= 0 && k >= 0 && nonzeros >= 0, IEX_ERR_BAD_ARGUMENT, "csr_check: negative dimension");
  IEX_REQUIRE(status && (m == 0 || row_offsets) && (nonzeros == 0 || column_indices), IEX_ERR_BAD_ARGUMENT, "csr_check: null pointer argument");
  IEX_REQUIRE(itype == IEX_I32 || itype == IEX_I16, IEX_ERR_UNSUPPORTED, "csr_check: column indices must be int32 or int16");
  if (m == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (itype == IEX_I32)
    hipLaunchKernelGGL(csr_check_kernel<int>, dim3((m + 3) / 4), dim3(256), 0, s, m, k, nonzeros, row_offsets, static_cast<const int*>(column_indices), status);
  else
    hipLaunchKernelGGL(csr_check_kernel<short>, dim3((m + 3) / 4), dim3(256), 0, s, m, k, nonzeros, row_offsets, static_cast<const short*>(column_indices), status);
  return iex::check_hip(hipGetLastError(), "csr_check launch");
}

int iex_csr_row_histogram(int m, const int* row_offsets, int* histogram, void* stream) {
  IEX_REQUIRE(m >= 0, IEX_ERR_BAD_ARGUMENT, "csr_row_histogram: negative dimension");
  IEX_REQUIRE(histogram && (m == 0 || row_offsets), IEX_ERR_BAD_ARGUMENT, "csr_row_histogram: null pointer argument");
  if (m == 0) return 0;
  hipLaunchKernelGGL(csr_row_histogram_kernel, dim3((m + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream), m, row_offsets, histogram);
  return iex::check_hip(hipGetLastError(), "csr_row_histogram launch");
}

int iex_copy_bytes(void* dst, const void* src, size_t nbytes, void* stream) {
  IEX_REQUIRE(dst && src, IEX_ERR_BAD_ARGUMENT, "copy: null pointer argument");
  IEX_REQUIRE(nbytes % 16 == 0 && iex::aligned(dst, 16) && iex::aligned(src, 16), IEX_ERR_UNSUPPORTED,
              "copy: size and pointers must be multiples of 16 bytes");
  if (nbytes == 0) return 0;
  const size_t n16 = nbytes / 16;
  const int blocks = (int)((n16 + 255) / 256 < 256 * 64 ? (n16 + 255) / 256 : 256 * 64);
  hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<uint4*>(dst),
                     static_cast<const uint4*>(src), n16);
  return iex::check_hip(hipGetLastError(), "copy launch");
}

int iex_abi_version(void) { return IEX_ABI_VERSION; }

const char* iex_last_error(void) { return iex::last_error_buffer(); }

const char* iex_last_kernels(void) { return iex::trail_buffer(); }

int iex_device_ok(void) {
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return 0;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return 0;
  return std::strncmp(prop.gcnArchName, "gfx950", 6) == 0 ? 1 : 0;
}

long long iex_echo_stream(void* stream) {
  hipError_t err = hipStreamQuery(static_cast<hipStream_t>(stream));
  if (err != hipSuccess && err != hipErrorNotReady) {
    iex::check_hip(err, "hipStreamQuery");
    return -1;
  }
  return (long long)reinterpret_cast<intptr_t>(stream);
}

long long iex_echo_event(void* event) {
  if (event == nullptr) {
    iex::fail(IEX_ERR_BAD_ARGUMENT, "event handle is null (record the event once before passing it)");
    return -1;
  }
  hipError_t err = hipEventQuery(static_cast<hipEvent_t>(event));
  if (err != hipSuccess && err != hipErrorNotReady) {
    iex::check_hip(err, "hipEventQuery");
    return -1;
  }
  return (long long)reinterpret_cast<intptr_t>(event);
}

}  // extern "C"
