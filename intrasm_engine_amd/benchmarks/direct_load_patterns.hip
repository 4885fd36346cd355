// Per-CU rate of direct-to-LDS loads from L2 for the access patterns of the GEMM: rows of A (K-contiguous, 64 or 128 bytes
// per row and K step, row stride S) and k rows of B (512 bytes per k row, stride S).  32 CUs of an XCD share panels as the
// GEMM's 4 x 8 tile groups do.  All addresses stay inside the allocation (checked on the host).
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 intrasm_engine_amd/benchmarks/direct_load_patterns.hip -o direct_load_patterns
//   ./direct_load_patterns
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
__device__ __forceinline__ void dma16(const void* g, unsigned lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_base) : "memory", "m0");
}
struct Pat {
  int a_row_bytes;   // 64 or 128 (0 = no A loads)
  int a_wrap;        // bytes along a row after which the k position wraps
  int b_on;          // 1 = B loads
  int b_wrap_rows;   // k rows after which B wraps
  long long S;       // row stride in bytes (A rows and B k rows)
  long long a_panel_bytes, b_panel_bytes;
  int stagger;       // 1 = every workgroup starts at its own k position
};
template <int WAVES>
__global__ __launch_bounds__(WAVES * 64, 1) void k(const unsigned char* __restrict__ ga, const unsigned char* __restrict__ gb, unsigned* out, int iters, Pat p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const unsigned base = (unsigned)(size_t)smem;
  const int local = blockIdx.x / 8;            // index inside the XCD (ids are dealt round-robin to 8 XCDs)
  const int xcd = blockIdx.x % 8;
  const unsigned char* A = ga + ((size_t)xcd * 4 + local / 8) * p.a_panel_bytes;
  const unsigned char* B = gb + ((size_t)xcd * 8 + local % 8) * p.b_panel_bytes;
  // A: 256 rows per iteration; an instruction covers 1024 / a_row_bytes rows
  const int a_rpi = p.a_row_bytes ? 1024 / p.a_row_bytes : 1;
  const int a_instr = p.a_row_bytes ? 256 / a_rpi / WAVES : 0;      // per wave
  const int lanes_per_row = p.a_row_bytes / 16;
  int ka = p.stagger ? (blockIdx.x * 256) % p.a_wrap : 0, kb = p.stagger ? (blockIdx.x * 32) % p.b_wrap_rows : 0;
  for (int it = 0; it < iters; ++it) {
    for (int q = 0; q < a_instr; ++q) {
      const int row = (wave * a_instr + q) * a_rpi + lane / lanes_per_row;
      dma16(A + (size_t)row * p.S + ka + (lane % lanes_per_row) * 16, __builtin_amdgcn_readfirstlane(base + (wave * 8 + q) * 1024));
    }
    if (p.b_on) {
      for (int q = 0; q < 2; ++q) {   // 32 k rows of 512 bytes per iteration: 2 instructions per wave, 2 rows each
        const int kr = kb + (wave * 2 + q) * 2 + lane / 32;
        dma16(B + (size_t)kr * p.S + (lane % 32) * 16, __builtin_amdgcn_readfirstlane(base + (wave * 8 + 4 + q) * 1024));
      }
    }
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    ka += p.a_row_bytes; if (ka >= p.a_wrap) ka = 0;
    kb += 32; if (kb >= p.b_wrap_rows) kb = 0;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (iters < 0) out[tid] = *reinterpret_cast<unsigned*>(smem + tid * 4);
}
// The other way to feed A: every wavefront loads its operand fragments straight into registers in the MFMA layout (lane
// = row lane & 31 of a 32-row fragment, 16 bytes = 8 k values at k offset (lane >> 5) * 8), four fragments of 32 rows and
// two 16-k sub-steps per K step of 32, as a 128 x 64 register tile needs.  The four wavefronts that share a row panel
// (wn = 0 .. 3) load the same bytes.  Plain loads, results folded into a checksum so that they are not dropped.
__global__ __launch_bounds__(512, 1) void frag_kernel(const unsigned char* __restrict__ ga, unsigned* out, int iters, long long S, int wrap) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int local = blockIdx.x / 8, xcd = blockIdx.x % 8;
  const unsigned char* A = ga + ((size_t)xcd * 4 + local / 8) * (256 * S);   // a panel of 256 rows, shared by 8 CUs of the XCD
  const int wm = wave / 4;                                                    // rows 128 wm .. + 127
  uint4 sum = {0u, 0u, 0u, 0u};
  int k = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint4 v = *reinterpret_cast<const uint4*>(A + (size_t)(wm * 128 + i * 32 + (lane & 31)) * S + k + s * 32 + (lane >> 5) * 16);
        sum.x ^= v.x; sum.y += v.y; sum.z ^= v.z; sum.w += v.w;
      }
    k += 64; if (k >= wrap) k = 0;
  }
  if ((sum.x ^ sum.y ^ sum.z ^ sum.w) == 0x12345678u) out[tid] = sum.x;   // (never true for the fill pattern: keeps the loads)
}

int main() {
  unsigned char *ga, *gb; unsigned* out;
  const size_t abytes = (size_t)768 << 20, bbytes = (size_t)1536 << 20;
  if (hipMalloc(&ga, abytes) != hipSuccess || hipMalloc(&gb, bbytes) != hipSuccess) return 1;
  hipMalloc(&out, 1 << 16); hipMemset(ga, 1, abytes); hipMemset(gb, 1, bbytes);
  auto kern = k<8>;
  hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  const int iters = 4000;
  auto run = [&](const char* name, Pat p) {
    p.a_panel_bytes = 256 * p.S;                 // 256 rows
    p.b_panel_bytes = (long long)p.b_wrap_rows * p.S;
    // bounds: 32 A panels, 64 B panels
    if ((size_t)32 * p.a_panel_bytes > abytes || (size_t)64 * p.b_panel_bytes > bbytes || p.a_wrap > p.S || 512 > p.S) { printf("%s: does not fit\n", name); return; }
    hipEvent_t a, b; hipEventCreate(&a); hipEventCreate(&b);
    hipLaunchKernelGGL(kern, dim3(256), dim3(512), 160 * 1024, 0, ga, gb, out, 300, p);
    hipEventRecord(a);
    hipLaunchKernelGGL(kern, dim3(256), dim3(512), 160 * 1024, 0, ga, gb, out, iters, p);
    hipEventRecord(b); hipEventSynchronize(b);
    float ms; hipEventElapsedTime(&ms, a, b);
    const double bytes = (double)iters * ((p.a_row_bytes ? 256.0 * p.a_row_bytes : 0) + (p.b_on ? 32 * 512.0 : 0));
    printf("%-58s stride %6lld: %7.3f ms  %5.1f B/clk/CU (2.4 GHz)\n", name, p.S, ms, bytes / (ms * 1e-3 * 2.4e9)); fflush(stdout);
    if (hipGetLastError() != hipSuccess) { printf("error\n"); exit(1); }
  };
  for (long long S : {16384ll, 8192ll, 22016ll}) {
    if ((size_t)32 * 256 * S > abytes) continue;
    hipEvent_t a, b; hipEventCreate(&a); hipEventCreate(&b);
    hipLaunchKernelGGL(frag_kernel, dim3(256), dim3(512), 0, 0, ga, out, 300, S, 2048);
    hipEventRecord(a);
    hipLaunchKernelGGL(frag_kernel, dim3(256), dim3(512), 0, 0, ga, out, iters, S, 2048);
    hipEventRecord(b); hipEventSynchronize(b);
    float ms; hipEventElapsedTime(&ms, a, b);
    // per K step of 32 and CU: 8 wavefronts x 4 fragments x 2 sub-steps x 1 KB = 64 KB into registers (16 KB distinct)
    printf("%-58s stride %6lld: %7.3f ms  %5.1f B/clk/CU into registers (2.4 GHz), %5.0f clk per K step of 32\n",
           "A fragments straight into registers (128 x 64 tiles)", S, ms, (double)iters * 65536.0 / (ms * 1e-3 * 2.4e9), ms * 1e-3 * 2.4e9 / iters);
    fflush(stdout);
    if (hipGetLastError() != hipSuccess) { printf("error\n"); return 1; }
  }
  for (long long S : {16384ll, 16384ll + 128, 16384ll + 512, 8192ll, 22016ll}) {
    run("A 64 B/row (16 rows per instruction)", Pat{64, 2048, 0, 256, S, 0, 0, 0});
    run("A 128 B/row (8 rows per instruction)", Pat{128, 2048, 0, 256, S, 0, 0, 0});
    run("B 512 B per k row", Pat{0, 2048, 1, 256, S, 0, 0, 0});
    run("A 64 B/row + B (the GEMM's K step: 32 KB)", Pat{64, 2048, 1, 256, S, 0, 0, 0});
    run("A 64 B/row + B, staggered k", Pat{64, 2048, 1, 256, S, 0, 0, 1});
  }
  return 0;
}
