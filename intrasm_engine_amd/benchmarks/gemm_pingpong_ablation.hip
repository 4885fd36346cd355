// Ablation of the main loop of the ping-pong GEMM tile (csrc/gemm_pp_device.cuh: eight wavefronts in two groups that
// alternate between "read fragments + issue direct loads" and "MFMA") on bf16 products with B as (K, N): the 4-wave
// 256 x 256 tile of gemm_dma_device.cuh, the ping-pong tile, the same with both groups in phase, and builds that leave
// one ingredient out each (results of those are wrong on purpose).  25 warm-up launches (the first launches after an
// idle period run at another clock and mislead by 10 % and more), then TFLOP/s from HIP events over 60 launches, twice.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         intrasm_engine_amd/benchmarks/gemm_pingpong_ablation.hip -o gemm_pingpong_ablation
//   ./gemm_pingpong_ablation [M N K [only_this_line [data: 0 = normal, 1 = zeros, 2 = small integers [batch]]]]
// Built with -DIEX_DMA_MOD='" sc0"' (or " sc1", " nt", " sc0 sc1") the direct loads carry that cache modifier.
#include "gemm_pingpong_ablation_device.cuh"
#include "../csrc/gemm_pp_device.cuh"
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <random>
using namespace iex;
namespace iex {
char* last_error_buffer() { static char b[512]; return b; }
int fail(int code, const char*, ...) { return code; }
int check_hip(hipError_t e, const char*) { return (int)e; }
}
template <bool TB, int WM, int WN, int WCN, int BK, int ST>
__global__ __launch_bounds__(WCN * 128, 1) void ref_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  int tm, tn;
  if (!xcd_tile(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn)) return;
  gemm_tile_dma<true, TB, WM, WN, WCN, BK, ST>(p, tm, tn, blockIdx.y, smem);
}
template <bool TB, int WM, int WN, int WCN, int BK, int ST, int GM, int DBG>
__global__ __launch_bounds__(WCN * 128, 1) void ppx_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  int tm, tn;
  if (!xcd_tile(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn)) return;
  gemm_tile_ppx<true, TB, WM, WN, WCN, BK, ST, GM, DBG>(p, tm, tn, blockIdx.y, smem);
}
template <bool TB, int WM, int WN, int WCN>
__global__ __launch_bounds__(WCN * 128, 1) void pp_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  int tm, tn;
  if (!xcd_tile(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn)) return;
  gemm_tile_pp<true, TB, WM, WN, WCN>(p, tm, tn, blockIdx.y, smem);
}
static int g_batch = 1;
template <typename K>
static double timeit(K kern, GemmParams p, int BM, int BN, int threads, int lds, int reps = 60) {
  hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int per_xcd = (p.tiles_m * p.tiles_n + kXcds - 1) / kXcds;
  hipEvent_t a, b;
  hipEventCreate(&a); hipEventCreate(&b);
  for (int i = 0; i < 25; ++i) hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds, g_batch), dim3(threads), lds, 0, p);
  hipEventRecord(a);
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds, g_batch), dim3(threads), lds, 0, p);
  hipEventRecord(b);
  hipEventSynchronize(b);
  float ms = 0;
  hipEventElapsedTime(&ms, a, b);
  if (hipGetLastError() != hipSuccess) return -1.0;
  return 2.0 * g_batch * p.M * p.N * p.K / (ms / reps * 1e-3) / 1e12;
}
static unsigned short f2bf(float f) { unsigned u; memcpy(&u, &f, 4); u += 0x7fff + ((u >> 16) & 1); return (unsigned short)(u >> 16); }

int main(int argc, char** argv) {
  const int M = argc > 1 ? atoi(argv[1]) : 8192, N = argc > 2 ? atoi(argv[2]) : 8192, K = argc > 3 ? atoi(argv[3]) : 8192;
  const int only = argc > 4 ? atoi(argv[4]) : -1;
  const int mode = argc > 5 ? atoi(argv[5]) : 0;
  g_batch = argc > 6 ? atoi(argv[6]) : 1;
  std::mt19937 rng(1); std::normal_distribution<float> nd(0.f, 1.f);
  std::vector<unsigned short> ha((size_t)M * K), hb((size_t)K * N);
  for (auto& x : ha) x = mode == 1 ? 0 : mode == 2 ? f2bf((float)((int)(rng() % 5) - 2)) : f2bf(nd(rng));
  for (auto& x : hb) x = mode == 1 ? 0 : mode == 2 ? f2bf((float)((int)(rng() % 5) - 2)) : f2bf(nd(rng));
  unsigned short *A, *B, *C;
  hipMalloc(&A, ha.size() * 2); hipMalloc(&B, hb.size() * 2); hipMalloc(&C, (size_t)M * N * 2 * g_batch);
  hipMemcpy(A, ha.data(), ha.size() * 2, hipMemcpyHostToDevice);
  hipMemcpy(B, hb.data(), hb.size() * 2, hipMemcpyHostToDevice);
  GemmParams p{M, N, K, A, B, C, 0, 0, (long long)M * N, 0, 0};
  printf("== %d x %d x %d  B as (K,N) data mode %d\n", M, N, K, mode); fflush(stdout);
  constexpr int L = gemm_dma_lds_bytes<4, 2, 4, 32, 4>();
  for (int round = 0; round < 2; ++round) {
  int id = 0;
  // (builds that leave nothing out must give the bits of the 4-wave tile: RUNC compares the output with line 0's)
  static std::vector<unsigned short> ref_c;
  auto mismatches = [&]() {
    std::vector<unsigned short> c((size_t)M * N);
    hipMemcpy(c.data(), C, c.size() * 2, hipMemcpyDeviceToHost);
    if (ref_c.empty()) { ref_c = c; return 0ll; }
    long long bad = 0;
    for (size_t i = 0; i < c.size(); ++i) bad += c[i] != ref_c[i];
    return bad;
  };
#define RUNC(name, expr) do { if (only < 0 || only == id) { hipMemset(C, 0xff, (size_t)M * N * 2); double t = (expr); printf("  [%2d] %-44s %7.0f   mismatches %lld\n", id, name, t, mismatches()); fflush(stdout);} ++id; } while (0)
#define RUN(name, expr) do { if (only < 0 || only == id) { double t = (expr); printf("  [%2d] %-44s %7.0f\n", id, name, t); fflush(stdout);} ++id; } while (0)
  RUNC("shipped 256x256 / 4 waves", timeit(ref_kernel<false, 4, 4, 2, 32, 4>, p, 256, 256, 256, gemm_dma_lds_bytes<4, 4, 2, 32, 4>()));
  RUNC("ping-pong 256x256", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 0>, p, 256, 256, 512, L));
  RUN("pp: no direct loads in loop", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 1>, p, 256, 256, 512, L));
  RUN("pp: fragments read once", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 2>, p, 256, 256, 512, L));
  RUN("pp: neither (MFMA + barriers)", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 3>, p, 256, 256, 512, L));
  RUN("pp: no A loads", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 16>, p, 256, 256, 512, L));
  RUN("pp: no B loads", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 32>, p, 256, 256, 512, L));
  RUN("in phase: as is", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 2, 0>, p, 256, 256, 512, L));
  RUN("in phase: no direct loads", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 2, 1>, p, 256, 256, 512, L));
  RUN("in phase: neither", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 2, 3>, p, 256, 256, 512, L));
  RUN("pp: loads issued, never waited for", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 64>, p, 256, 256, 512, L));
  RUN("pp: 5 stages (160 KB)", timeit(ppx_kernel<false, 4, 2, 4, 32, 5, 0, 0>, p, 256, 256, 512, gemm_dma_lds_bytes<4, 2, 4, 32, 5>()));
  RUN("pp: 3 stages", timeit(ppx_kernel<false, 4, 2, 4, 32, 3, 0, 0>, p, 256, 256, 512, gemm_dma_lds_bytes<4, 2, 4, 32, 3>()));
  RUN("pp: 3 stages, no waits", timeit(ppx_kernel<false, 4, 2, 4, 32, 3, 0, 64>, p, 256, 256, 512, gemm_dma_lds_bytes<4, 2, 4, 32, 3>()));
  RUN("pp: all loads from one L1-resident 16 KB", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 128>, p, 256, 256, 512, L));
  RUNC("pp: B through registers, A direct", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 256>, p, 256, 256, 512, L));
  RUNC("pp: A through registers, B direct", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 512>, p, 256, 256, 512, L));
  RUNC("pp: A and B through registers", timeit(ppx_kernel<false, 4, 2, 4, 32, 4, 0, 768>, p, 256, 256, 512, L));
  RUNC("pp: K steps of 64, two stages of 64 KB", timeit(ppx_kernel<false, 4, 2, 4, 64, 2, 0, 0>, p, 256, 256, 512, gemm_dma_lds_bytes<4, 2, 4, 64, 2>()));
  RUNC("pp, A in 64-k stages (3) + B 32-k (4)", timeit(pp_kernel<false, 4, 2, 4>, p, 256, 256, 512, gemm_pp_lds_bytes<true, false, 4, 2, 4>()));
  }
  return 0;
}
