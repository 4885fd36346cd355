// Ablation of the main loop of the direct-load GEMM (gemm_dma_device.cuh) on bf16 products with B as (K, N): the kernel
// as shipped, and instrumented builds of a copy of its tile routine that leave out one ingredient each (the DBG switches of
// gemm_tile_dma_ablation, gemm_loop_ablation_device.cuh; results of those builds are wrong on purpose, every address they use stays in bounds).  Prints
// TFLOP/s from HIP events over 10 launches, for 256 x 256 tiles by four waves and 128 x 256 tiles by eight.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         intrasm_engine_amd/benchmarks/gemm_loop_ablation.hip -o gemm_loop_ablation && ./gemm_loop_ablation
#include "gemm_loop_ablation_device.cuh"

#include <cstdio>
#include <cstdlib>
#include <vector>

using namespace iex;
namespace iex {   // the three symbols of core.hip that the device headers declare
char* last_error_buffer() { static char b[512]; return b; }
int fail(int code, const char*, ...) { return code; }
int check_hip(hipError_t e, const char*) { return (int)e; }
}  // namespace iex

template <int WM, int WN, int WCN, int DBG>
__global__ __launch_bounds__(WCN * 128, 1) void ablation_kernel(GemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  int tile_m, tile_n;
  if (!xcd_tile(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n)) return;
  gemm_tile_dma_ablation<true, false, WM, WN, WCN, 32, 4, false, DBG>(p, tile_m, tile_n, blockIdx.y, smem);
}

template <int WM, int WN, int WCN, int DBG>
static double run(GemmParams p, int reps = 10) {
  constexpr int BM = 2 * WM * 32, BN = WCN * WN * 32;
  constexpr int lds = gemm_dma_lds_bytes<WM, WN, WCN, 32, 4>();
  auto kern = ablation_kernel<WM, WN, WCN, DBG>;
  hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  p.tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int per_xcd = (p.tiles_m * p.tiles_n + kXcds - 1) / kXcds;
  hipEvent_t a, b;
  hipEventCreate(&a);
  hipEventCreate(&b);
  for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds, 1), dim3(WCN * 128), lds, 0, p);
  hipEventRecord(a);
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(kern, dim3(per_xcd * kXcds, 1), dim3(WCN * 128), lds, 0, p);
  hipEventRecord(b);
  hipEventSynchronize(b);
  float ms = 0;
  hipEventElapsedTime(&ms, a, b);
  if (hipGetLastError() != hipSuccess) return -1.0;
  return 2.0 * p.M * p.N * p.K / (ms / reps * 1e-3) / 1e12;
}

template <int WM, int WN, int WCN>
static void table(const char* tile, const GemmParams& p) {
  printf("%d x %d x %d, %s (TFLOP/s)\n", p.M, p.N, p.K, tile);
  printf("  as shipped                                              %6.0f\n", run<WM, WN, WCN, 0>(p));
  printf("  no direct loads after the prologue (LDS keeps 3 tiles)   %6.0f\n", run<WM, WN, WCN, 1>(p));
  printf("  address arithmetic of the direct loads, no loads        %6.0f\n", run<WM, WN, WCN, 8>(p));
  printf("  no barrier per K step                                   %6.0f\n", run<WM, WN, WCN, 2>(p));
  printf("  no fragment reads from LDS                              %6.0f\n", run<WM, WN, WCN, 4>(p));
  printf("  no direct loads and no fragment reads                   %6.0f\n", run<WM, WN, WCN, 5>(p));
  printf("  nothing but the MFMAs (none of the three)               %6.0f\n", run<WM, WN, WCN, 7>(p));
}

int main() {
  const int shapes[2][3] = {{8192, 8192, 8192}, {4096, 2048, 4096}};
  for (const auto& sh : shapes) {
    const int M = sh[0], N = sh[1], K = sh[2];
    std::vector<unsigned short> ha((size_t)M * K), hb((size_t)K * N);
    for (size_t i = 0; i < ha.size(); ++i) ha[i] = 0x3c00 + (unsigned short)(rand() & 0xff);   // bf16 values near 0.01
    for (size_t i = 0; i < hb.size(); ++i) hb[i] = 0x3c00 + (unsigned short)(rand() & 0xff);
    unsigned short *A = nullptr, *B = nullptr, *C = nullptr;
    if (hipMalloc(&A, ha.size() * 2) != hipSuccess || hipMalloc(&B, hb.size() * 2) != hipSuccess || hipMalloc(&C, (size_t)M * N * 2) != hipSuccess) return 1;
    hipMemcpy(A, ha.data(), ha.size() * 2, hipMemcpyHostToDevice);
    hipMemcpy(B, hb.data(), hb.size() * 2, hipMemcpyHostToDevice);
    GemmParams p{M, N, K, A, B, C, 0, 0, 0, 0, 0};
    table<4, 4, 2>("256 x 256 tiles by four waves", p);
    table<2, 2, 4>("128 x 256 tiles by eight waves", p);
    hipFree(A); hipFree(B); hipFree(C);
  }
  return 0;
}
