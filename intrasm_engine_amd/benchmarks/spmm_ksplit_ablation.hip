// Ablation of the k-split SpMM kernel (spmm_ksplit_device.cuh beside this file; it was family 9 of the library until it was measured and taken out) on the shape of the 4096 x 4096 fp32
// sweep, n = 256: the kernel as shipped, and instrumented builds of the same template that leave out one
// ingredient each (the DBG switches of spmm_ksplit_block; results of those builds are wrong on purpose, every
// address they use stays in bounds).  Prints microseconds per launch (HIP events, 20 launches) of the main kernel
// alone; the partial-sum kernel that follows it in the library is not part of this.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         intrasm_engine_amd/benchmarks/spmm_ksplit_ablation.hip -o spmm_ksplit_ablation && ./spmm_ksplit_ablation [densities ...]
//   IEX_ABLATION_SHORT=1: three launches of the shipped kernel only (8 and 16 wavefronts), for rocprofv3 --pmc.
#include "spmm_ksplit_device.cuh"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

using namespace iex;
namespace iex {   // the three symbols of core.hip that the device headers declare
char* last_error_buffer() { static char b[512]; return b; }
int fail(int code, const char*, ...) { return code; }
int check_hip(hipError_t e, const char*) { return (int)e; }
}  // namespace iex

template <int VEC, int WAVES, int KB, int DBG>
__global__ __launch_bounds__(WAVES * kWave, WAVES == 8 ? 2 : 1) void ablation_kernel(KsplitParams q) {
  extern __shared__ __align__(16) unsigned char smem[];
  spmm_ksplit_block<float, int, VEC, 8, WAVES, KB, DBG>(q, blockIdx.x / q.slices, blockIdx.x % q.slices, blockIdx.y, blockIdx.z, smem);
}

struct Csr {
  int m, k;
  std::vector<int> ro, ci, ri;
  std::vector<float> v;
};

// geometric row lengths (mean k * density), uniformly drawn sorted columns, rows ranked by decreasing length
static Csr make(int m, int k, double density, unsigned seed) {
  std::mt19937 g(seed);
  Csr c;
  c.m = m;
  c.k = k;
  c.ro.assign(m + 1, 0);
  std::geometric_distribution<int> geo(1.0 / (k * density));
  std::vector<int> lens(m), perm(k);
  for (int r = 0; r < m; ++r) lens[r] = std::min(k, std::max(1, geo(g) + 1));
  for (int r = 0; r < m; ++r) c.ro[r + 1] = c.ro[r] + lens[r];
  c.ci.resize(c.ro[m]);
  c.v.resize(c.ro[m]);
  std::normal_distribution<float> nd(0, 0.02f);
  for (int r = 0; r < m; ++r) {
    for (int i = 0; i < k; ++i) perm[i] = i;
    for (int i = 0; i < lens[r]; ++i) std::swap(perm[i], perm[i + g() % (k - i)]);
    std::sort(perm.begin(), perm.begin() + lens[r]);
    for (int i = 0; i < lens[r]; ++i) {
      c.ci[c.ro[r] + i] = perm[i];
      c.v[c.ro[r] + i] = nd(g);
    }
  }
  c.ri.resize(m);
  for (int r = 0; r < m; ++r) c.ri[r] = r;
  std::stable_sort(c.ri.begin(), c.ri.end(), [&](int a, int b) { return lens[a] > lens[b]; });
  return c;
}

template <class T>
static T* upload(const std::vector<T>& h) {
  T* d = nullptr;
  if (hipMalloc(&d, h.size() * sizeof(T)) != hipSuccess || hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) {
    fprintf(stderr, "device allocation or copy failed\n");
    exit(1);
  }
  return d;
}

template <int VEC, int WAVES, int KB, int DBG>
static void run(const char* what, SpmmParams p, int slices, float* partial, int reps = 20) {
  constexpr int lds = spmm_ksplit_lds_bytes<VEC, float, KB>();
  auto kern = ablation_kernel<VEC, WAVES, KB, DBG>;
  hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  KsplitParams q{p, (p.m + WAVES * 8 - 1) / (WAVES * 8), slices, 0, partial};
  q.slice_rows = ((p.k + slices - 1) / slices + KB - 1) / KB * KB;
  q.slices = (p.k + q.slice_rows - 1) / q.slice_rows;
  int wgs_per_cu = -1;
  hipOccupancyMaxActiveBlocksPerMultiprocessor(&wgs_per_cu, kern, WAVES * 64, lds);
  hipEvent_t a, b;
  hipEventCreate(&a);
  hipEventCreate(&b);
  const dim3 grid(q.row_blocks * q.slices, (p.n + 64 * VEC - 1) / (64 * VEC), 1);
  for (int i = 0; i < 3; ++i) hipLaunchKernelGGL(kern, grid, dim3(WAVES * 64), lds, 0, q);
  hipEventRecord(a);
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(kern, grid, dim3(WAVES * 64), lds, 0, q);
  hipEventRecord(b);
  hipEventSynchronize(b);
  float ms = 0;
  hipEventElapsedTime(&ms, a, b);
  printf("  %2d wavefronts, stages of %2d rows, %d workgroups per CU | %-58s %7.1f us%s\n", WAVES, KB, wgs_per_cu, what, ms / reps * 1e3,
         hipGetLastError() == hipSuccess ? "" : "  (HIP error)");
}

int main(int argc, char** argv) {
  const int m = 4096, k = 4096, n = 256, slices = 8;
  std::vector<double> densities = {0.02, 0.1, 0.3};
  if (argc > 1) {
    densities.clear();
    for (int i = 1; i < argc; ++i) densities.push_back(atof(argv[i]));
  }
  const bool brief = getenv("IEX_ABLATION_SHORT") != nullptr;
  for (double d : densities) {
    const Csr c = make(m, k, d, 7);
    std::vector<float> B((size_t)k * n);
    std::mt19937 g(3);
    std::normal_distribution<float> nd(0, 1);
    for (auto& x : B) x = nd(g);
    int *ri = upload(c.ri), *ro = upload(c.ro), *ci = upload(c.ci);
    float *v = upload(c.v), *b = upload(B), *out = nullptr, *partial = nullptr;
    hipMalloc(&out, (size_t)m * n * 4);
    hipMalloc(&partial, (size_t)slices * m * n * 4);
    const SpmmParams p{m, k, n, (int)c.ci.size(), ri, v, ro, ci, b, nullptr, out, 0, 0, 0};
    printf("A %d x %d, density %.2f (%zu nonzeros, geometric row lengths), n = %d, %d k slices\n", m, k, d, c.ci.size(), n, slices);
    if (brief) {
      run<4, 8, 32, 0>("as shipped", p, slices, partial, 3);
      run<4, 16, 64, 0>("as shipped", p, slices, partial, 3);
    } else {
      run<4, 8, 32, 0>("as shipped", p, slices, partial);
      run<4, 8, 32, 1>("no gathers (stages, barriers, bookkeeping, partial stores)", p, slices, partial);
      run<4, 8, 32, 2>("no direct loads of the dense operand", p, slices, partial);
      run<4, 8, 32, 3>("neither (the skeleton)", p, slices, partial);
      run<4, 8, 32, 8>("no barrier between stages", p, slices, partial);
      run<4, 8, 32, 16>("(column, value) from arithmetic instead of v_readlane", p, slices, partial);
      run<4, 8, 32, 32>("no LDS read per nonzero", p, slices, partial);
      run<4, 8, 32, 48>("neither v_readlane nor LDS read: address add + 4 FMAs per nonzero", p, slices, partial);
      run<4, 8, 32, 50>("... and no direct loads", p, slices, partial);
      run<4, 16, 64, 0>("as shipped", p, slices, partial);
      run<4, 16, 64, 16>("(column, value) from arithmetic instead of v_readlane", p, slices, partial);
    }
    hipFree(ri); hipFree(ro); hipFree(ci); hipFree(v); hipFree(b); hipFree(out); hipFree(partial);
  }
  return 0;
}
