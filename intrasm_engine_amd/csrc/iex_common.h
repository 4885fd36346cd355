// Shared host/device helpers of libiex_hip.so (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <type_traits>

#include "../../include/iex_hip.h"

namespace iex {

constexpr int kWave = 64;

// ---- error text (thread local) ------------------------------------------------
char* last_error_buffer();
int fail(int code, const char* fmt, ...);
int check_hip(hipError_t err, const char* what);
// Names of the kernels the current entry point has launched on this thread (iex_last_kernels):
// trail_reset() at the start of an entry point, note_kernel() beside every launch.
void trail_reset();
void note_kernel(const char* fmt, ...);
template <typename T> inline const char* type_name();
template <> inline const char* type_name<float>() { return "float"; }
template <> inline const char* type_name<__half>() { return "__half"; }
template <> inline const char* type_name<__hip_bfloat16>() { return "__hip_bfloat16"; }
template <> inline const char* type_name<int>() { return "int"; }
template <> inline const char* type_name<short>() { return "short"; }

#define IEX_REQUIRE(cond, code, ...)                 \
  do {                                               \
    if (!(cond)) return ::iex::fail(code, __VA_ARGS__); \
  } while (0)

// ---- element traits -------------------------------------------------------------
template <typename T> struct elem;
template <> struct elem<float> {
  static __device__ __forceinline__ float to_float(float v) { return v; }
  static __device__ __forceinline__ float from_float(float v) { return v; }
};
template <> struct elem<__half> {
  static __device__ __forceinline__ float to_float(__half v) { return __half2float(v); }
  static __device__ __forceinline__ __half from_float(float v) { return __float2half_rn(v); }
};
template <> struct elem<__hip_bfloat16> {
  static __device__ __forceinline__ float to_float(__hip_bfloat16 v) { return __bfloat162float(v); }
  static __device__ __forceinline__ __hip_bfloat16 from_float(float v) { return __float2bfloat16(v); }
};

// A VEC-wide register vector of T moved with one load/store instruction.
template <typename T, int VEC> struct alignas(sizeof(T) * VEC) vec_t { T v[VEC]; };

// The same vector at element alignment only: still one instruction (the hardware takes 128-bit
// accesses at any dword / element boundary), for rows whose length is not a multiple of VEC.
template <typename T, int VEC> struct alignas(sizeof(T)) vec_unaligned_t { T v[VEC]; };

template <typename T, int VEC, bool ALIGNED = true>
__device__ __forceinline__ vec_t<T, VEC> load_vec(const T* p) {
  if constexpr (ALIGNED) {
    return *reinterpret_cast<const vec_t<T, VEC>*>(p);
  } else {
    const vec_unaligned_t<T, VEC> u = *reinterpret_cast<const vec_unaligned_t<T, VEC>*>(p);
    vec_t<T, VEC> r;
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.v[i] = u.v[i];
    return r;
  }
}
template <typename T, int VEC, bool ALIGNED = true>
__device__ __forceinline__ void store_vec(T* p, const vec_t<T, VEC>& x) {
  if constexpr (ALIGNED) {
    *reinterpret_cast<vec_t<T, VEC>*>(p) = x;
  } else {
    vec_unaligned_t<T, VEC> u;
#pragma unroll
    for (int i = 0; i < VEC; ++i) u.v[i] = x.v[i];
    *reinterpret_cast<vec_unaligned_t<T, VEC>*>(p) = u;
  }
}

// The same store with the streaming hint: for outputs far larger than the caches, written once
// and not read again by the kernel (measured on 3.8 GB of SpMM output: 4.5 -> 5.3 TB/s).
template <int BYTES> struct stream_word;
template <> struct stream_word<16> { typedef unsigned int type __attribute__((ext_vector_type(4))); };
template <> struct stream_word<8> { typedef unsigned int type __attribute__((ext_vector_type(2))); };
template <> struct stream_word<4> { typedef unsigned int type; };
template <> struct stream_word<2> { typedef unsigned short type; };
template <typename T, int VEC, bool ALIGNED = true>
__device__ __forceinline__ void store_vec_stream(T* p, const vec_t<T, VEC>& x) {
  typedef typename stream_word<sizeof(T) * VEC>::type W;
  // The pointer passes through an empty asm so that the compiler sees another address than in the plain
  // store of the other branch: it would otherwise merge the two stores of an `if (stream) ... else ...`
  // into one and drop the hint, which only one of them carries.
  asm volatile("" : "+v"(p));
  if constexpr (ALIGNED) {
    __builtin_nontemporal_store(__builtin_bit_cast(W, x), reinterpret_cast<W*>(p));
  } else {
    typedef W WU __attribute__((aligned(sizeof(T))));
    __builtin_nontemporal_store(__builtin_bit_cast(W, x), reinterpret_cast<WU*>(p));
  }
}

// ---- wave64 cross-lane helpers --------------------------------------------------
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Broadcast lane `src` (wave-uniform) of a VGPR into a scalar register.
__device__ __forceinline__ int bcast_i(int v, int src) { return __builtin_amdgcn_readlane(v, src); }
__device__ __forceinline__ float bcast_f(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// Sum over aligned groups of LANES consecutive lanes (LANES in {1,2,4,8,16});
// every lane of the group ends up with the total.  DPP only, no LDS traffic.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
  if (LANES >= 2) v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
  if (LANES >= 4) v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  if (LANES >= 8) v += dpp_f<0x141>(v);  // row_half_mirror
  if (LANES >= 16) v += dpp_f<0x140>(v); // row_mirror
  return v;
}

template <int CTRL>
__device__ __forceinline__ float dpp_max_f(float v) {
  return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, 0xf, 0xf, false)));
}
// Whole-wave (64 lanes) sum / max; result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v) {
  v = group_sum<16>(v);
  return bcast_f(v, 0) + bcast_f(v, 16) + bcast_f(v, 32) + bcast_f(v, 48);
}
__device__ __forceinline__ float wave_max(float v) {
  v = dpp_max_f<0xB1>(v);
  v = dpp_max_f<0x4E>(v);
  v = dpp_max_f<0x141>(v);
  v = dpp_max_f<0x140>(v);
  return fmaxf(fmaxf(bcast_f(v, 0), bcast_f(v, 16)), fmaxf(bcast_f(v, 32), bcast_f(v, 48)));
}

inline int ceil_div(long long a, long long b) { return (int)((a + b - 1) / b); }
inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

}  // namespace iex
