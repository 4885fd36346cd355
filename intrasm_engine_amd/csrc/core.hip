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
}  // namespace

extern "C" {

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
