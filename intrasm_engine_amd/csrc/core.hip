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

int check_hip(hipError_t err, const char* what) {
  if (err == hipSuccess) return 0;
  snprintf(last_error_buffer(), 512, "%s: %s (hipError_t %d)", what, hipGetErrorString(err), (int)err);
  return (int)err;
}

}  // namespace iex

extern "C" {

int iex_abi_version(void) { return IEX_ABI_VERSION; }

const char* iex_last_error(void) { return iex::last_error_buffer(); }

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
