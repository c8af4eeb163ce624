// Status / error-string plumbing of the C ABI.
#include "common.hpp"
#include <string.h>
#include <atomic>

namespace clgrpo {

static thread_local char g_err[512] = "";

char* error_buffer() { return g_err; }

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(CLGRPO_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
  return CLGRPO_OK;
}

// The limit is a per-device property of a kernel; a process may drive several devices and call from
// several threads.  Small fixed table: at most kMaxKernels kernels on kMaxDevices devices.
int ensure_dynamic_lds(const void* kernel, int bytes, const char* name) {
  constexpr int kMaxKernels = 32, kMaxDevices = 64;
  static std::atomic<const void*> keys[kMaxKernels];
  static std::atomic<unsigned char> done[kMaxKernels][kMaxDevices];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(CLGRPO_ELAUNCH, "%s: hipGetDevice: %s", name, hipGetErrorString(e));
  int slot = -1;
  for (int i = 0; i < kMaxKernels && slot < 0; ++i) {
    const void* cur = keys[i].load(std::memory_order_acquire);
    if (cur == kernel) slot = i;
    else if (cur == nullptr) {
      const void* expected = nullptr;
      if (keys[i].compare_exchange_strong(expected, kernel) || expected == kernel) slot = i;
    }
  }
  const bool tracked = slot >= 0 && dev >= 0 && dev < kMaxDevices;
  if (tracked && done[slot][dev].load(std::memory_order_acquire)) return CLGRPO_OK;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);   // idempotent
  if (e != hipSuccess) return fail(CLGRPO_ELAUNCH, "%s: LDS attribute: %s", name, hipGetErrorString(e));
  if (tracked) done[slot][dev].store(1, std::memory_order_release);
  return CLGRPO_OK;
}

int device_cu_count() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n > 0) return n;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

}  // namespace clgrpo

extern "C" int clgrpo_version(void) { return 202; }
extern "C" const char* clgrpo_last_error_string(void) { return clgrpo::error_buffer(); }
