// Shared host-side helpers of the C ABI: status codes, the per-thread error
// string, and launch checking.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include "../../include/clgrpo.h"

namespace clgrpo {

char* error_buffer();            // thread-local, 512 bytes
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);
// Raises the kernel's dynamic-LDS limit to `bytes` on the current device, once per (kernel, device).
int ensure_dynamic_lds(const void* kernel, int bytes, const char* name);
// Compute units of the current device (looked up once per device; 256 if the query fails).
int device_cu_count();

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
inline int64_t round_up64(int64_t x, int64_t a) { return (x + a - 1) / a * a; }
inline size_t dtype_bytes(int32_t d) { return d == CLGRPO_BF16 ? 2 : (d == CLGRPO_F32 ? 4 : 8); }

}  // namespace clgrpo

#define CLGRPO_REQUIRE_PTR(p, name) \
  if ((p) == nullptr) return ::clgrpo::fail(CLGRPO_ENULL, "%s: %s is NULL", __func__, name)
