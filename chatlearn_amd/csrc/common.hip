// Status / error-string plumbing of the C ABI.
#include "common.hpp"
#include <string.h>

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

}  // namespace clgrpo

extern "C" int clgrpo_version(void) { return 100; }
extern "C" const char* clgrpo_last_error_string(void) { return clgrpo::error_buffer(); }
