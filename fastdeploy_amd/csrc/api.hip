// Error reporting and identification shared by every entry point of libfdattn.so.
#include <stdarg.h>
#include <stdio.h>

#include "fdattn_common.h"

namespace fdattn {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  return fail((int)e, "%s: launch failed: %s", what, hipGetErrorString(e));
}

}  // namespace fdattn

extern "C" const char* fdattn_version(void) { return "fdattn 0.1 gfx950"; }
extern "C" const char* fdattn_last_error(void) { return fdattn::g_err; }
