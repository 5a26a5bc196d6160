// Version string, thread-local error message and trace switch of the library.
#include <cstdlib>
#include <cstring>

#include "common.h"

namespace xmk {
namespace {
thread_local char g_error[512] = "";
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  if (trace_enabled()) fprintf(stderr, "[xmk] error %d: %s\n", code, g_error);
  return code;
}

bool trace_enabled() {
  static const bool on = [] {
    const char* v = getenv("XMK_TRACE");
    return v && *v && strcmp(v, "0") != 0;
  }();
  return on;
}

void trace(const char* fmt, ...) {
  if (!trace_enabled()) return;
  va_list ap;
  va_start(ap, fmt);
  fputs("[xmk] ", stderr);
  vfprintf(stderr, fmt, ap);
  fputc('\n', stderr);
  va_end(ap);
}
}  // namespace xmk

extern "C" const char* xmk_version(void) { return "xmk 0.1 (gfx950)"; }
extern "C" const char* xmk_last_error(void) { return xmk::g_error; }
