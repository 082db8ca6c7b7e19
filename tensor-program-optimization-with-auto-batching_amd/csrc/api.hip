// Library-level entry points of the C ABI: version and per-thread error message.
#include "common.h"

namespace {
thread_local char g_err[512] = "";
}

int mlora_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

extern "C" int mlora_version(void) { return 1; }

extern "C" const char* mlora_last_error(void) { return g_err; }
