// Last-error bookkeeping and library identification for libfwdmi (no GPU runtime needed).
#include "status.h"

#include <cstring>

namespace fwdmi {
namespace {
thread_local char g_last_error[512] = "";
}

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_last_error[0] = '\0'; }

}  // namespace fwdmi

extern "C" {

const char* fwdmi_version(void) { return "fwdmi 0.2 (gfx950)"; }

const char* fwdmi_last_error(void) { return fwdmi::g_last_error; }

}  // extern "C"
