// Status codes, last-error text and argument checks of libfwdmi that need no GPU runtime: shared by
// the launch code and by the host-only parts (launch planning, sidecar files) and their CPU tests.
#pragma once

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "fwdmi.h"

namespace fwdmi {

// Records printf-style text as the calling thread's last error and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

inline bool is_float_dtype(int t) { return t == FWDMI_F32 || t == FWDMI_F16; }
inline bool is_index_dtype(int t) { return t == FWDMI_I32 || t == FWDMI_I64; }
inline size_t dtype_size(int t) {
  switch (t) {
    case FWDMI_F32: return 4;
    case FWDMI_F16: return 2;
    case FWDMI_I8: return 1;
    case FWDMI_I32: return 4;
    case FWDMI_BOOL: return 1;
    case FWDMI_I64: return 8;
    default: return 0;
  }
}

}  // namespace fwdmi

#define FWDMI_REQUIRE(cond, ...)                                         \
  do {                                                                   \
    if (!(cond)) return ::fwdmi::set_error(FWDMI_ERR_BAD_ARG, __VA_ARGS__); \
  } while (0)
