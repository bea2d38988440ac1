// Shared host-side helpers of libfwdmi: status codes, last-error text, HIP call checking.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
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

#define FWDMI_HIP_CHECK(expr)                                                                 \
  do {                                                                                        \
    hipError_t e_ = (expr);                                                                   \
    if (e_ != hipSuccess)                                                                     \
      return ::fwdmi::set_error(FWDMI_ERR_HIP, "%s failed: %s (%s:%d)", #expr,                \
                                hipGetErrorString(e_), __FILE__, __LINE__);                   \
  } while (0)

#define FWDMI_REQUIRE(cond, ...)                                         \
  do {                                                                   \
    if (!(cond)) return ::fwdmi::set_error(FWDMI_ERR_BAD_ARG, __VA_ARGS__); \
  } while (0)
