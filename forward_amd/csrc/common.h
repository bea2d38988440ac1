// Shared host-side helpers of libfwdmi: status codes, last-error text, HIP call checking.
#pragma once

#include <hip/hip_runtime.h>

#include "status.h"

#define FWDMI_HIP_CHECK(expr)                                                                 \
  do {                                                                                        \
    hipError_t e_ = (expr);                                                                   \
    if (e_ != hipSuccess)                                                                     \
      return ::fwdmi::set_error(FWDMI_ERR_HIP, "%s failed: %s (%s:%d)", #expr,                \
                                hipGetErrorString(e_), __FILE__, __LINE__);                   \
  } while (0)
