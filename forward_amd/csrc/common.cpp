// Device enumeration for libfwdmi.
#include "common.h"

extern "C" {

int fwdmi_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

}  // extern "C"
