// bz_common.hip -- error reporting and the device probe of the kernel layer.
#include "bz_common.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

namespace bz {

namespace {
thread_local char g_err[1024] = "";
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

}  // namespace bz

extern "C" {

const char* bz_last_error(void) { return bz::g_err; }

int bz_device_check(char* name, size_t cap) {
  int dev = 0;
  BZ_HIP_OK(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  BZ_HIP_OK(hipGetDeviceProperties(&prop, dev));
  if (name != nullptr && cap > 0) {
    strncpy(name, prop.gcnArchName, cap - 1);
    name[cap - 1] = 0;
  }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return bz::fail(BZ_ENOTSUP, "device %d is %s; this library is built for gfx950 only", dev, prop.gcnArchName);
  return BZ_OK;
}

}  // extern "C"
