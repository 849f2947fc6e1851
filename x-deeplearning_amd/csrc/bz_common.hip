// bz_common.hip -- error reporting and the device probe of the kernel layer.
#include "bz_common.h"

#include <hip/hip_runtime.h>
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

namespace {
// one wave that watches the constant-rate clock (100 MHz) until `ticks` have passed; the pass count bounds it so that
// it ends whatever the clock does
__global__ void bz_spin_kernel(long long ticks) {
  const long long t0 = wall_clock64();
  for (int i = 0; i < (1 << 17) && wall_clock64() - t0 < ticks; ++i) __builtin_amdgcn_s_sleep(8);
}
}  // namespace

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

int bz_spin(int64_t microseconds, bz_stream_t stream) {
  if (microseconds < 0 || microseconds > 10000) return bz::fail(BZ_EINVAL, "bz_spin: %lld us (0 .. 10000)", (long long)microseconds);
  hipLaunchKernelGGL(bz_spin_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (long long)microseconds * 100);
  BZ_HIP_OK(hipGetLastError());
  return BZ_OK;
}

}  // extern "C"
