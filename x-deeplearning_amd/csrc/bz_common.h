// bz_common.h -- shared helpers of the gfx950 kernel layer (error plumbing, small device utilities).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "blaze_hip.h"

namespace bz {

// Records the message returned by bz_last_error() for this thread and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define BZ_REQUIRE(cond, ...)                       \
  do {                                              \
    if (!(cond)) return ::bz::fail(BZ_EINVAL, __VA_ARGS__); \
  } while (0)

#define BZ_HIP_OK(expr)                                                                                   \
  do {                                                                                                    \
    hipError_t e_ = (expr);                                                                               \
    if (e_ != hipSuccess) return ::bz::fail(BZ_EHIP, "%s failed: %s", #expr, hipGetErrorString(e_));      \
  } while (0)

// A kernel launch reports configuration errors through hipGetLastError.
#define BZ_LAUNCH_OK(what)                                                                                \
  do {                                                                                                    \
    hipError_t e_ = hipGetLastError();                                                                    \
    if (e_ != hipSuccess) return ::bz::fail(BZ_EHIP, "launch of %s failed: %s", what, hipGetErrorString(e_)); \
  } while (0)

inline hipStream_t as_stream(bz_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int dtype_size(int dt) {
  switch (dt) {
    case BZ_F32: return 4;
    case BZ_I32: return 4;
    case BZ_F16: return 2;
    case BZ_BF16: return 2;
    case BZ_I8: return 1;
    case BZ_I64: return 8;
    default: return 0;
  }
}

constexpr int kWave = 64;       // CDNA wavefront
constexpr int kNumXcd = 8;      // MI355X: 8 accelerator complex dies, workgroups are dealt to them round robin

}  // namespace bz
