// common.h -- substrate of the host layer: exceptions, element types, logging, HIP error checks.
//
// Mirrors the parts of the reference's blaze/common/ that the sparse CTR path touches:
//   exception.h:35-89   BLAZE_THROW / BLAZE_CONDITION_THROW / CHECK (C++ exceptions inside, caught at the API)
//   types.h:50-83,129-166   float16 (RNE narrowing, exact widening), DataTypeSize
//   log.h               leveled printf-style logging
// Element type numbers are the wire values of blaze/proto/blaze.proto:6-19.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include <exception>
#include <sstream>
#include <string>
#include <vector>

namespace blaze {

typedef size_t TIndex;

enum DataType {
  kFloat = 1,
  kInt32 = 2,
  kByte = 3,
  kString = 4,
  kBool = 5,
  kUInt8 = 6,
  kInt8 = 7,
  kUInt16 = 8,
  kInt16 = 9,
  kInt64 = 10,
  kFloat16 = 12,
  kDouble = 13,
};

// device_type 1 is the accelerator of this build (the reference calls it kCUDA, blaze.proto:36-39):
// existing NetDefs that say device_type : 1 run on the MI355X unchanged.
enum DeviceType { kCPU = 0, kHIP = 1, kCUDA = 1 };

// ------------------------------------------------------------------------------------------ errors
inline void MakeStringInternal(std::stringstream&) {}
template <typename T, typename... Args>
inline void MakeStringInternal(std::stringstream& ss, const T& t, const Args&... args) {
  ss << t;
  MakeStringInternal(ss, args...);
}
template <typename... Args>
std::string MakeString(const Args&... args) {
  std::stringstream ss;
  MakeStringInternal(ss, args...);
  return ss.str();
}

class Exception : public std::exception {
 public:
  Exception(const char* file, int line, const char* condition, const std::string& msg) {
    std::stringstream ss;
    ss << "[" << file << ":" << line << "] ";
    if (condition && *condition) ss << "check failed: " << condition << " ";
    ss << msg;
    full_msg_ = ss.str();
  }
  const char* what() const noexcept override { return full_msg_.c_str(); }

 private:
  std::string full_msg_;
};

#define BLAZE_THROW(...) throw ::blaze::Exception(__FILE__, __LINE__, "", ::blaze::MakeString(__VA_ARGS__))
#define BLAZE_CONDITION_THROW(condition, ...)                                                     \
  do {                                                                                            \
    if (!(condition)) throw ::blaze::Exception(__FILE__, __LINE__, #condition, ::blaze::MakeString(__VA_ARGS__)); \
  } while (false)
#define BLAZE_CHECK(condition, ...) BLAZE_CONDITION_THROW(condition, __VA_ARGS__)

#define HIP_CHECK(expr)                                                                    \
  do {                                                                                     \
    hipError_t e_ = (expr);                                                                \
    if (e_ != hipSuccess) BLAZE_THROW(#expr, " failed: ", hipGetErrorString(e_));          \
  } while (false)

// a kernel-layer call (include/blaze_hip.h) that returns a negative code throws with the layer's message
#define BZ_CHECK(expr)                                                          \
  do {                                                                          \
    int rc_ = (expr);                                                           \
    if (rc_ != 0) BLAZE_THROW(#expr, " rc=", rc_, ": ", bz_last_error());       \
  } while (false)

// ------------------------------------------------------------------------------------------ logging
enum LogLevel { kLogDebug = 0, kLogInfo = 1, kLogError = 2, kLogFatal = 3 };
void LogMessage(int level, const char* file, int line, const char* fmt, ...) __attribute__((format(printf, 4, 5)));
void SetLogLevel(int level);  // default kLogError; env BLAZE_LOG_LEVEL overrides
#define LOG_DEBUG(...) ::blaze::LogMessage(::blaze::kLogDebug, __FILE__, __LINE__, __VA_ARGS__)
#define LOG_INFO(...) ::blaze::LogMessage(::blaze::kLogInfo, __FILE__, __LINE__, __VA_ARGS__)
#define LOG_ERROR(...) ::blaze::LogMessage(::blaze::kLogError, __FILE__, __LINE__, __VA_ARGS__)

// ------------------------------------------------------------------------------------------ types
inline size_t DataTypeSize(int data_type) {
  switch (data_type) {
    case kFloat: return 4;
    case kDouble: return 8;
    case kFloat16: return 2;
    case kInt32: return 4;
    case kBool: return 1;
    case kUInt8: return 1;
    case kInt8: return 1;
    case kUInt16: return 2;
    case kInt16: return 2;
    case kInt64: return 8;
    default: BLAZE_THROW("Not supported type=", data_type);
  }
}

// binary32 -> binary16, round to nearest even; binary16 -> binary32 exact (types.cc:9-30 via F16C)
uint16_t FloatToHalf(float f);
float HalfToFloat(uint16_t h);

}  // namespace blaze
