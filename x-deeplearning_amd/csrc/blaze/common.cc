#include "blaze/common.h"

#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

namespace blaze {

namespace {
int g_log_level = -1;
int CurrentLevel() {
  if (g_log_level < 0) {
    const char* e = getenv("BLAZE_LOG_LEVEL");
    g_log_level = e ? atoi(e) : kLogError;
  }
  return g_log_level;
}
}  // namespace

void SetLogLevel(int level) { g_log_level = level; }

void LogMessage(int level, const char* file, int line, const char* fmt, ...) {
  if (level < CurrentLevel()) return;
  static const char* kNames[] = {"DEBUG", "INFO", "ERROR", "FATAL"};
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  const char* base = strrchr(file, '/');
  fprintf(stderr, "[%s %s:%d] %s\n", kNames[level < 0 || level > 3 ? 2 : level], base ? base + 1 : file, line, buf);
}

uint16_t FloatToHalf(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) {  // inf / nan
    const uint32_t man = ax & 0x7fffffu;
    return (uint16_t)(sign | 0x7c00u | (man ? (0x200u | (man >> 13)) : 0));
  }
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds up to infinity
  if (ax < 0x33000001u) return (uint16_t)sign;               // rounds down to zero
  const int e = (int)(ax >> 23) - 127;
  const uint32_t man = (ax & 0x7fffffu) | 0x800000u;
  const uint32_t shift = e < -14 ? (uint32_t)(13 + (-14 - e)) : 13u;
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  const uint32_t out = e < -14 ? q : (((uint32_t)(e + 15) - 1u) << 10) + q;
  return (uint16_t)(sign | out);
}

float HalfToFloat(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do {
        ++e;
        man <<= 1;
      } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

}  // namespace blaze
