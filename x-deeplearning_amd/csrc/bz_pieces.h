// bz_pieces.h -- a tensor given as a concat of pieces computed on the fly (bz_concat_ew_desc), in the form the kernels
// take it: shared by the kernel that writes such a tensor (elementwise.hip) and the FC kernel that multiplies it without
// its ever being stored (fc_fused.hip).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "bz_common.h"

namespace bz {

template <typename T>
__device__ __forceinline__ float ldv(const T* p);
template <>
__device__ __forceinline__ float ldv<float>(const float* p) {
  return *p;
}
template <>
__device__ __forceinline__ float ldv<__half>(const __half* p) {
  return __half2float(*p);
}
template <>
__device__ __forceinline__ float ldv<__hip_bfloat16>(const __hip_bfloat16* p) {
  return __bfloat162float(*p);
}
template <typename T>
__device__ __forceinline__ void stv(T* p, float v);
template <>
__device__ __forceinline__ void stv<float>(float* p, float v) {
  *p = v;
}
template <>
__device__ __forceinline__ void stv<__half>(__half* p, float v) {
  *p = __float2half_rn(v);
}
template <>
__device__ __forceinline__ void stv<__hip_bfloat16>(__hip_bfloat16* p, float v) {
  *p = __float2bfloat16(v);
}

struct CewP {
  const void* x[BZ_CEW_MAX];
  const void* y[BZ_CEW_MAX];
  int64_t xs[BZ_CEW_MAX][2], ys[BZ_CEW_MAX][2];
  int32_t op[BZ_CEW_MAX];
  int32_t col0[BZ_CEW_MAX + 1];  // first output column of each piece; col0[n] = total
  int n;
  int64_t rows, r1, dst_pitch;
};

// VEC consecutive elements as one aligned load or store
template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) CewPack {
  T e[VEC];
};

// Piece k of one row, VEC columns from column cv * VEC of the piece, for pieces that do not divide: one fused
// multiply-add whose operands are chosen per piece,
//   x + y = fma(x, 1, y)    x - y = fma(x, 1, -y)    x * y = fma(x, y, -0)
// each rounded once like the plain operation (-0 as the addend keeps the sign of a zero product); a copy keeps the
// loaded bits.  xk / yk: the operands already loaded (a piece without a second operand passes its first one twice).
template <typename T, int VEC>
__device__ __forceinline__ CewPack<T, VEC> cew_piece(int op, const CewPack<T, VEC>& xk, const CewPack<T, VEC>& yk) {
  const bool mul = op == BZ_EW_MUL, neg = op == BZ_EW_SUB, copy = op == BZ_EW_ASSIGN;
  CewPack<T, VEC> o;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    const float a = ldv<T>(&xk.e[e]), b = ldv<T>(&yk.e[e]);
    const float r = __builtin_fmaf(a, mul ? b : 1.f, mul ? -0.f : (neg ? -b : b));
    stv<T>(&o.e[e], r);
    if (copy) o.e[e] = xk.e[e];
  }
  return o;
}

// Checks a descriptor and turns it into kernel arguments.  *vec: the widest power of two (<= 8) that divides every
// width, stride and element address, so that VEC elements are one aligned access.  with_dst: also check and fit
// dst / dst_pitch (a consumer that keeps the tensor on chip has neither).
inline int cew_build(const bz_concat_ew_desc& d, bool with_dst, CewP* out, int* vec_out, const char* who) {
  BZ_REQUIRE(d.n >= 1 && d.n <= BZ_CEW_MAX, "%s: %d pieces outside 1..%d", who, d.n, BZ_CEW_MAX);
  BZ_REQUIRE(d.dtype == BZ_F32 || d.dtype == BZ_F16 || d.dtype == BZ_BF16, "%s: unsupported dtype %d", who, d.dtype);
  BZ_REQUIRE(d.r0 >= 0 && d.r1 >= 0, "%s: r0=%lld r1=%lld", who, (long long)d.r0, (long long)d.r1);
  BZ_REQUIRE(!with_dst || d.dst != nullptr, "%s: null dst", who);
  const int es = bz::dtype_size(d.dtype);
  CewP p = {};
  p.n = d.n;
  p.rows = d.r0 * d.r1;
  p.r1 = d.r1 > 0 ? d.r1 : 1;
  p.dst_pitch = d.dst_pitch;
  int vec = 8;
  auto fit = [&](int64_t q) {
    while (vec > 1 && q % vec != 0) vec >>= 1;
  };
  int64_t total = 0;
  for (int i = 0; i < d.n; ++i) {
    BZ_REQUIRE(d.op[i] >= BZ_EW_ADD && d.op[i] <= BZ_EW_ASSIGN, "%s: piece %d: unknown op %d", who, i, d.op[i]);
    BZ_REQUIRE(d.x[i] != nullptr && (d.op[i] == BZ_EW_ASSIGN || d.y[i] != nullptr), "%s: piece %d: null operand", who, i);
    BZ_REQUIRE(d.width[i] > 0, "%s: piece %d: width %d", who, i, d.width[i]);
    p.x[i] = d.x[i];
    p.y[i] = d.y[i];
    p.op[i] = d.op[i];
    p.col0[i] = (int32_t)total;
    total += d.width[i];
    fit(d.width[i]);
    fit((int64_t)((uintptr_t)d.x[i] / es));
    BZ_REQUIRE((uintptr_t)d.x[i] % es == 0, "%s: piece %d: misaligned operand", who, i);
    for (int k = 0; k < 2; ++k) {
      BZ_REQUIRE(d.x_stride[i][k] >= 0 && d.y_stride[i][k] >= 0, "%s: piece %d: negative stride", who, i);
      p.xs[i][k] = d.x_stride[i][k];
      p.ys[i][k] = d.y_stride[i][k];
      fit(d.x_stride[i][k]);
      if (d.op[i] != BZ_EW_ASSIGN) fit(d.y_stride[i][k]);
    }
    if (d.op[i] != BZ_EW_ASSIGN) {
      BZ_REQUIRE((uintptr_t)d.y[i] % es == 0, "%s: piece %d: misaligned operand", who, i);
      fit((int64_t)((uintptr_t)d.y[i] / es));
    }
  }
  BZ_REQUIRE(total < (1ll << 31), "%s: widths sum to %lld", who, (long long)total);
  p.col0[d.n] = (int32_t)total;
  if (with_dst) {
    BZ_REQUIRE(total <= d.dst_pitch, "%s: widths sum to %lld, row pitch is %lld", who, (long long)total, (long long)d.dst_pitch);
    BZ_REQUIRE((uintptr_t)d.dst % es == 0, "%s: misaligned dst", who);
    fit(d.dst_pitch);
    fit((int64_t)((uintptr_t)d.dst / es));
  }
  *out = p;
  *vec_out = vec;
  return BZ_OK;
}

// every piece as wide as the first and none divides: the form the branch-free kernels take
inline bool cew_uniform(const CewP& p) {
  for (int k = 0; k < p.n; ++k)
    if (p.col0[k + 1] - p.col0[k] != p.col0[1] || p.op[k] == BZ_EW_DIV) return false;
  return true;
}

}  // namespace bz
