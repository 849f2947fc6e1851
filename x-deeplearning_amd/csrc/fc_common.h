// fc_common.h -- what the FC kernels of fc_fused.hip and fc_pieces.hip share: the epilogue (Gemm's alpha / beta / bias,
// then the folded activation) and the MFMA element traits.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "bz_common.h"

namespace bz {
namespace fc {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr float kDiceEps = 1e-8f;  // blaze/operator/common_helper.h:90

struct Epilogue {
  const float* bias;
  const float* p0;
  const float* p1;
  const float* p2;
  int bias_rows;
  int act;
  int act_size;
  int dice_nosqrt;
  float alpha, beta, act_alpha;
  // the N columns are `split_n`-wide slices (sibling FCs stacked along N): column n belongs to slice n / split_n, whose
  // output matrix [M, split_n] (row pitch ldy) starts split_stride elements after the previous slice's; a full bias is
  // laid out the same way, slice after slice.  split_n == 0: one matrix.
  int split_n;
  int64_t split_stride;
};

// element offset of output (m, n) in Y, and of the same element in a full [.., N] bias
__device__ __forceinline__ int64_t out_index(const Epilogue& ep, int64_t m, int n, int64_t ldy) {
  if (ep.split_n == 0) return m * ldy + n;
  const int p = n / ep.split_n;
  return p * ep.split_stride + m * ldy + (n - p * ep.split_n);
}
__device__ __forceinline__ int64_t full_bias_index(const Epilogue& ep, int64_t m, int n, int M, int N) {
  if (ep.split_n == 0) return m * N + n;
  const int p = n / ep.split_n;
  return ((int64_t)p * M + m) * ep.split_n + (n - p * ep.split_n);
}

__device__ __forceinline__ float apply_act(float v, int n, const Epilogue& e) {
  switch (e.act) {
    case BZ_ACT_PRELU: {
      const float w = e.p0[e.act_size == 1 ? 0 : n];
      return v * ((float)(v > 0.f) + (float)(v < 0.f) * w);  // math/activation.h:37-42
    }
    case BZ_ACT_DICE: {
      const float var = e.p2[n];
      const float den = e.dice_nosqrt ? var : sqrtf(var + kDiceEps);
      const float t = expf(-1.f * (v - e.p1[n]) / den);
      const float p = 1.f / (1.f + t);
      return (1.f - p) * e.p0[n] * v + p * v;
    }
    case BZ_ACT_LEAKY_RELU:
      return v >= 0.f ? v : e.act_alpha * v;
    case BZ_ACT_SIGMOID: {
      const float t = expf(v);
      return t / (1.f + t);
    }
    default:
      return v;
  }
}

// the same with the column's parameters already in registers (p0 = slope | gamma, p1 = mean, p2 = var)
__device__ __forceinline__ float apply_act_regs(float v, const Epilogue& e, float p0, float p1, float p2) {
  switch (e.act) {
    case BZ_ACT_PRELU:
      return v * ((float)(v > 0.f) + (float)(v < 0.f) * p0);
    case BZ_ACT_DICE: {
      const float den = e.dice_nosqrt ? p2 : sqrtf(p2 + kDiceEps);
      const float t = expf(-1.f * (v - p1) / den);
      const float p = 1.f / (1.f + t);
      return (1.f - p) * p0 * v + p * v;
    }
    case BZ_ACT_LEAKY_RELU:
      return v >= 0.f ? v : e.act_alpha * v;
    case BZ_ACT_SIGMOID: {
      const float t = expf(v);
      return t / (1.f + t);
    }
    default:
      return v;
  }
}

// log2(e) / (the Dice denominator of a column): computed once per column, before the K loop
__device__ __forceinline__ float dice_inv_den(const Epilogue& e, float var) {
  return 1.44269504088896341f / (e.dice_nosqrt ? var : sqrtf(var + kDiceEps));
}

// The tile kernels' epilogue, activation fixed at compile time.  For Dice p2 is dice_inv_den() of the column, not its
// variance, and the element costs five plain instructions, one v_exp_f32 and one v_rcp_f32 (the attention MLP applies
// Dice to 120 outputs a history position: at 51200 x 50 positions the activation arithmetic alone is microseconds of
// every SIMD): a lane applies the activation to 32..128 outputs one after the other with one or two waves on its SIMD, so
// the exact expf and the two divisions per element (some 80 dependent instructions) were a third to a half of the run
// time of the attention layers (51200 x 216 -> 80: 23.6 us with Dice, 13.2 without).  v_exp_f32 and v_rcp_f32 are
// good to about 1 ulp of fp32 each; what they change in the result is far below the rounding of a 2-byte output and
// below 1e-6 relative for fp32 outputs.
template <int ACT>
__device__ __forceinline__ float apply_act_t(float v, const Epilogue& e, float p0, float p1, float p2) {
  if constexpr (ACT == BZ_ACT_PRELU) {
    return v * ((float)(v > 0.f) + (float)(v < 0.f) * p0);
  } else if constexpr (ACT == BZ_ACT_DICE) {
    const float t = __builtin_amdgcn_exp2f((p1 - v) * p2);  // e^((mean - v) / den)
    const float p = __builtin_amdgcn_rcpf(1.f + t);
    return fmaf(p, 1.f - p0, p0) * v;  // ((1 - p) gamma + p) v; 1 - gamma is the column's, hoisted out of the rows
  } else if constexpr (ACT == BZ_ACT_LEAKY_RELU) {
    return v >= 0.f ? v : e.act_alpha * v;
  } else if constexpr (ACT == BZ_ACT_SIGMOID) {
    const float t = expf(v);
    return t / (1.f + t);
  } else {
    return v;
  }
}

template <typename OutT>
__device__ __forceinline__ void store_out(OutT* p, float v);
template <>
__device__ __forceinline__ void store_out<float>(float* p, float v) {
  *p = v;
}
template <>
__device__ __forceinline__ void store_out<__half>(__half* p, float v) {
  *p = __float2half_rn(v);
}
template <>
__device__ __forceinline__ void store_out<__hip_bfloat16>(__hip_bfloat16* p, float v) {
  *p = __float2bfloat16(v);
}

// ---------------------------------------------------------------------------------------------
// element traits
// ---------------------------------------------------------------------------------------------
template <int DT>
struct In;
template <>
struct In<BZ_F16> {
  static constexpr int kSize = 2;
  static constexpr int kChunk = 8;   // elements per 16 bytes
  static constexpr int kStepK = 16;  // K consumed per fragment pair (both lane halves)
  static __device__ __forceinline__ void mma(const uint4& a, const uint4& b, floatx16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(*(const half8*)&a, *(const half8*)&b, acc, 0, 0, 0);
  }
};
template <>
struct In<BZ_BF16> {
  static constexpr int kSize = 2;
  static constexpr int kChunk = 8;
  static constexpr int kStepK = 16;
  static __device__ __forceinline__ void mma(const uint4& a, const uint4& b, floatx16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)&a, *(const bf16x8*)&b, acc, 0, 0, 0);
  }
};
template <>
struct In<BZ_F32> {
  static constexpr int kSize = 4;
  static constexpr int kChunk = 4;
  static constexpr int kStepK = 8;
  // lane half h holds k = 4h..4h+3 of the 8-wide step; instruction i multiplies element i of both
  // halves, i.e. k in {i, 4+i}: a permutation of k applied equally to A and W.
  static __device__ __forceinline__ void mma(const uint4& a, const uint4& b, floatx16& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), acc, 0, 0, 0);
  }
};


constexpr int kSkinnyMaxN = 8;

}  // namespace fc

// fc_pieces.hip: the layer whose A operand is given as pieces (bz_fc_desc.a_pieces); called by bz_fc_fused after its
// argument checks
int fc_pieces_launch(const bz_fc_desc& d, const fc::Epilogue& ep, hipStream_t st);
// The layer on a stored A, one function per operand type (fc_fused_f16.hip, fc_fused_bf16.hip, fc_fused_f32.hip): with a
// head when d.head_n != 0, else the skinny, tile or streaming kernel.  bz_fc_fused has checked the descriptor.
int fc_run_f16(const bz_fc_desc& d, const fc::Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st);
int fc_run_bf16(const bz_fc_desc& d, const fc::Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st);
int fc_run_f32(const bz_fc_desc& d, const fc::Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st);

}  // namespace bz
