// activation.hip -- standalone PRelu / Dice / LeakyRelu / Sigmoid / Softmax over a [rows, cols]
// tensor, for graphs where the producer is not a Gemm (otherwise they ride in the FC epilogue).
// Formulas follow the reference's CPU operators: prelu_op.cc:11-30 (math/activation.h:37-42),
// dice_op.cc:15-34, leaky_relu_op.cc:15-21 (math/activation.h:29-34), sigmoid_op.cc:15-21,
// softmax_op.cc:21-78 (axis = last).  All arithmetic in fp32; bandwidth bound (one read, one write).
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include "bz_common.h"

namespace {

constexpr float kDiceEps = 1e-8f;  // blaze/operator/common_helper.h:90

struct ActP {
  const float* p0;
  const float* p1;
  const float* p2;
  int act, act_size, nosqrt;
  float alpha;
};

template <typename T>
__device__ __forceinline__ float ldf(const T* p);
template <>
__device__ __forceinline__ float ldf<float>(const float* p) {
  return *p;
}
template <>
__device__ __forceinline__ float ldf<__half>(const __half* p) {
  return __half2float(*p);
}
template <typename T>
__device__ __forceinline__ void stf(T* p, float v);
template <>
__device__ __forceinline__ void stf<float>(float* p, float v) {
  *p = v;
}
template <>
__device__ __forceinline__ void stf<__half>(__half* p, float v) {
  *p = __float2half_rn(v);
}

template <typename T>
__global__ __launch_bounds__(256) void bz_act_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t total, int64_t cols,
                                                     ActP a) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const float v = ldf<T>(x + i);
    float r = v;
    switch (a.act) {
      case BZ_ACT_PRELU: {
        const float w = a.p0[i % a.act_size];  // slope broadcast over the trailing dims
        r = v * ((float)(v > 0.f) + (float)(v < 0.f) * w);
        break;
      }
      case BZ_ACT_DICE: {
        const int64_t c = i % cols;
        const float den = a.nosqrt ? a.p2[c] : sqrtf(a.p2[c] + kDiceEps);
        const float t = expf(-1.f * (v - a.p1[c]) / den);
        const float p = 1.f / (1.f + t);
        r = (1.f - p) * a.p0[c] * v + p * v;
        break;
      }
      case BZ_ACT_LEAKY_RELU:
        r = v >= 0.f ? v : a.alpha * v;
        break;
      case BZ_ACT_SIGMOID: {
        const float t = expf(v);
        r = t / (1.f + t);
        break;
      }
      default:
        break;
    }
    stf<T>(y + i, r);
  }
}

// one wavefront per row; max, then exp/sum, then divide
template <typename T>
__global__ __launch_bounds__(256) void bz_softmax_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows,
                                                         int64_t cols) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + row * cols;
  T* yr = y + row * cols;
  float mx = -INFINITY;
  for (int64_t c = lane; c < cols; c += 64) mx = fmaxf(mx, ldf<T>(xr + c));
  for (int d = 32; d > 0; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
  float sum = 0.f;
  for (int64_t c = lane; c < cols; c += 64) sum += expf(ldf<T>(xr + c) - mx);
  for (int d = 32; d > 0; d >>= 1) sum += __shfl_xor(sum, d, 64);
  for (int64_t c = lane; c < cols; c += 64) stf<T>(yr + c, expf(ldf<T>(xr + c) - mx) / sum);
}

// side-by-side concatenation: blockIdx.y picks the piece; a thread copies the widest power-of-two granule (16 ... 1
// bytes) that the piece's addresses, width and both pitches are all multiples of
template <typename G>
__device__ __forceinline__ void concat_piece(const char* src, char* dst, int64_t width, int64_t sp, int64_t dp, int64_t rows) {
  const int64_t cpr = width / (int64_t)sizeof(G), total = cpr * rows;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / cpr, c = i - r * cpr;
    *(G*)(dst + r * dp + c * sizeof(G)) = *(const G*)(src + r * sp + c * sizeof(G));
  }
}

__global__ __launch_bounds__(256) void bz_concat_kernel(bz_concat_desc d) {
  const int k = blockIdx.y;
  const char* src = (const char*)d.src[k];
  const int64_t width = d.width[k];
  int64_t col = 0;
  for (int i = 0; i < k; ++i) col += d.width[i];
  char* dst = (char*)d.dst + col;
  const int64_t sp = d.src_pitch[k];
  const uint64_t all = (uint64_t)(uintptr_t)src | (uint64_t)(uintptr_t)dst | (uint64_t)width | (uint64_t)d.dst_pitch | (uint64_t)sp;
  if (all % 16 == 0)
    concat_piece<uint4>(src, dst, width, sp, d.dst_pitch, d.rows);
  else if (all % 8 == 0)
    concat_piece<uint2>(src, dst, width, sp, d.dst_pitch, d.rows);
  else if (all % 4 == 0)
    concat_piece<uint32_t>(src, dst, width, sp, d.dst_pitch, d.rows);
  else if (all % 2 == 0)
    concat_piece<uint16_t>(src, dst, width, sp, d.dst_pitch, d.rows);
  else
    concat_piece<uint8_t>(src, dst, width, sp, d.dst_pitch, d.rows);
}

}  // namespace

extern "C" int bz_concat_cols(const bz_concat_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_concat_cols: null descriptor");
  const bz_concat_desc& d = *desc;
  BZ_REQUIRE(d.n > 0 && d.n <= BZ_CONCAT_MAX && d.dst != nullptr && d.rows >= 0, "bz_concat_cols: n=%d rows=%lld", d.n,
             (long long)d.rows);
  int64_t total = 0, widest = 0;
  for (int i = 0; i < d.n; ++i) {
    BZ_REQUIRE(d.width[i] >= 0 && (d.width[i] == 0 || d.src[i] != nullptr), "bz_concat_cols: piece %d is null", i);
    BZ_REQUIRE(d.src_pitch[i] == 0 || d.src_pitch[i] >= d.width[i], "bz_concat_cols: piece %d has pitch %lld < width %lld", i,
               (long long)d.src_pitch[i], (long long)d.width[i]);
    total += d.width[i];
    widest = d.width[i] > widest ? d.width[i] : widest;
  }
  BZ_REQUIRE(total <= d.dst_pitch, "bz_concat_cols: pieces are %lld bytes wide, output rows only %lld", (long long)total,
             (long long)d.dst_pitch);
  if (d.rows == 0 || widest == 0) return BZ_OK;
  const int64_t work = (widest / 16 + 1) * d.rows;
  const int gx = (int)(((work + 255) / 256) < 2048 ? ((work + 255) / 256) : 2048);
  hipLaunchKernelGGL(bz_concat_kernel, dim3(gx, d.n), dim3(256), 0, bz::as_stream(stream), d);
  BZ_LAUNCH_OK("bz_concat_kernel");
  return BZ_OK;
}

extern "C" int bz_activation(const bz_act_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_activation: null descriptor");
  const bz_act_desc& d = *desc;
  BZ_REQUIRE(d.x && d.y && d.rows >= 0 && d.cols > 0, "bz_activation: null x/y or bad shape");
  BZ_REQUIRE(d.dtype == BZ_F32 || d.dtype == BZ_F16, "bz_activation: unsupported dtype %d", d.dtype);
  if (d.rows == 0) return BZ_OK;
  hipStream_t s = bz::as_stream(stream);
  const int64_t total = d.rows * d.cols;
  if (d.act == BZ_ACT_SOFTMAX) {
    const int grid = (int)((d.rows + 3) / 4);
    if (d.dtype == BZ_F32)
      hipLaunchKernelGGL(bz_softmax_kernel<float>, dim3(grid), dim3(256), 0, s, (const float*)d.x, (float*)d.y, d.rows, d.cols);
    else
      hipLaunchKernelGGL(bz_softmax_kernel<__half>, dim3(grid), dim3(256), 0, s, (const __half*)d.x, (__half*)d.y, d.rows,
                         d.cols);
    BZ_LAUNCH_OK("bz_softmax_kernel");
    return BZ_OK;
  }
  ActP a;
  a.p0 = d.p0;
  a.p1 = d.p1;
  a.p2 = d.p2;
  a.act = d.act;
  a.act_size = d.act_size;
  a.nosqrt = d.dice_nosqrt;
  a.alpha = d.act_alpha;
  switch (d.act) {
    case BZ_ACT_NONE:
    case BZ_ACT_LEAKY_RELU:
    case BZ_ACT_SIGMOID:
      break;
    case BZ_ACT_PRELU:
      BZ_REQUIRE(d.p0 && d.act_size > 0 && total % d.act_size == 0, "bz_activation: PRelu slope size %d does not divide %lld",
                 d.act_size, (long long)total);
      break;
    case BZ_ACT_DICE:
      BZ_REQUIRE(d.p0 && d.p1 && d.p2, "bz_activation: Dice needs gamma, mean and var");
      break;
    default:
      return bz::fail(BZ_EINVAL, "bz_activation: unknown activation %d", d.act);
  }
  const int64_t want = (total + 255) / 256;
  const int grid = (int)(want < 256 * 16 ? want : 256 * 16);
  if (d.dtype == BZ_F32)
    hipLaunchKernelGGL(bz_act_kernel<float>, dim3(grid), dim3(256), 0, s, (const float*)d.x, (float*)d.y, total, d.cols, a);
  else
    hipLaunchKernelGGL(bz_act_kernel<__half>, dim3(grid), dim3(256), 0, s, (const __half*)d.x, (__half*)d.y, total, d.cols, a);
  BZ_LAUNCH_OK("bz_act_kernel");
  return BZ_OK;
}
