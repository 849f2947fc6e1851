// Device side of the synthetic-workload generator (x-deeplearning_amd/philox.py): fills tensors that are too large to
// come from the host (config 4's 34 GB and config 5's 102 GB of tables) with Philox4x32-10 draws.  Element e of a
// stream is word e % 4 of call e / 4; call i has counter (i mod 2^32, i div 2^32, stream id, 0) and key (seed mod 2^32,
// seed div 2^32).  Only integer arithmetic, a table lookup and single correctly rounded float operations are used, so
// the host recomputes any element bit for bit.  Harness code: built into lib/libblaze_synth.so, not into the drop-in
// library.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

struct Words {
  uint32_t w[4];
};

__device__ __forceinline__ Words philox4x32_10(uint64_t call, uint32_t stream, uint64_t seed) {
  uint32_t c0 = (uint32_t)call, c1 = (uint32_t)(call >> 32), c2 = stream, c3 = 0;
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    if (r) {
      k0 += 0x9E3779B9u;
      k1 += 0xBB67AE85u;
    }
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
  }
  return {{c0, c1, c2, c3}};
}

enum { kNormalF32 = 0, kNormalF16 = 1, kInt8 = 2, kUniformF32 = 3 };

// One thread per call: up to four consecutive elements.  `first` need not be a multiple of 4: the thread's elements are
// those of its call that fall into [first, first + n).
template <int KIND>
__global__ __launch_bounds__(256) void bz_synth_fill_kernel(void* out, int64_t n, int64_t first, uint64_t seed, uint32_t stream, float a,
                                                            float b, const float* __restrict__ quantiles) {
  const int64_t call0 = first >> 2;
  const int64_t ncalls = ((first + n + 3) >> 2) - call0;
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < ncalls; t += (int64_t)gridDim.x * blockDim.x) {
    const Words x = philox4x32_10((uint64_t)(call0 + t), stream, seed);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t e = ((call0 + t) << 2) + j - first;
      if (e < 0 || e >= n) continue;
      const uint32_t w = x.w[j];
      if constexpr (KIND == kNormalF32) {
        ((float*)out)[e] = __fmul_rn(quantiles[w >> 16], a);
      } else if constexpr (KIND == kNormalF16) {
        // the product is rounded to float first and then to half, as numpy does it: without the opaque copy the compiler
        // joins the two into v_fma_mixlo_f16, which rounds the exact product once and differs in the double-rounding cases
        float x = __fmul_rn(quantiles[w >> 16], a);
        asm volatile("" : "+v"(x));
        ((__half*)out)[e] = __float2half_rn(x);
      } else if constexpr (KIND == kInt8) {
        ((int8_t*)out)[e] = (int8_t)((int)(((uint64_t)w * 255u) >> 32) - 127);
      } else {
        const float u = __fmul_rn((float)(w >> 8), 5.9604644775390625e-08f);  // 2^-24, exact
        ((float*)out)[e] = __fadd_rn(a, __fmul_rn(u, __fsub_rn(b, a)));
      }
    }
  }
}

}  // namespace

extern "C" __attribute__((visibility("default"))) int bz_synth_fill(void* out, int kind, int64_t n, int64_t first, uint64_t seed,
                                                                     uint32_t stream, float a, float b, const float* quantiles,
                                                                     void* hip_stream) {
  if (out == nullptr || n < 0 || first < 0 || kind < 0 || kind > 3 || ((kind == kNormalF32 || kind == kNormalF16) && quantiles == nullptr))
    return -22;
  if (n == 0) return 0;
  const int64_t ncalls = ((first + n + 3) >> 2) - (first >> 2);
  int64_t grid = (ncalls + 255) / 256;
  if (grid > 256 * 64) grid = 256 * 64;
  hipStream_t st = (hipStream_t)hip_stream;
  switch (kind) {
    case kNormalF32: hipLaunchKernelGGL(bz_synth_fill_kernel<kNormalF32>, dim3((int)grid), dim3(256), 0, st, out, n, first, seed, stream, a, b, quantiles); break;
    case kNormalF16: hipLaunchKernelGGL(bz_synth_fill_kernel<kNormalF16>, dim3((int)grid), dim3(256), 0, st, out, n, first, seed, stream, a, b, quantiles); break;
    case kInt8: hipLaunchKernelGGL(bz_synth_fill_kernel<kInt8>, dim3((int)grid), dim3(256), 0, st, out, n, first, seed, stream, a, b, quantiles); break;
    default: hipLaunchKernelGGL(bz_synth_fill_kernel<kUniformF32>, dim3((int)grid), dim3(256), 0, st, out, n, first, seed, stream, a, b, quantiles); break;
  }
  return hipGetLastError() == hipSuccess ? 0 : -5;
}
