// bgemm.hip -- strided-batched small GEMM for gfx950: C[i] = alpha*op(A[i])*op(B[i]) + beta*C[i].
//
// Stands in for GemmStridedBatched (blaze/math/gemm.cc:82-139, gemm.cu:251-336) as the
// reference reaches it from MatMul / BroadcastGemm_NxN (blaze/operator/op/matmul_op.h:77-89,
// blaze/math/broadcast.h:157-222), FusedParallelGemm (fused_parallel_gemm_op.h:96-129) and
// FusedParallelMatMul / BatchedBroadcastGemm_NxN (blaze/math/broadcast.h:267-381).
//
// On this path the matrices are tiny (the DIN attention sum is 1xT . TxD with T<=50, D=54):
// the work is one pass over B, i.e. memory bound.  One wavefront owns one batch item; its
// lanes own output elements (m,n) with n fastest, so reads of a non-transposed B row and
// writes of C are contiguous; A values are wave-uniform broadcasts.  fp32 accumulate in
// ascending k.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include "bz_common.h"

namespace {

template <typename T>
__device__ __forceinline__ float ld(const T* p);
template <>
__device__ __forceinline__ float ld<float>(const float* p) {
  return *p;
}
template <>
__device__ __forceinline__ float ld<__half>(const __half* p) {
  return __half2float(*p);
}
template <typename T>
__device__ __forceinline__ void st(T* p, float v);
template <>
__device__ __forceinline__ void st<float>(float* p, float v) {
  *p = v;
}
template <>
__device__ __forceinline__ void st<__half>(__half* p, float v) {
  *p = __float2half_rn(v);
}

// One wave per batch item, one lane per output element; K is walked in steps of kUnroll with all loads of a step
// issued before the first multiply-add (the products are still added in ascending k, so the sum is the plain loop's).
constexpr int kUnroll = 16;

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(256) void bz_bgemm_kernel(const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C,
                                                       int64_t sa, int64_t sb, int64_t sc, int M, int N, int K, int batch,
                                                       float alpha, float beta) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= batch) return;
  const T* a = A + sa * item;
  const T* b = B + sb * item;
  T* c = C + sc * item;
  const int lda = TA ? M : K, ldb = TB ? K : N;
  for (int e = lane; e < M * N; e += 64) {
    const int m = e / N, n = e - m * N;
    const T* ap = TA ? a + m : a + (int64_t)m * lda;  // element k: ap[k * (TA ? lda : 1)]
    const T* bp = TB ? b + (int64_t)n * ldb : b + n;  // element k: bp[k * (TB ? 1 : ldb)]
    const int64_t as = TA ? lda : 1, bs = TB ? 1 : ldb;
    float acc = 0.f;
    for (int k0 = 0; k0 < K; k0 += kUnroll) {
      float av[kUnroll], bv[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int k = k0 + u < K ? k0 + u : K - 1;  // clamped address; the product is skipped below
        av[u] = ld<T>(ap + k * as);
        bv[u] = ld<T>(bp + k * bs);
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        if (k0 + u < K) acc = fmaf(av[u], bv[u], acc);
    }
    float v = alpha * acc;
    if (beta != 0.f) v += beta * ld<T>(c + e);  // beta == 0: C is not read (BLAS rule)
    st<T>(c + e, v);
  }
}

template <typename T>
void launch_bgemm(const bz_bgemm_desc& d, int grid, hipStream_t s) {
#define BZ_BGEMM(TA, TB)                                                                                                     \
  hipLaunchKernelGGL((bz_bgemm_kernel<T, TA, TB>), dim3(grid), dim3(256), 0, s, (const T*)d.a, (const T*)d.b, (T*)d.c, d.stride_a, \
                     d.stride_b, d.stride_c, d.m, d.n, d.k, d.batch, d.alpha, d.beta)
  if (d.trans_a && d.trans_b)
    BZ_BGEMM(true, true);
  else if (d.trans_a)
    BZ_BGEMM(true, false);
  else if (d.trans_b)
    BZ_BGEMM(false, true);
  else
    BZ_BGEMM(false, false);
#undef BZ_BGEMM
}

}  // namespace

extern "C" int bz_gemm_strided_batched(const bz_bgemm_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_gemm_strided_batched: null descriptor");
  const bz_bgemm_desc& d = *desc;
  BZ_REQUIRE(d.a && d.b && d.c, "bz_gemm_strided_batched: null a/b/c");
  BZ_REQUIRE(d.m > 0 && d.n > 0 && d.k > 0 && d.batch >= 0, "bz_gemm_strided_batched: bad shape m=%d n=%d k=%d batch=%d",
             d.m, d.n, d.k, d.batch);
  BZ_REQUIRE((int64_t)d.m * d.n < (1ll << 31), "bz_gemm_strided_batched: m*n too large");
  BZ_REQUIRE(d.stride_c >= (int64_t)d.m * d.n || d.batch <= 1, "bz_gemm_strided_batched: outputs overlap (stride_c=%lld)",
             (long long)d.stride_c);
  if (d.batch == 0) return BZ_OK;
  const int grid = (d.batch + 3) / 4;
  hipStream_t s = bz::as_stream(stream);
  if (d.dtype == BZ_F32)
    launch_bgemm<float>(d, grid, s);
  else if (d.dtype == BZ_F16)
    launch_bgemm<__half>(d, grid, s);
  else
    return bz::fail(BZ_ENOTSUP, "bz_gemm_strided_batched: unsupported dtype %d", d.dtype);
  BZ_LAUNCH_OK("bz_bgemm_kernel");
  return BZ_OK;
}
