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

// One wave per batch item, lanes over the channels.  Both sums walk t in ascending order, the weighted one with the
// fused multiply-add bz_bgemm_kernel uses for C = A^T * B, the plain one with separate adds like bz_reduce_sum_kernel,
// and the weight is rounded to the tensor type first, as the Mul operator would have stored it: the results are the
// three operators' results bit for bit.
// (a history of 50 in one round of loads: with one wave per item and four waves per CU the kernel is a chain of
// round trips to memory, 10 us at 16 steps per round on [1024, 50, 54])
constexpr int kPoolUnroll = 64;

template <typename T>
__global__ __launch_bounds__(256) void bz_weighted_pool_kernel(const T* __restrict__ w, const T* __restrict__ mask,
                                                               const T* __restrict__ x, T* __restrict__ att, T* __restrict__ sum,
                                                               int64_t batch, int t_len, int c_len, int64_t ld_att, int64_t ld_sum,
                                                               const T* __restrict__ copy_src, T* __restrict__ copy_dst, int copy_c,
                                                               int64_t ld_copy_src, int64_t ld_copy_dst) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * 4 + wave;
  if (item >= batch) return;
  // the piece copied alongside (asked for first: its loads travel with the history's)
  for (int c = lane; c < copy_c; c += 64) copy_dst[item * ld_copy_dst + c] = copy_src[item * ld_copy_src + c];
  const T* wp = w + item * t_len;
  const T* mp = mask ? mask + item * t_len : nullptr;
  const T* xp = x + item * (int64_t)t_len * c_len;
  // The channel loop is uniform over the wave: every lane runs every pass, so that lane u holds the weight of step
  // t0 + u when it is read with v_readlane below, whatever c_len is; a lane past the last channel reads the last
  // channel's address and stores nothing.
  for (int c0 = 0; c0 < c_len; c0 += 64) {
    const bool live = c0 + lane < c_len;
    const int c = live ? c0 + lane : c_len - 1;
    float acc_w = 0.f, acc_s = 0.f;
    for (int t0 = 0; t0 < t_len; t0 += kPoolUnroll) {
      // lane l fetches the weight of step t0 + l (every lane needs every weight: they are handed round below), then
      // its own channel of all the steps; nothing is used before everything has been asked for
      const int tl = t0 + lane < t_len ? t0 + lane : t_len - 1;
      const float w_raw = ld<T>(wp + tl);
      const float m_raw = mp ? ld<T>(mp + tl) : 1.f;
      float xv[kPoolUnroll];
#pragma unroll
      for (int u = 0; u < kPoolUnroll; ++u) {
        const int t = t0 + u < t_len ? t0 + u : t_len - 1;  // clamped address; the term is skipped below
        xv[u] = ld<T>(xp + (int64_t)t * c_len + c);
      }
      float w_mine = w_raw;
      if (mp) {
        T r;
        st<T>(&r, __fmul_rn(w_raw, m_raw));
        w_mine = ld<T>(&r);
      }
#pragma unroll
      for (int u = 0; u < kPoolUnroll; ++u)
        if (t0 + u < t_len) {
          const float wu = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w_mine), u));
          acc_w = fmaf(wu, xv[u], acc_w);
          acc_s = __fadd_rn(acc_s, xv[u]);
        }
    }
    if (live && att) st<T>(att + item * ld_att + c, acc_w);
    if (live && sum) st<T>(sum + item * ld_sum + c, acc_s);
  }
}

}  // namespace

extern "C" int bz_weighted_pool(const bz_weighted_pool_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_weighted_pool: null descriptor");
  const bz_weighted_pool_desc& d = *desc;
  BZ_REQUIRE(d.x != nullptr && (d.att != nullptr || d.sum != nullptr), "bz_weighted_pool: null x, or neither output asked for");
  BZ_REQUIRE(d.att == nullptr || d.w != nullptr, "bz_weighted_pool: the weighted sum needs w");
  BZ_REQUIRE(d.batch >= 0 && d.t > 0 && d.c > 0, "bz_weighted_pool: bad shape batch=%lld t=%d c=%d", (long long)d.batch, d.t, d.c);
  const int64_t ld_att = d.ld_att ? d.ld_att : d.c, ld_sum = d.ld_sum ? d.ld_sum : d.c;
  const int64_t ld_cs = d.ld_copy_src ? d.ld_copy_src : d.copy_c, ld_cd = d.ld_copy_dst ? d.ld_copy_dst : d.copy_c;
  BZ_REQUIRE(ld_att >= d.c && ld_sum >= d.c, "bz_weighted_pool: ld_att=%lld / ld_sum=%lld below c=%d", (long long)ld_att, (long long)ld_sum, d.c);
  BZ_REQUIRE(d.copy_c >= 0 && (d.copy_c == 0 || (d.copy_src != nullptr && d.copy_dst != nullptr && ld_cs >= d.copy_c && ld_cd >= d.copy_c)),
             "bz_weighted_pool: copied piece of %d elements with a null pointer or a leading dimension below it", d.copy_c);
  if (d.batch == 0) return BZ_OK;
  BZ_REQUIRE((d.batch + 3) / 4 < (1ll << 31), "bz_weighted_pool: batch %lld too large", (long long)d.batch);
  const int grid = (int)((d.batch + 3) / 4);
  hipStream_t s = bz::as_stream(stream);
  const void* w = d.att ? d.w : d.x;  // no weighted sum: any readable address of t elements per item will do
  if (d.dtype == BZ_F32)
    hipLaunchKernelGGL(bz_weighted_pool_kernel<float>, dim3(grid), dim3(256), 0, s, (const float*)w, (const float*)(d.att ? d.mask : nullptr),
                       (const float*)d.x, (float*)d.att, (float*)d.sum, d.batch, d.t, d.c, ld_att, ld_sum, (const float*)d.copy_src,
                       (float*)d.copy_dst, d.copy_c, ld_cs, ld_cd);
  else if (d.dtype == BZ_F16)
    hipLaunchKernelGGL(bz_weighted_pool_kernel<__half>, dim3(grid), dim3(256), 0, s, (const __half*)w,
                       (const __half*)(d.att ? d.mask : nullptr), (const __half*)d.x, (__half*)d.att, (__half*)d.sum, d.batch, d.t, d.c,
                       ld_att, ld_sum, (const __half*)d.copy_src, (__half*)d.copy_dst, d.copy_c, ld_cs, ld_cd);
  else
    return bz::fail(BZ_ENOTSUP, "bz_weighted_pool: unsupported dtype %d", d.dtype);
  BZ_LAUNCH_OK("bz_weighted_pool_kernel");
  return BZ_OK;
}

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
