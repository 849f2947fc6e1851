// fc_fused.hip -- bz_fc_fused: argument checks and the choice of path for an FC layer (GEMM + bias + activation in one
// kernel).  The kernels are in fc_fused_impl.h, compiled once per operand type; a layer on a_pieces goes to
// fc_pieces.hip.  bz_fc_pack_weight is here as well.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "bz_common.h"
#include "fc_common.h"

namespace {

using namespace bz::fc;

// ---------------------------------------------------------------------------------------------
// weight packing
// ---------------------------------------------------------------------------------------------
template <typename SrcT, typename DstT>
__global__ void bz_pack_weight_kernel(const SrcT* __restrict__ src, DstT* __restrict__ dst, int K, int N, int64_t ldw,
                                      int trans_b) {
  const int64_t total = (int64_t)N * ldw;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t n = i / ldw, k = i % ldw;
    float v = 0.f;
    if (k < K) v = (float)src[trans_b ? n * K + k : k * (int64_t)N + n];
    dst[i] = (DstT)v;
  }
}


}  // namespace

extern "C" {

int bz_fc_fused(const bz_fc_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_fc_fused: null descriptor");
  const bz_fc_desc& d = *desc;
  BZ_REQUIRE((d.a || d.a_pieces) && d.w && (d.y || d.head_n > 0 || d.next), "bz_fc_fused: null a/w/y");
  BZ_REQUIRE(d.next == nullptr || d.a_pieces != nullptr, "bz_fc_fused: a second layer (next) only follows a layer on a_pieces");
  BZ_REQUIRE(d.m >= 0 && d.n > 0 && d.k > 0, "bz_fc_fused: bad shape m=%d n=%d k=%d", d.m, d.n, d.k);
  BZ_REQUIRE(d.n_split >= 0 && (d.n_split == 0 || (d.n % d.n_split == 0 && d.y_split_stride >= 0)),
             "bz_fc_fused: n_split=%d must divide n=%d", d.n_split, d.n);
  BZ_REQUIRE(d.n_split == 0 || (d.head_n == 0 && d.act != BZ_ACT_SOFTMAX), "bz_fc_fused: split outputs take no head and no softmax");
  BZ_REQUIRE((d.a_pieces != nullptr || d.lda >= d.k) && d.ldw >= d.k && d.ldy >= (d.n_split ? d.n_split : d.n),
             "bz_fc_fused: leading dimension smaller than row (lda=%lld ldw=%lld ldy=%lld)", (long long)d.lda, (long long)d.ldw,
             (long long)d.ldy);
  BZ_REQUIRE(d.in_dtype == BZ_F16 || d.in_dtype == BZ_BF16 || d.in_dtype == BZ_F32, "bz_fc_fused: unsupported in dtype %d",
             d.in_dtype);
  BZ_REQUIRE(d.bias_rows == 0 || d.bias != nullptr, "bz_fc_fused: bias_rows=%d without bias", d.bias_rows);
  BZ_REQUIRE(d.bias_rows == 0 || d.bias_rows == 1 || d.bias_rows == d.m, "bz_fc_fused: bias_rows=%d must be 0, 1 or m=%d",
             d.bias_rows, d.m);
  switch (d.act) {
    case BZ_ACT_NONE:
    case BZ_ACT_LEAKY_RELU:
    case BZ_ACT_SIGMOID:
      break;
    case BZ_ACT_PRELU:
      BZ_REQUIRE(d.act_p0 && (d.act_size == 1 || d.act_size == d.n), "bz_fc_fused: PRelu slope size %d must be 1 or n=%d",
                 d.act_size, d.n);
      break;
    case BZ_ACT_DICE:
      BZ_REQUIRE(d.act_p0 && d.act_p1 && d.act_p2, "bz_fc_fused: Dice needs gamma, mean and var");
      break;
    case BZ_ACT_SOFTMAX:
      if (d.n > kSkinnyMaxN) return bz::fail(BZ_ENOTSUP, "bz_fc_fused: fused softmax needs n <= %d (n=%d)", kSkinnyMaxN, d.n);
      break;
    default:
      return bz::fail(BZ_EINVAL, "bz_fc_fused: unknown activation %d", d.act);
  }
  if (d.m == 0) return BZ_OK;
  Epilogue ep;
  ep.bias = (const float*)d.bias;
  ep.p0 = d.act_p0;
  ep.p1 = d.act_p1;
  ep.p2 = d.act_p2;
  ep.bias_rows = d.bias_rows;
  ep.act = d.act;
  ep.act_size = d.act_size;
  ep.dice_nosqrt = d.dice_nosqrt;
  ep.alpha = d.alpha;
  ep.beta = d.beta;
  ep.act_alpha = d.act_alpha;
  ep.split_n = d.n_split;
  ep.split_stride = d.y_split_stride;
  const int es = bz::dtype_size(d.in_dtype);
  const bool vec_a = ((uintptr_t)d.a % 16 == 0) && ((d.lda * es) % 16 == 0);
  const bool vec_w = ((uintptr_t)d.w % 16 == 0) && ((d.ldw * es) % 16 == 0);
  hipStream_t st = bz::as_stream(stream);
  if (d.a_pieces != nullptr) {
    if ((d.head_n != 0 && d.next == nullptr) || d.n_split != 0 || d.bias_rows > 1 || d.act == BZ_ACT_SOFTMAX || es != 2 || !vec_w)
      return bz::fail(BZ_ENOTSUP, "bz_fc_fused: a_pieces take a 2-byte layer with aligned weight rows, no head, no split outputs, no softmax and a per-column bias");
    return bz::fc_pieces_launch(d, ep, st);
  }
  if (d.head_n != 0) {
    const int chunk = 16 / es;
    BZ_REQUIRE(d.head_n > 0 && d.head_n <= kSkinnyMaxN && d.head_w && d.head_y, "bz_fc_fused: head of %d outputs (1..%d) or null head_w/head_y",
               d.head_n, kSkinnyMaxN);
    if (d.n > 256 || d.n <= kSkinnyMaxN || d.n % chunk != 0)
      return bz::fail(BZ_ENOTSUP, "bz_fc_fused: a fused head needs %d < n <= 256 and n a multiple of %d (n=%d)", kSkinnyMaxN, chunk, d.n);
    if (!(vec_a && vec_w && d.k % chunk == 0))
      return bz::fail(BZ_ENOTSUP, "bz_fc_fused: a fused head needs 16-byte aligned operand rows and k a multiple of %d", chunk);
    BZ_REQUIRE(d.out_dtype == d.in_dtype, "bz_fc_fused: with a fused head the layer's output type must be its input type");
    BZ_REQUIRE(d.act != BZ_ACT_SOFTMAX && (d.bias_rows == 0 || d.bias_rows == 1), "bz_fc_fused: fused head after softmax or a full bias");
    BZ_REQUIRE(d.head_act == BZ_ACT_NONE || d.head_act == BZ_ACT_SIGMOID || d.head_act == BZ_ACT_SOFTMAX,
               "bz_fc_fused: head activation %d (none, sigmoid or softmax)", d.head_act);
    BZ_REQUIRE(d.head_ldw >= d.n && (d.head_ldw * es) % 16 == 0 && (uintptr_t)d.head_w % 16 == 0 && d.head_ldy >= d.head_n,
               "bz_fc_fused: head_ldw=%lld (>= n, rows 16-byte aligned) head_ldy=%lld (>= head_n)", (long long)d.head_ldw,
               (long long)d.head_ldy);
    BZ_REQUIRE(d.head_out_dtype == BZ_F32 || d.head_out_dtype == BZ_F16 || d.head_out_dtype == BZ_BF16, "bz_fc_fused: head out dtype %d",
               d.head_out_dtype);
  }
  switch (d.in_dtype) {
    case BZ_F16: return bz::fc_run_f16(d, ep, vec_a, vec_w, st);
    case BZ_BF16: return bz::fc_run_bf16(d, ep, vec_a, vec_w, st);
    default: return bz::fc_run_f32(d, ep, vec_a, vec_w, st);
  }
}

int bz_fc_pack_weight(const void* src, int src_dtype, int trans_b, int k, int n, void* dst, int dst_dtype, int64_t ldw,
                      bz_stream_t stream) {
  BZ_REQUIRE(src && dst && k > 0 && n > 0, "bz_fc_pack_weight: null pointer or bad shape k=%d n=%d", k, n);
  BZ_REQUIRE(ldw >= k && ldw % 8 == 0, "bz_fc_pack_weight: ldw=%lld must be >= k=%d and a multiple of 8", (long long)ldw, k);
  const int64_t total = (int64_t)n * ldw;
  const int grid = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
  hipStream_t st = bz::as_stream(stream);
#define BZ_PACK(S, D)                                                                                        \
  hipLaunchKernelGGL((bz_pack_weight_kernel<S, D>), dim3(grid), dim3(256), 0, st, (const S*)src, (D*)dst, k, n, ldw, \
                     trans_b)
  if (src_dtype == BZ_F32 && dst_dtype == BZ_F32)
    BZ_PACK(float, float);
  else if (src_dtype == BZ_F32 && dst_dtype == BZ_F16)
    BZ_PACK(float, _Float16);
  else if (src_dtype == BZ_F32 && dst_dtype == BZ_BF16)
    BZ_PACK(float, __bf16);
  else if (src_dtype == BZ_F16 && dst_dtype == BZ_F16)
    BZ_PACK(_Float16, _Float16);
  else if (src_dtype == BZ_F16 && dst_dtype == BZ_F32)
    BZ_PACK(_Float16, float);
  else if (src_dtype == BZ_BF16 && dst_dtype == BZ_BF16)
    BZ_PACK(__bf16, __bf16);
  else
    return bz::fail(BZ_ENOTSUP, "bz_fc_pack_weight: no conversion %d -> %d", src_dtype, dst_dtype);
#undef BZ_PACK
  BZ_LAUNCH_OK("bz_pack_weight_kernel");
  return BZ_OK;
}

}  // extern "C"
