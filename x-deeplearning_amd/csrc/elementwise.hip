// elementwise.hip -- the shape / elementwise operators around DIN's attention unit, for gfx950.
//
// Add / Sub / Mul / Div / BroadcastTo / Where with multidirectional broadcasting
// (blaze/operator/op/elementwise_op.{h,cc,cu}, shape rule blaze/math/broadcast.h:39-67), ReduceSum
// (blaze/operator/op/reduce_sum_op.h:17-58, blaze/math/reduce.cc:13-29), BatchNormalization in its inference
// form (blaze/operator/op/batch_normalization_op.cc:11-18) and Softmax over an inner axis
// (blaze/operator/op/softmax_op.cc:21-78).  All of them are one read and one write per element: HBM bound.
//
// Broadcast kernel: the host merges adjacent output dims whose operand strides allow it, then dispatches on
// the merged dims (up to 6).  A thread owns `VEC` consecutive elements of the innermost merged dim, so the index
// decomposition is paid once per VEC elements.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "bz_common.h"
#include "bz_pieces.h"

namespace {

using bz::ldv;
using bz::stv;
using bz::CewP;
using bz::CewPack;

struct BcastP {
  int64_t dims[BZ_MAX_RANK];  // merged, outermost first; only [0, rank) valid
  int64_t sa[BZ_MAX_RANK], sb[BZ_MAX_RANK], sc[BZ_MAX_RANK];
  int rank;
  int op;
  int64_t total;  // number of output elements
};

// VEC consecutive output elements of the innermost dim per thread (the host picks a VEC that divides that dim).
template <typename T, typename CondT, int VEC>
__global__ __launch_bounds__(256) void bz_bcast_kernel(const void* __restrict__ a_, const T* __restrict__ b, const T* __restrict__ c,
                                                       T* __restrict__ out, BcastP p) {
  const int64_t nvec = p.total / VEC;
  for (int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * 256) {
    int64_t lin = v * VEC;
    int64_t oa = 0, ob = 0, oc = 0;
    int64_t rem = lin;
#pragma unroll
    for (int d = BZ_MAX_RANK - 1; d >= 0; --d) {
      if (d < p.rank) {
        const int64_t q = rem / p.dims[d];
        const int64_t i = rem - q * p.dims[d];
        rem = q;
        oa += i * p.sa[d];
        ob += i * p.sb[d];
        oc += i * p.sc[d];
      }
    }
    const int last = p.rank - 1;
    const int64_t ia = p.sa[last], ib = p.sb[last], ic = p.sc[last];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      float r;
      if (p.op == BZ_EW_WHERE) {
        const CondT cond = ((const CondT*)a_)[oa + e * ia];
        r = cond != 0 ? ldv<T>(b + ob + e * ib) : ldv<T>(c + oc + e * ic);
      } else {
        const float x = ldv<T>((const T*)a_ + oa + e * ia);
        if (p.op == BZ_EW_ASSIGN) {
          r = x;
        } else {
          const float y = ldv<T>(b + ob + e * ib);
          r = p.op == BZ_EW_ADD ? __fadd_rn(x, y) : p.op == BZ_EW_SUB ? __fsub_rn(x, y) : p.op == BZ_EW_MUL ? __fmul_rn(x, y) : __fdiv_rn(x, y);
        }
      }
      stv<T>(out + lin + e, r);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bz_reduce_sum_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t outer, int64_t dim,
                                                            int64_t inner) {
  const int64_t total = outer * inner;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t o = i / inner, k = i - o * inner;
    const T* p = x + o * dim * inner + k;
    float acc = 0.f;
    int64_t j = 0;
    for (; j + 4 <= dim; j += 4) {  // four loads in flight, added in order
      const float v0 = ldv<T>(p + (j + 0) * inner), v1 = ldv<T>(p + (j + 1) * inner);
      const float v2 = ldv<T>(p + (j + 2) * inner), v3 = ldv<T>(p + (j + 3) * inner);
      acc = __fadd_rn(__fadd_rn(__fadd_rn(__fadd_rn(acc, v0), v1), v2), v3);
    }
    for (; j < dim; ++j) acc = __fadd_rn(acc, ldv<T>(p + j * inner));
    stv<T>(y + i, acc);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void bz_batch_norm_kernel(const T* __restrict__ x, T* __restrict__ y, bz_bn_desc d) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < d.size; i += (int64_t)gridDim.x * 256) {
    const int64_t c = i % d.channels;
    const float den = d.nosqrt ? d.var[c] : __fsqrt_rn(__fadd_rn(d.var[c], d.eps));
    const float xn = __fdiv_rn(__fsub_rn(ldv<T>(x + i), d.mean[c]), den);
    stv<T>(y + i, __fadd_rn(__fmul_rn(d.gamma[c], xn), d.beta[c]));
  }
}

// one thread per (outer, inner) column of the axis: three passes over c values that stay in L1/L2
template <typename T>
__global__ __launch_bounds__(256) void bz_softmax_axis_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t outer, int64_t c,
                                                              int64_t inner) {
  const int64_t total = outer * inner;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t o = i / inner, k = i - o * inner;
    const T* xp = x + o * c * inner + k;
    T* yp = y + o * c * inner + k;
    float mx = ldv<T>(xp);
    for (int64_t j = 1; j < c; ++j) mx = fmaxf(mx, ldv<T>(xp + j * inner));
    float sum = 0.f;
    for (int64_t j = 0; j < c; ++j) sum += expf(ldv<T>(xp + j * inner) - mx);
    for (int64_t j = 0; j < c; ++j) stv<T>(yp + j * inner, expf(ldv<T>(xp + j * inner) - mx) / sum);
  }
}

int grid_for(int64_t work) {
  const int64_t want = (work + 255) / 256;
  return (int)(want < 1 ? 1 : (want < 256 * 32 ? want : 256 * 32));
}

// ---- concat of pieces computed on the fly -------------------------------------------------------------------
// VEC consecutive columns of one output row per lane (the host picks a VEC that divides every width, stride and
// address, so a lane's VEC elements are one aligned load or store).  A wave owns a row at a time: which row, and where
// its operands start, is worked out once per row for the whole wave; inside the row a lane only has to find its piece.
// (One flat index per thread cost two integer divisions per VEC elements and element-wise accesses: 24.7 us for the
// [51200, 216] fp16 attention input of a DIN model, whose 54-wide pieces allow no more than VEC = 2.)
template <typename T, int VEC, typename IdxT>
__global__ __launch_bounds__(256) void bz_concat_ew_kernel(T* __restrict__ dst, CewP arg) {
  // the piece table is indexed with a run-time piece number: from LDS, not from a per-lane copy of the arguments
  __shared__ CewP p;
  static_assert(sizeof(CewP) % 4 == 0, "copied in 32-bit words");
  for (int w = threadIdx.x; w < (int)(sizeof(CewP) / 4); w += 256) ((uint32_t*)&p)[w] = ((const uint32_t*)&arg)[w];
  __syncthreads();
  using Pack = CewPack<T, VEC>;
  const int per_row = p.col0[p.n] / VEC;
  const int lane = threadIdx.x & 63;
  const IdxT rows = (IdxT)p.rows, r1 = (IdxT)p.r1;
  const IdxT nwaves = (IdxT)gridDim.x * 4;
  for (IdxT row = (IdxT)blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += nwaves) {
    const IdxT i0 = row / r1, i1 = row - i0 * r1;
    T* out_row = dst + (int64_t)row * p.dst_pitch;
    for (int cv = lane; cv < per_row; cv += 64) {
      const int col = cv * VEC;
      int k = 0;
#pragma unroll
      for (int q = 1; q < BZ_CEW_MAX; ++q) k += (q < p.n && col >= p.col0[q]);
      const int c = col - p.col0[k];
      const Pack x = *(const Pack*)((const T*)p.x[k] + (int64_t)i0 * p.xs[k][0] + (int64_t)i1 * p.xs[k][1] + c);
      const int op = p.op[k];
      Pack o = x;
      if (op != BZ_EW_ASSIGN) {
        const Pack y = *(const Pack*)((const T*)p.y[k] + (int64_t)i0 * p.ys[k][0] + (int64_t)i1 * p.ys[k][1] + c);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float a = ldv<T>(&x.e[e]), b = ldv<T>(&y.e[e]);
          stv<T>(&o.e[e], op == BZ_EW_ADD ? __fadd_rn(a, b) : op == BZ_EW_SUB ? __fsub_rn(a, b) : op == BZ_EW_MUL ? __fmul_rn(a, b) : __fdiv_rn(a, b));
        }
      }
      *(Pack*)(out_row + col) = o;
    }
  }
}

// The same when every piece has the same width W, W / VEC <= 64 and no piece divides (the attention input
// [q, k, q-k, q*k]): a lane owns VEC columns of a piece and walks the pieces, so it needs no search for its piece, and
// 64 / (W / VEC) rows share a wave so that no lane idles.  NP >= the number of pieces is a compile-time bound, and
// there is no branch in the row loop: a branch makes the compiler wait for every load in flight, and selecting among
// the results of all four operations per element cost some 700 instructions a row (20.9 us on [51200, 216] fp16).
// Instead every piece is one fused multiply-add whose operands are chosen per piece,
//   x + y = fma(x, 1, y)    x - y = fma(x, 1, -y)    x * y = fma(x, y, -0)
// each rounded once like the plain operation (-0 as the addend keeps the sign of a zero product), and a copy keeps the
// loaded bits.  A piece without a second operand reads its first one twice; an absent piece reads piece 0 again.
template <typename T, int VEC, int NP>
__global__ __launch_bounds__(256) void bz_concat_ew_uniform_kernel(T* __restrict__ dst, CewP p) {
  using Pack = CewPack<T, VEC>;
  const int per_piece = p.col0[1] / VEC;
  const int rows_per_wave = 64 / per_piece;
  const int lane = threadIdx.x & 63;
  const int sub = lane / per_piece, cv = lane - sub * per_piece;
  if (sub >= rows_per_wave) return;
  const uint32_t rows = (uint32_t)p.rows, r1 = (uint32_t)p.r1;
  const uint32_t step = gridDim.x * 4 * rows_per_wave;
  for (uint32_t row = (blockIdx.x * 4 + (threadIdx.x >> 6)) * rows_per_wave + sub; row < rows; row += step) {
    const uint32_t i0 = row / r1, i1 = row - i0 * r1;
    T* out = dst + (int64_t)row * p.dst_pitch + cv * VEC;
    Pack xs[NP], ys[NP];
#pragma unroll
    for (int k = 0; k < NP; ++k) {
      const int kk = k < p.n ? k : 0;
      const bool two = p.op[kk] != BZ_EW_ASSIGN;
      const T* yb = two ? (const T*)p.y[kk] : (const T*)p.x[kk];
      const int64_t ys0 = two ? p.ys[kk][0] : p.xs[kk][0], ys1 = two ? p.ys[kk][1] : p.xs[kk][1];
      xs[k] = *(const Pack*)((const T*)p.x[kk] + (int64_t)i0 * p.xs[kk][0] + (int64_t)i1 * p.xs[kk][1] + cv * VEC);
      ys[k] = *(const Pack*)(yb + (int64_t)i0 * ys0 + (int64_t)i1 * ys1 + cv * VEC);
    }
#pragma unroll
    for (int k = 0; k < NP; ++k) {
      const Pack o = bz::cew_piece<T, VEC>(p.op[k < p.n ? k : 0], xs[k], ys[k]);
      if (k < p.n) *(Pack*)(out + p.col0[k]) = o;
    }
  }
}

template <typename T, typename IdxT>
int launch_concat_ew_i(void* dst, const CewP& p, int vec, hipStream_t s) {
  if (p.col0[1] / vec <= 64 && sizeof(IdxT) == 4 && bz::cew_uniform(p)) {
    const int rows_per_wave = 64 / (p.col0[1] / vec);
    const int64_t blocks = (p.rows + 4 * rows_per_wave - 1) / (4 * rows_per_wave);
    const int grid = (int)(blocks < 256 * 32 ? blocks : 256 * 32);
#define BZ_CEW_U(V, NP) hipLaunchKernelGGL((bz_concat_ew_uniform_kernel<T, V, NP>), dim3(grid), dim3(256), 0, s, (T*)dst, p)
#define BZ_CEW_UV(V)       \
  do {                     \
    if (p.n <= 2)          \
      BZ_CEW_U(V, 2);      \
    else if (p.n <= 4)     \
      BZ_CEW_U(V, 4);      \
    else                   \
      BZ_CEW_U(V, BZ_CEW_MAX); \
  } while (0)
    switch (vec) {
      case 8: BZ_CEW_UV(8); break;
      case 4: BZ_CEW_UV(4); break;
      case 2: BZ_CEW_UV(2); break;
      default: BZ_CEW_UV(1); break;
    }
#undef BZ_CEW_UV
#undef BZ_CEW_U
    BZ_LAUNCH_OK("bz_concat_ew_uniform_kernel");
    return BZ_OK;
  }
  const int64_t blocks = (p.rows + 3) / 4;  // a wave per row, four waves per block
  const int grid = (int)(blocks < 256 * 32 ? blocks : 256 * 32);
  switch (vec) {
    case 8: hipLaunchKernelGGL((bz_concat_ew_kernel<T, 8, IdxT>), dim3(grid), dim3(256), 0, s, (T*)dst, p); break;
    case 4: hipLaunchKernelGGL((bz_concat_ew_kernel<T, 4, IdxT>), dim3(grid), dim3(256), 0, s, (T*)dst, p); break;
    case 2: hipLaunchKernelGGL((bz_concat_ew_kernel<T, 2, IdxT>), dim3(grid), dim3(256), 0, s, (T*)dst, p); break;
    default: hipLaunchKernelGGL((bz_concat_ew_kernel<T, 1, IdxT>), dim3(grid), dim3(256), 0, s, (T*)dst, p); break;
  }
  BZ_LAUNCH_OK("bz_concat_ew_kernel");
  return BZ_OK;
}

template <typename T>
int launch_concat_ew(void* dst, const CewP& p, int vec, hipStream_t s) {
  // (the grid-stride loop adds at most 2^15 to a row index below rows)
  if (p.rows < (1ll << 31) - (1ll << 16) && p.r1 < (1ll << 31)) return launch_concat_ew_i<T, uint32_t>(dst, p, vec, s);
  return launch_concat_ew_i<T, int64_t>(dst, p, vec, s);
}

template <typename T, typename CondT>
int launch_bcast(const bz_bcast_desc& d, const BcastP& p, int vec, hipStream_t s) {
  const int grid = grid_for(p.total / vec);
  const T* b = (const T*)d.b;
  const T* c = (const T*)d.c;
  T* out = (T*)d.out;
  switch (vec) {
    case 8:
      hipLaunchKernelGGL((bz_bcast_kernel<T, CondT, 8>), dim3(grid), dim3(256), 0, s, d.a, b, c, out, p);
      break;
    case 4:
      hipLaunchKernelGGL((bz_bcast_kernel<T, CondT, 4>), dim3(grid), dim3(256), 0, s, d.a, b, c, out, p);
      break;
    case 2:
      hipLaunchKernelGGL((bz_bcast_kernel<T, CondT, 2>), dim3(grid), dim3(256), 0, s, d.a, b, c, out, p);
      break;
    default:
      hipLaunchKernelGGL((bz_bcast_kernel<T, CondT, 1>), dim3(grid), dim3(256), 0, s, d.a, b, c, out, p);
      break;
  }
  BZ_LAUNCH_OK("bz_bcast_kernel");
  return BZ_OK;
}

template <typename T>
int launch_bcast_t(const bz_bcast_desc& d, const BcastP& p, int vec, hipStream_t s) {
  if (d.op == BZ_EW_WHERE && d.cond_dtype == BZ_I64) return launch_bcast<T, int64_t>(d, p, vec, s);
  return launch_bcast<T, int32_t>(d, p, vec, s);
}


// Gather along one axis: y[o, j, :] = data[o, idx[j], :] for `inner` contiguous units of W bytes (gather_op.cc:9-21, a
// memcpy per index there).  An index outside [0, axis_size) -- undefined behaviour in the reference, whose memcpy reads
// whatever lies there -- gives a row of zeros here.
template <typename Unit, typename Index>
__global__ __launch_bounds__(256) void bz_gather_kernel(const Unit* __restrict__ data, const Index* __restrict__ idx,
                                                        Unit* __restrict__ y, int64_t outer, int64_t axis_size, int64_t inner,
                                                        int64_t n_idx) {
  const int64_t total = outer * n_idx * inner;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / inner, e = i - row * inner;
    const int64_t o = row / n_idx, j = row - o * n_idx;
    const int64_t src = (int64_t)idx[j];
    Unit v = {};
    if (src >= 0 && src < axis_size) v = data[(o * axis_size + src) * inner + e];
    y[i] = v;
  }
}

}  // namespace

extern "C" int bz_broadcast_op(const bz_bcast_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_broadcast_op: null descriptor");
  const bz_bcast_desc& d = *desc;
  BZ_REQUIRE(d.rank >= 1 && d.rank <= BZ_MAX_RANK, "bz_broadcast_op: rank %d outside 1..%d", d.rank, BZ_MAX_RANK);
  BZ_REQUIRE(d.op >= BZ_EW_ADD && d.op <= BZ_EW_WHERE, "bz_broadcast_op: unknown op %d", d.op);
  BZ_REQUIRE(d.dtype == BZ_F32 || d.dtype == BZ_F16 || d.dtype == BZ_BF16, "bz_broadcast_op: unsupported dtype %d", d.dtype);
  BZ_REQUIRE(d.a != nullptr && d.out != nullptr, "bz_broadcast_op: null operand");
  BZ_REQUIRE(d.op == BZ_EW_ASSIGN || d.b != nullptr, "bz_broadcast_op: null second operand");
  if (d.op == BZ_EW_WHERE) {
    BZ_REQUIRE(d.c != nullptr, "bz_broadcast_op: Where needs three operands");
    BZ_REQUIRE(d.cond_dtype == BZ_I32 || d.cond_dtype == BZ_I64, "bz_broadcast_op: condition dtype %d", d.cond_dtype);
  }
  const bool use_b = d.op != BZ_EW_ASSIGN, use_c = d.op == BZ_EW_WHERE;
  int64_t total = 1;
  for (int i = 0; i < d.rank; ++i) {
    BZ_REQUIRE(d.dims[i] >= 0, "bz_broadcast_op: dim %d is %lld", i, (long long)d.dims[i]);
    BZ_REQUIRE(d.a_stride[i] >= 0 && d.b_stride[i] >= 0 && d.c_stride[i] >= 0, "bz_broadcast_op: negative stride");
    total *= d.dims[i];
  }
  if (total == 0) return BZ_OK;
  // merge adjacent dims: dims (outer, inner) fuse when every operand has stride_outer == stride_inner * dim_inner
  // (which covers "both broadcast": 0 == 0 * n); dims of size 1 are dropped
  BcastP p = {};
  int r = 0;
  for (int i = 0; i < d.rank; ++i) {
    if (d.dims[i] == 1) continue;
    const int64_t sa = d.a_stride[i], sb = use_b ? d.b_stride[i] : 0, sc = use_c ? d.c_stride[i] : 0;
    if (r > 0 && p.sa[r - 1] == sa * d.dims[i] && p.sb[r - 1] == sb * d.dims[i] && p.sc[r - 1] == sc * d.dims[i]) {
      p.dims[r - 1] *= d.dims[i];
      p.sa[r - 1] = sa;
      p.sb[r - 1] = sb;
      p.sc[r - 1] = sc;
    } else {
      p.dims[r] = d.dims[i];
      p.sa[r] = sa;
      p.sb[r] = sb;
      p.sc[r] = sc;
      ++r;
    }
  }
  if (r == 0) {  // a single element
    p.dims[0] = 1;
    r = 1;
  }
  p.rank = r;
  p.op = d.op;
  p.total = total;
  // a thread takes `vec` consecutive elements of the innermost dim: needs the dim to divide evenly
  int vec = 8;
  while (vec > 1 && p.dims[r - 1] % vec != 0) vec >>= 1;
  hipStream_t s = bz::as_stream(stream);
  if (d.dtype == BZ_F32) return launch_bcast_t<float>(d, p, vec > 4 ? 4 : vec, s);
  if (d.dtype == BZ_F16) return launch_bcast_t<__half>(d, p, vec, s);
  return launch_bcast_t<__hip_bfloat16>(d, p, vec, s);
}

extern "C" int bz_concat_ew(const bz_concat_ew_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_concat_ew: null descriptor");
  const bz_concat_ew_desc& d = *desc;
  CewP p;
  int vec = 1;
  const int rc = bz::cew_build(d, true, &p, &vec, "bz_concat_ew");
  if (rc != BZ_OK) return rc;
  if (p.rows == 0) return BZ_OK;
  hipStream_t s = bz::as_stream(stream);
  if (d.dtype == BZ_F32) return launch_concat_ew<float>(d.dst, p, vec, s);
  if (d.dtype == BZ_F16) return launch_concat_ew<__half>(d.dst, p, vec, s);
  return launch_concat_ew<__hip_bfloat16>(d.dst, p, vec, s);
}

extern "C" int bz_reduce_sum(const void* x, void* y, int64_t outer, int64_t dim, int64_t inner, int dtype, bz_stream_t stream) {
  BZ_REQUIRE(x != nullptr && y != nullptr, "bz_reduce_sum: null operand");
  BZ_REQUIRE(outer >= 0 && dim >= 0 && inner >= 0, "bz_reduce_sum: negative size");
  BZ_REQUIRE(dtype == BZ_F32 || dtype == BZ_F16 || dtype == BZ_BF16, "bz_reduce_sum: unsupported dtype %d", dtype);
  if (outer * inner == 0) return BZ_OK;
  hipStream_t s = bz::as_stream(stream);
  const int grid = grid_for(outer * inner);
  if (dtype == BZ_F32)
    hipLaunchKernelGGL(bz_reduce_sum_kernel<float>, dim3(grid), dim3(256), 0, s, (const float*)x, (float*)y, outer, dim, inner);
  else if (dtype == BZ_F16)
    hipLaunchKernelGGL(bz_reduce_sum_kernel<__half>, dim3(grid), dim3(256), 0, s, (const __half*)x, (__half*)y, outer, dim, inner);
  else
    hipLaunchKernelGGL(bz_reduce_sum_kernel<__hip_bfloat16>, dim3(grid), dim3(256), 0, s, (const __hip_bfloat16*)x,
                       (__hip_bfloat16*)y, outer, dim, inner);
  BZ_LAUNCH_OK("bz_reduce_sum_kernel");
  return BZ_OK;
}

extern "C" int bz_batch_norm(const bz_bn_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_batch_norm: null descriptor");
  const bz_bn_desc& d = *desc;
  BZ_REQUIRE(d.x && d.y && d.gamma && d.beta && d.mean && d.var, "bz_batch_norm: null operand");
  BZ_REQUIRE(d.size >= 0 && d.channels > 0, "bz_batch_norm: size=%lld channels=%lld", (long long)d.size, (long long)d.channels);
  BZ_REQUIRE(d.dtype == BZ_F32 || d.dtype == BZ_F16 || d.dtype == BZ_BF16, "bz_batch_norm: unsupported dtype %d", d.dtype);
  if (d.size == 0) return BZ_OK;
  hipStream_t s = bz::as_stream(stream);
  const int grid = grid_for(d.size);
  if (d.dtype == BZ_F32)
    hipLaunchKernelGGL(bz_batch_norm_kernel<float>, dim3(grid), dim3(256), 0, s, (const float*)d.x, (float*)d.y, d);
  else if (d.dtype == BZ_F16)
    hipLaunchKernelGGL(bz_batch_norm_kernel<__half>, dim3(grid), dim3(256), 0, s, (const __half*)d.x, (__half*)d.y, d);
  else
    hipLaunchKernelGGL(bz_batch_norm_kernel<__hip_bfloat16>, dim3(grid), dim3(256), 0, s, (const __hip_bfloat16*)d.x,
                       (__hip_bfloat16*)d.y, d);
  BZ_LAUNCH_OK("bz_batch_norm_kernel");
  return BZ_OK;
}

extern "C" int bz_softmax_axis(const void* x, void* y, int64_t outer, int64_t c, int64_t inner, int dtype, bz_stream_t stream) {
  BZ_REQUIRE(x != nullptr && y != nullptr, "bz_softmax_axis: null operand");
  BZ_REQUIRE(outer >= 0 && c > 0 && inner > 0, "bz_softmax_axis: outer=%lld c=%lld inner=%lld", (long long)outer, (long long)c,
             (long long)inner);
  BZ_REQUIRE(dtype == BZ_F32 || dtype == BZ_F16, "bz_softmax_axis: unsupported dtype %d", dtype);
  if (outer == 0) return BZ_OK;
  if (inner == 1) {  // rows of c contiguous values: one wave per row
    bz_act_desc a = {};
    a.x = x;
    a.y = y;
    a.rows = outer;
    a.cols = c;
    a.dtype = dtype;
    a.act = BZ_ACT_SOFTMAX;
    return bz_activation(&a, stream);
  }
  hipStream_t s = bz::as_stream(stream);
  const int grid = grid_for(outer * inner);
  if (dtype == BZ_F32)
    hipLaunchKernelGGL(bz_softmax_axis_kernel<float>, dim3(grid), dim3(256), 0, s, (const float*)x, (float*)y, outer, c, inner);
  else
    hipLaunchKernelGGL(bz_softmax_axis_kernel<__half>, dim3(grid), dim3(256), 0, s, (const __half*)x, (__half*)y, outer, c, inner);
  BZ_LAUNCH_OK("bz_softmax_axis_kernel");
  return BZ_OK;
}

extern "C" int bz_gather_rows(const void* data, const void* indices, int index_dtype, void* y, int64_t outer, int64_t axis_size,
                              int64_t inner_bytes, int64_t n_indices, bz_stream_t stream) {
  BZ_REQUIRE(outer >= 0 && axis_size >= 0 && inner_bytes > 0 && n_indices >= 0, "bz_gather_rows: outer=%lld axis_size=%lld inner_bytes=%lld n=%lld",
             (long long)outer, (long long)axis_size, (long long)inner_bytes, (long long)n_indices);
  BZ_REQUIRE(index_dtype == BZ_I32 || index_dtype == BZ_I64, "bz_gather_rows: indices->data_type()=%d", index_dtype);
  if (outer * n_indices == 0) return BZ_OK;
  BZ_REQUIRE(data != nullptr && indices != nullptr && y != nullptr, "bz_gather_rows: null operand");
  hipStream_t s = bz::as_stream(stream);
  // the widest unit that both tensors' rows are made of and aligned to
  const uintptr_t bits = (uintptr_t)data | (uintptr_t)y | (uintptr_t)inner_bytes;
#define BZ_GATHER(Unit)                                                                                                      \
  do {                                                                                                                       \
    const int64_t inner = inner_bytes / (int64_t)sizeof(Unit);                                                               \
    const int grid = grid_for(outer * n_indices * inner);                                                                    \
    if (index_dtype == BZ_I32)                                                                                               \
      hipLaunchKernelGGL((bz_gather_kernel<Unit, int32_t>), dim3(grid), dim3(256), 0, s, (const Unit*)data, (const int32_t*)indices, \
                         (Unit*)y, outer, axis_size, inner, n_indices);                                                      \
    else                                                                                                                     \
      hipLaunchKernelGGL((bz_gather_kernel<Unit, int64_t>), dim3(grid), dim3(256), 0, s, (const Unit*)data, (const int64_t*)indices, \
                         (Unit*)y, outer, axis_size, inner, n_indices);                                                      \
  } while (0)
  if (bits % 16 == 0)
    BZ_GATHER(uint4);
  else if (bits % 4 == 0)
    BZ_GATHER(uint32_t);
  else if (bits % 2 == 0)
    BZ_GATHER(uint16_t);
  else
    BZ_GATHER(uint8_t);
#undef BZ_GATHER
  BZ_LAUNCH_OK("bz_gather_kernel");
  return BZ_OK;
}
