// mlp_fused.hip -- a whole FC stack (Gemm + bias + activation, layer after layer) in ONE kernel for gfx950.
//
// Stands in for the chain  Gemm -> PRelu|Dice|... -> Gemm -> ... -> Gemm -> Softmax|Sigmoid  that the
// reference runs as one library GEMM plus one activation kernel per layer (blaze/operator/op/gemm_op.h:33-107,
// prelu_op.cc:11-30, dice_op.cc:15-34, softmax_op.cc:21-78; executed op by op by blaze/graph/simple_net.cc:35-46).
// The result equals the layer-by-layer composition evaluated in fp32 from the same rounded inputs, with every
// hidden activation rounded to the tensor dtype exactly where the op-by-op path stores it.
//
// Why one kernel: at CTR sizes (batch 2048, widths 896-512-256-2) each layer alone is a few microseconds of
// latency-bound work and the intermediates make a round trip through HBM/L2.  Here a workgroup owns 64 rows of the
// batch for the whole stack; hidden activations never leave the CU (they live in LDS, 160 KB per CU on this part),
// and the only global traffic is the input slab once and the weights, streamed from L2.
//
// Work split: 256 threads = 4 waves; each wave owns a quarter of the layer's output columns for all 64 rows, so
// the accumulators of a 64 x 512 layer are 128 registers per lane.  Operand A comes from LDS (layer 0: input tiles
// staged global -> registers -> LDS, double buffered; later layers: the previous layer's activations in place).
// Operand W never touches LDS: waves do not share columns, so each wave loads its MFMA fragments straight from
// global memory.  bz_mlp_pack_weight lays the weight out in that order ("fragment major": one wave-wide 16-byte
// load = 1 KB contiguous), which makes every weight load fully coalesced.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <type_traits>

#include "bz_common.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 64;              // rows per workgroup (32 when that is what it takes to put 64 workgroups on the chip)
constexpr int kBK = 64;              // K per step
constexpr int kThreads = 256;
constexpr int kAPitch = kBK * 2 + 16;  // staged input tile: 64 rows x 128 bytes, padded against bank conflicts
constexpr float kDiceEps = 1e-8f;    // blaze/operator/common_helper.h:90
// K steps of a packed weight: a whole number of the longest trip of the K loop (4 steps), zero filled beyond K
__host__ __device__ constexpr int ktp_of(int k) { return (k + 4 * kBK - 1) / (4 * kBK) * 4; }

struct LayerP {
  const char* w;  // wide layer: fragment-major pack; skinny layer: [n, ldw] K contiguous
  const float* bias;
  const float* p0;
  const float* p1;
  const float* p2;
  int n, k;
  int ldw;  // skinny layer only
  int act, act_size, nosqrt;
  float alpha, beta, act_alpha;
};

struct MlpP {
  const char* x;
  char* y;
  int64_t ldx, ldy;  // elements
  int m;
  int n_layers;
  int out_dtype;
  int skinny_last;
  int warm_l2;   // touch the weights ahead of use (see the kernel)
  int h_off[2];  // byte offsets of the two activation buffers in LDS
  int head_off;  // byte offset of the head layer's weights in LDS ([n][k], staged once per workgroup)
  LayerP l[BZ_MLP_MAX_LAYERS];
};

template <int DT>
__device__ __forceinline__ void mma(const uint4& a, const uint4& b, floatx16& acc) {
  if constexpr (DT == BZ_F16)
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(*(const half8*)&a, *(const half8*)&b, acc, 0, 0, 0);
  else
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8*)&a, *(const bf16x8*)&b, acc, 0, 0, 0);
}

template <int DT>
__device__ __forceinline__ uint16_t to_bits(float v) {
  if constexpr (DT == BZ_F16) {
    return __half_as_ushort(__float2half_rn(v));
  } else {
    const uint32_t u = __float_as_uint(v);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
  }
}

template <int DT>
__device__ __forceinline__ float from_bits(uint16_t b) {
  if constexpr (DT == BZ_F16)
    return __half2float(__ushort_as_half(b));
  else
    return __uint_as_float((uint32_t)b << 16);
}

// The activation is a template parameter wherever it is applied to many elements: a run-time switch per element
// turns an unrolled epilogue into hundreds of taken branches over code larger than the instruction cache.
template <int ACT>
__device__ __forceinline__ float act_apply_t(float v, bool nosqrt, float act_alpha, float p0, float p1, float p2) {
  if constexpr (ACT == BZ_ACT_PRELU) {
    // math/activation.h:37-42 is x * ((x > 0) + (x < 0) * w): x for x > 0, x * w below, 0 (and NaN) kept
    return v > 0.f ? v : v * p0;
  } else if constexpr (ACT == BZ_ACT_DICE) {
    const float den = nosqrt ? p2 : sqrtf(p2 + kDiceEps);
    const float t = expf(-1.f * (v - p1) / den);
    const float p = 1.f / (1.f + t);
    return (1.f - p) * p0 * v + p * v;
  } else if constexpr (ACT == BZ_ACT_LEAKY_RELU) {
    return v >= 0.f ? v : act_alpha * v;
  } else if constexpr (ACT == BZ_ACT_SIGMOID) {
    const float t = expf(v);
    return t / (1.f + t);
  } else {
    return v;
  }
}

__device__ __forceinline__ float act_apply(float v, const LayerP& L, float p0, float p1, float p2) {
  switch (L.act) {
    case BZ_ACT_PRELU:
      return act_apply_t<BZ_ACT_PRELU>(v, false, 0.f, p0, p1, p2);
    case BZ_ACT_DICE:
      return act_apply_t<BZ_ACT_DICE>(v, L.nosqrt != 0, 0.f, p0, p1, p2);
    case BZ_ACT_LEAKY_RELU:
      return act_apply_t<BZ_ACT_LEAKY_RELU>(v, false, L.act_alpha, p0, p1, p2);
    case BZ_ACT_SIGMOID:
      return act_apply_t<BZ_ACT_SIGMOID>(v, false, 0.f, p0, p1, p2);
    default:
      return v;
  }
}

// f(integral_constant<int, P>) for P = B .. E-1, unrolled at compile time (register sets are indexed by P)
template <int B, int E, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>());
    static_for<B + 1, E>(f);
  }
}

// One wide layer for this workgroup's rows.  NB = 32-column blocks per wave (N = 128 * NB).
// STREAM_A: operand A is staged from global memory tile by tile (layer 0); otherwise it is read in place from
// the activation buffer `hin` (pitch hin_pitch bytes).  Output goes to `hout` (pitch N*2 + 16) in the tensor dtype.
template <int DT, int BM, int NB, bool STREAM_A>
__device__ __forceinline__ void wide_layer(const MlpP& P, const LayerP& L, int m0, char* lds, const char* hin, int hin_pitch,
                                           char* hout) {
  constexpr int TMS = BM / 32;                // 32-row blocks per wave
  constexpr int A_PER = BM * 8 / kThreads;    // 16-byte chunks of one input tile per thread
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int K = L.k;
  // DW register sets of weights: the loads of step s + DW - 1 are issued during step s.  With 32 rows per workgroup
  // the accumulators leave room for four sets, i.e. three steps (about 1.5 us of MFMA work) of latency cover: the
  // weights arrive from the last-level cache, not from L2, whenever a pooling kernel ran since their last use.
  constexpr int DW = (BM == 32 && NB <= 2) ? 4 : 2;  // (four sets of a 4-block layer would not fit the register file)
  constexpr int DA = DW;  // register sets of input tiles (STREAM_A)
  const int KT = (K + kBK - 1) / kBK;
  const int KTP = ktp_of(K);                 // steps in the pack (zero filled beyond K)
  const int KTR = (KT + DW - 1) / DW * DW;   // steps run: a whole number of trips, <= KTP
  const int frag_row = lane & 31, frag_half = lane >> 5;

  floatx16 acc[TMS][NB];
#pragma unroll
  for (int i = 0; i < TMS; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // per-column epilogue parameters, requested first so that their latency hides under the K loop
  float cbias[NB], cp0[NB], cp1[NB], cp2[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int n = wave * (NB * 32) + j * 32 + frag_row;
    cbias[j] = L.bias ? L.bias[n] : 0.f;
    cp0[j] = cp1[j] = cp2[j] = 0.f;
    if (L.act == BZ_ACT_PRELU) cp0[j] = L.p0[L.act_size == 1 ? 0 : n];
    if (L.act == BZ_ACT_DICE) {
      cp0[j] = L.p0[n];
      cp1[j] = L.p1[n];
      cp2[j] = L.p2[n];
    }
  }

  // weight fragments of step s: NB*4 wave-wide 16-byte loads, each 1 KB contiguous
  const char* wbase = L.w + ((int64_t)wave * KTP * NB * 4) * 1024 + lane * 16;
  uint4 rw[DW][NB][4];
  auto gload_w = [&](int set, int s) {
    const char* p = wbase + (int64_t)s * (NB * 4 * 1024);
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) rw[set][j][kk] = *(const uint4*)(p + (j * 4 + kk) * 1024);
  };

  // input tile of step s (STREAM_A): BM rows x 64 k = BM * 8 16-byte chunks, A_PER per thread
  uint4 ra[DA][A_PER];
  auto gload_a = [&](int set, int s) {
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
      const int q = tid + i * kThreads;
      const int r = q >> 3, ch = q & 7;
      int m = m0 + r;
      m = m < P.m ? m : P.m - 1;
      int k = s * kBK + ch * 8;
      k = k < K ? k : 0;  // clamped address; the value is masked when it is stored
      ra[set][i] = *(const uint4*)(P.x + ((int64_t)m * P.ldx + k) * 2);
    }
  };
  auto lstore_a = [&](int set, int buf, int s) {
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
      const int q = tid + i * kThreads;
      const int r = q >> 3, ch = q & 7;
      const uint32_t keep = (s * kBK + ch * 8) < K ? 0xffffffffu : 0u;
      uint4 v = ra[set][i];
      v.x &= keep;
      v.y &= keep;
      v.z &= keep;
      v.w &= keep;
      *(uint4*)(lds + buf * (BM * kAPitch) + r * kAPitch + ch * 16) = v;
    }
  };

  // One K step: the MFMAs of step s out of rw[set], with the weight loads of step `s_next` into rw[set_next] dealt
  // among them, one load per TMS MFMAs.  A wave issues in order, and a wave-wide 16-byte load occupies the CU's
  // address unit for about as long as the matrix unit needs for two MFMAs; a burst of loads in front of the MFMAs
  // would keep the matrix unit idle until the whole burst has been accepted.
  auto compute = [&](auto set_c, auto next_c, const char* a_base, int a_pitch, int s_next) {
    constexpr int set = decltype(set_c)::value, set_next = decltype(next_c)::value;
    // a_base points at this lane's fragment of k-substep 0 in M tile 0
    uint4 fa[TMS][4];
#pragma unroll
    for (int i = 0; i < TMS; ++i)
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) fa[i][kk] = *(const uint4*)(a_base + i * 32 * a_pitch + kk * 32);
    const char* pn = wbase + (int64_t)s_next * (NB * 4 * 1024);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        rw[set_next][j][kk] = *(const uint4*)(pn + (j * 4 + kk) * 1024);
#pragma unroll
        for (int i = 0; i < TMS; ++i) mma<DT>(fa[i][kk], rw[set][j][kk], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);  // pin this order: the scheduler would otherwise regroup loads and MFMAs
      }
    }
  };
  // DW steps per trip, no conditionals inside: loads are issued in the order they are consumed, so the compiler's
  // wait counts are exact.  Before step s: rw[s % DW .. (s + DW - 2) % DW] hold the weights of steps s .. s + DW - 2.
#pragma unroll
  for (int d = 0; d < DW - 1; ++d) gload_w(d, d < KTR ? d : KTR - 1);

  if constexpr (STREAM_A) {
    // Before step s: tile s is in LDS buffer s & 1, registers ra[(s + 1) % DA ..] hold tiles s + 1 .. s + DA - 1.
#pragma unroll
    for (int d = 0; d < DA; ++d) gload_a(d, d);
    lstore_a(0, 0, 0);
    __syncthreads();
    for (int s0 = 0; s0 < KTR; s0 += DW) {
      static_for<0, DW>([&](auto p_c) {
        constexpr int p = decltype(p_c)::value;
        const int s = s0 + p;
        gload_a(p % DA, s + DA);  // set p held tile s, which already sits in LDS
        __builtin_amdgcn_sched_barrier(0);
        compute(std::integral_constant<int, p % DW>(), std::integral_constant<int, (p + DW - 1) % DW>(),
                lds + (p & 1) * (BM * kAPitch) + frag_row * kAPitch + frag_half * 16, kAPitch,
                s + DW - 1 < KTR ? s + DW - 1 : KTR - 1);
        lstore_a((p + 1) % DA, (p + 1) & 1, s + 1);
        __syncthreads();
      });
    }
  } else {
    for (int s0 = 0; s0 < KTR; s0 += DW) {
      static_for<0, DW>([&](auto p_c) {
        constexpr int p = decltype(p_c)::value;
        const int s = s0 + p;
        // steps beyond K multiply zero weights: they read step 0's (this row's own, finite) activations again rather
        // than whatever lies behind the row in LDS
        const int sa = s < KT ? s : 0;
        compute(std::integral_constant<int, p % DW>(), std::integral_constant<int, (p + DW - 1) % DW>(),
                hin + frag_row * hin_pitch + (sa * kBK) * 2 + frag_half * 16, hin_pitch, s + DW - 1 < KTR ? s + DW - 1 : KTR - 1);
      });
    }
  }

  // epilogue: lane owns column n and rows 8*(r/4) + 4*(lane/32) + r%4 of each 32x32 block
  const int out_pitch = L.n * 2 + 16;
  const float alpha = L.alpha, beta = L.bias ? L.beta : 0.f, act_alpha = L.act_alpha;
  const bool nosqrt = L.nosqrt != 0;
  auto epilogue = [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int n = wave * (NB * 32) + j * 32 + frag_row;
      const float bj = beta * cbias[j];
#pragma unroll
      for (int i = 0; i < TMS; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = i * 32 + 8 * (r >> 2) + 4 * frag_half + (r & 3);
          const float v = act_apply_t<ACT>(alpha * acc[i][j][r] + bj, nosqrt, act_alpha, cp0[j], cp1[j], cp2[j]);
          *(uint16_t*)(hout + row * out_pitch + n * 2) = to_bits<DT>(v);
        }
      }
    }
  };
  switch (L.act) {
    case BZ_ACT_PRELU:
      epilogue(std::integral_constant<int, BZ_ACT_PRELU>());
      break;
    case BZ_ACT_DICE:
      epilogue(std::integral_constant<int, BZ_ACT_DICE>());
      break;
    case BZ_ACT_LEAKY_RELU:
      epilogue(std::integral_constant<int, BZ_ACT_LEAKY_RELU>());
      break;
    case BZ_ACT_SIGMOID:
      epilogue(std::integral_constant<int, BZ_ACT_SIGMOID>());
      break;
    default:
      epilogue(std::integral_constant<int, BZ_ACT_NONE>());
      break;
  }
}

template <int DT, int BM, bool STREAM_A>
__device__ __forceinline__ void wide_layer_any(const MlpP& P, const LayerP& L, int m0, char* lds, const char* hin, int hin_pitch,
                                               char* hout) {
  switch (L.n / 128) {
    case 1:
      wide_layer<DT, BM, 1, STREAM_A>(P, L, m0, lds, hin, hin_pitch, hout);
      break;
    case 2:
      wide_layer<DT, BM, 2, STREAM_A>(P, L, m0, lds, hin, hin_pitch, hout);
      break;
    case 3:
      wide_layer<DT, BM, 3, STREAM_A>(P, L, m0, lds, hin, hin_pitch, hout);
      break;
    default:
      wide_layer<DT, BM, 4, STREAM_A>(P, L, m0, lds, hin, hin_pitch, hout);
      break;
  }
}

// The head: N <= 8 outputs per row from the activations in LDS.  kThreads / BM lanes share a row (an equal part of K
// each) and reduce by shuffles; the logits go through a small LDS scratch, then one lane per row applies the activation /
// softmax.  Loops over the outputs are kept rolled: this code runs once per launch, and unrolled it would cost more
// in instruction fetch than it saves in issue slots.
template <int DT, int BM>
__device__ __forceinline__ void skinny_layer(const MlpP& P, const LayerP& L, int m0, const char* hin, int hin_pitch,
                                             const char* wl, const float* hp, float* logits) {
  constexpr int LPR = kThreads / BM;  // lanes per row: 4 or 8
  const int tid = threadIdx.x;
  const int row = tid / LPR, part = tid % LPR;
  const int K = L.k;  // a multiple of 128
  const int N = L.n;
  const int act = L.act;
  const float alpha = L.alpha, beta = L.bias ? L.beta : 0.f;
  const int kq = K / LPR;
  const char* ap = hin + row * hin_pitch + part * kq * 2;
  const char* wp = wl + part * kq * 2;
#pragma unroll 1
  for (int j = 0; j < N; ++j) {
    float dot = 0.f;
    for (int c = 0; c < kq; c += 8) {
      const uint4 av = *(const uint4*)(ap + c * 2);
      const uint4 wv = *(const uint4*)(wp + (j * K + c) * 2);
      const uint32_t ar[4] = {av.x, av.y, av.z, av.w};
      const uint32_t wr[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        dot += from_bits<DT>((uint16_t)(ar[e] & 0xffffu)) * from_bits<DT>((uint16_t)(wr[e] & 0xffffu));
        dot += from_bits<DT>((uint16_t)(ar[e] >> 16)) * from_bits<DT>((uint16_t)(wr[e] >> 16));
      }
    }
#pragma unroll
    for (int d = 1; d < LPR; d <<= 1) dot += __shfl_xor(dot, d, 64);
    // hp: [bias | p0 | p1 | p2] x 8, staged in LDS at kernel start (zero where a parameter does not apply)
    if (part == 0) logits[row * BZ_MLP_MAX_HEAD + j] = alpha * dot + beta * hp[j];
  }
  __syncthreads();
  if (tid >= BM) return;
  float* lr = logits + tid * BZ_MLP_MAX_HEAD;
  const int m = m0 + tid;
  float mx = -INFINITY;
#pragma unroll 1
  for (int j = 0; j < N; ++j) {
    float t = lr[j];
    if (act != BZ_ACT_SOFTMAX && act != BZ_ACT_NONE) t = act_apply(t, L, hp[8 + j], hp[16 + j], hp[24 + j]);
    lr[j] = t;
    mx = fmaxf(mx, t);
  }
  float sum = 1.f;
  if (act == BZ_ACT_SOFTMAX) {  // softmax_op.cc:21-78: subtract the max, exp, divide by the sum
    sum = 0.f;
#pragma unroll 1
    for (int j = 0; j < N; ++j) {
      const float e = expf(lr[j] - mx);
      lr[j] = e;
      sum += e;
    }
  }
  if (m >= P.m) return;
  const bool f32 = P.out_dtype == BZ_F32;
#pragma unroll 1
  for (int j = 0; j < N; ++j) {
    const float v = act == BZ_ACT_SOFTMAX ? lr[j] / sum : lr[j];
    if (f32)
      ((float*)P.y)[(int64_t)m * P.ldy + j] = v;
    else
      ((uint16_t*)P.y)[(int64_t)m * P.ldy + j] = to_bits<DT>(v);
  }
}

template <int DT, int BM>
__global__ __launch_bounds__(kThreads, 1) void bz_mlp_kernel(MlpP P) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int m0 = blockIdx.x * BM;
  const int n_wide = P.n_layers - P.skinny_last;
  const char* hin = nullptr;
  int hin_pitch = 0;
  // Warm-up of the L2: every workgroup streams ALL the weights, so the workgroups that share an XCD (the hardware
  // deals workgroup ids round robin over the 8 XCDs) would each miss on the same lines one K step after the other when
  // the weights are not in that XCD's L2 -- which is the normal case after a pooling kernel.  Instead each of them
  // first touches its own eighth of every layer's pack, one dword per 128-byte line, so that between them the whole
  // pack is on its way before the K loop starts.  The values are folded into `warm`, which is consumed (by a store
  // that never happens) after the first layer.
  uint32_t warm = 0;
  if (P.warm_l2) {
    const int slice = (blockIdx.x / 8) & 7;
    for (int li = 0; li < n_wide; ++li) {
      const int64_t bytes = (int64_t)ktp_of(P.l[li].k) * kBK * P.l[li].n * 2;
      const int64_t lo = bytes * slice / 8 / 128 * 128, hi = bytes * (slice + 1) / 8;
      // eight loads in flight per thread and trip (one trip covers 256 KB of a slice: every layer up to 512 x 2048)
#pragma unroll 1
      for (int64_t base = lo + (int64_t)threadIdx.x * 128; base < hi; base += (int64_t)8 * kThreads * 128) {
        uint32_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int64_t off = base + (int64_t)u * kThreads * 128;
          v[u] = off < hi ? *(const uint32_t*)(P.l[li].w + off) : 0u;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) warm ^= v[u];
      }
    }
  }
  // the head's weights (at most 8 x 512 elements) are requested now and parked in LDS after the first layer, so
  // that the head finds them on chip instead of paying a round trip to L2 per chunk
  uint4 hw[2] = {};
  const LayerP& H = P.l[P.n_layers - 1];
  const int head_chunks = P.skinny_last ? H.n * H.k / 8 : 0;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = threadIdx.x + i * kThreads;
    if (q < head_chunks) {
      const int cpr = H.k / 8;
      const int j = q / cpr, ch = q - j * cpr;
      hw[i] = *(const uint4*)(H.w + ((int64_t)j * H.ldw + ch * 8) * 2);
    }
  }
  // ... and its per-output parameters: thread 8*a + j fetches element j of array a (bias, p0, p1, p2)
  float hp = 0.f;
  if (P.skinny_last && threadIdx.x < 32) {
    const int a = threadIdx.x >> 3, j = threadIdx.x & 7;
    const float* src = a == 0 ? H.bias : (a == 1 ? H.p0 : (a == 2 ? H.p1 : H.p2));
    const bool used = a == 0 || (a == 1 && (H.act == BZ_ACT_PRELU || H.act == BZ_ACT_DICE)) || (a >= 2 && H.act == BZ_ACT_DICE);
    if (src != nullptr && used && j < H.n) hp = src[(a == 1 && H.act == BZ_ACT_PRELU && H.act_size == 1) ? 0 : j];
  }
  for (int li = 0; li < n_wide; ++li) {
    char* hout = lds + P.h_off[li & 1];
    if (li == 0) {
      wide_layer_any<DT, BM, true>(P, P.l[0], m0, lds, nullptr, 0, hout);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int q = threadIdx.x + i * kThreads;
        if (q < head_chunks) *(uint4*)(lds + P.head_off + q * 16) = hw[i];
      }
      if (P.skinny_last && threadIdx.x < 32) *(float*)(lds + P.head_off + head_chunks * 16 + threadIdx.x * 4) = hp;
      if (warm == 0x9e3779b9u && P.m < 0) *(uint32_t*)P.y = warm;  // (m is never negative)
    } else {
      wide_layer_any<DT, BM, false>(P, P.l[li], m0, lds, hin, hin_pitch, hout);
    }
    __syncthreads();
    hin = hout;
    hin_pitch = P.l[li].n * 2 + 16;
  }
  if (P.skinny_last) {
    skinny_layer<DT, BM>(P, P.l[P.n_layers - 1], m0, hin, hin_pitch, lds + P.head_off,
                     (const float*)(lds + P.head_off + head_chunks * 16), (float*)lds);
  } else {
    // the last wide layer's tile: LDS -> global, 16 bytes per lane along rows
    const int n = P.l[n_wide - 1].n;
    const int cpr = n / 8;
    for (int q = threadIdx.x; q < BM * cpr; q += kThreads) {
      const int r = q / cpr, ch = q - r * cpr;
      const int m = m0 + r;
      if (m < P.m) *(uint4*)(P.y + ((int64_t)m * P.ldy + ch * 8) * 2) = *(const uint4*)(hin + r * hin_pitch + ch * 16);
    }
  }
}

// [N, ldw] K-contiguous -> fragment major: element (((wave*KTP + s)*NB + j)*4 + kk)*512 + lane*8 + e holds
// W[n = wave*NB*32 + j*32 + lane%32][k = s*64 + kk*16 + (lane/32)*8 + e], zero beyond K (KTP = ktp_of(K) steps).
__global__ __launch_bounds__(256) void bz_mlp_pack_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int K, int N,
                                                          int64_t ldw, int KT2) {
  const int NB = N / 128;
  const int64_t groups = (int64_t)4 * KT2 * NB * 4 * 64;  // 8-element groups
  for (int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x; g < groups; g += (int64_t)gridDim.x * 256) {
    const int lane = (int)(g & 63);
    int64_t t = g >> 6;
    const int kk = (int)(t & 3);
    t >>= 2;
    const int j = (int)(t % NB);
    t /= NB;
    const int s = (int)(t % KT2);
    const int wave = (int)(t / KT2);
    const int n = wave * NB * 32 + j * 32 + (lane & 31);
    const int k0 = s * 64 + kk * 16 + (lane >> 5) * 8;
    uint16_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (k0 + e) < K ? src[(int64_t)n * ldw + k0 + e] : (uint16_t)0;
    uint4 o;
    o.x = v[0] | ((uint32_t)v[1] << 16);
    o.y = v[2] | ((uint32_t)v[3] << 16);
    o.z = v[4] | ((uint32_t)v[5] << 16);
    o.w = v[6] | ((uint32_t)v[7] << 16);
    *(uint4*)(dst + g * 8) = o;
  }
}

}  // namespace

extern "C" int64_t bz_mlp_packed_elems(int k, int n) {
  if (k <= 0 || n <= 0 || n % 128 != 0) return 0;
  return (int64_t)ktp_of(k) * kBK * n;
}

extern "C" int bz_mlp_pack_weight(const void* w_nk, int dtype, int k, int n, int64_t ldw, void* dst, bz_stream_t stream) {
  BZ_REQUIRE(w_nk != nullptr && dst != nullptr, "bz_mlp_pack_weight: null pointer");
  BZ_REQUIRE(dtype == BZ_F16 || dtype == BZ_BF16, "bz_mlp_pack_weight: dtype %d (fp16 and bf16 only)", dtype);
  BZ_REQUIRE(k > 0 && n > 0 && n % 128 == 0 && n <= BZ_MLP_MAX_WIDTH, "bz_mlp_pack_weight: k=%d n=%d (n: multiple of 128, <= %d)", k, n,
             BZ_MLP_MAX_WIDTH);
  BZ_REQUIRE(ldw >= k, "bz_mlp_pack_weight: ldw=%lld < k=%d", (long long)ldw, k);
  BZ_REQUIRE((uintptr_t)dst % 16 == 0, "bz_mlp_pack_weight: dst must be 16-byte aligned");
  const int KT2 = ktp_of(k);
  const int64_t groups = (int64_t)KT2 * kBK * n / 8;
  const int grid = (int)((groups + 255) / 256 < 4096 ? (groups + 255) / 256 : 4096);
  hipLaunchKernelGGL(bz_mlp_pack_kernel, dim3(grid), dim3(256), 0, bz::as_stream(stream), (const uint16_t*)w_nk, (uint16_t*)dst, k, n,
                     ldw, KT2);
  BZ_LAUNCH_OK("bz_mlp_pack_kernel");
  return BZ_OK;
}

extern "C" int bz_mlp_fused(const bz_mlp_desc* desc, bz_stream_t stream) {
  BZ_REQUIRE(desc != nullptr, "bz_mlp_fused: null descriptor");
  const bz_mlp_desc& d = *desc;
  BZ_REQUIRE(d.dtype == BZ_F16 || d.dtype == BZ_BF16, "bz_mlp_fused: dtype %d (fp16 and bf16 only)", d.dtype);
  BZ_REQUIRE(d.n_layers >= 1 && d.n_layers <= BZ_MLP_MAX_LAYERS, "bz_mlp_fused: %d layers (1..%d)", d.n_layers, BZ_MLP_MAX_LAYERS);
  BZ_REQUIRE(d.x != nullptr && d.y != nullptr && d.m >= 0, "bz_mlp_fused: null x/y or negative m");
  BZ_REQUIRE((uintptr_t)d.x % 16 == 0 && d.ldx % 8 == 0, "bz_mlp_fused: x must be 16-byte aligned with ldx %% 8 == 0");
  const bz_mlp_layer& last = d.layer[d.n_layers - 1];
  const int skinny_last = last.n <= BZ_MLP_MAX_HEAD ? 1 : 0;
  BZ_REQUIRE(d.n_layers - skinny_last >= 1, "bz_mlp_fused: needs at least one wide layer");
  MlpP P = {};
  // 64 rows per workgroup amortise the weight stream over twice the MFMA work; below 64 such workgroups the chip is
  // better used by twice as many of 32 rows (a batch of 2048: 64 workgroups instead of 32)
  const int bm = (d.m + kBM - 1) / kBM >= 64 ? kBM : 32;
  int k_in = d.layer[0].k;
  BZ_REQUIRE(k_in > 0 && k_in % 8 == 0 && d.ldx >= k_in, "bz_mlp_fused: input width %d (multiple of 8, <= ldx)", k_in);
  int h_size[2] = {0, 0};
  for (int i = 0; i < d.n_layers; ++i) {
    const bz_mlp_layer& s = d.layer[i];
    const bool skinny = skinny_last && i == d.n_layers - 1;
    BZ_REQUIRE(s.w != nullptr && s.k == k_in, "bz_mlp_fused: layer %d: null weight or k=%d does not follow %d", i, s.k, k_in);
    BZ_REQUIRE((uintptr_t)s.w % 16 == 0, "bz_mlp_fused: layer %d: weight must be 16-byte aligned", i);
    if (skinny) {
      BZ_REQUIRE(s.n >= 1 && s.ldw >= s.k && s.ldw % 8 == 0, "bz_mlp_fused: head: n=%d ldw=%d", s.n, s.ldw);
      BZ_REQUIRE(s.act == BZ_ACT_NONE || s.act == BZ_ACT_SOFTMAX || s.act == BZ_ACT_SIGMOID || s.act == BZ_ACT_LEAKY_RELU ||
                     s.act == BZ_ACT_PRELU || s.act == BZ_ACT_DICE,
                 "bz_mlp_fused: head: unknown activation %d", s.act);
    } else {
      BZ_REQUIRE(s.n % 128 == 0 && s.n >= 128 && s.n <= BZ_MLP_MAX_WIDTH, "bz_mlp_fused: layer %d: n=%d (multiple of 128, <= %d)", i,
                 s.n, BZ_MLP_MAX_WIDTH);
      BZ_REQUIRE(s.act != BZ_ACT_SOFTMAX, "bz_mlp_fused: layer %d: softmax only on a head of at most %d outputs", i, BZ_MLP_MAX_HEAD);
      const int bytes = bm * (s.n * 2 + 16);
      h_size[i & 1] = bytes > h_size[i & 1] ? bytes : h_size[i & 1];
    }
    if (s.act == BZ_ACT_PRELU) BZ_REQUIRE(s.p0 != nullptr && (s.act_size == 1 || s.act_size == s.n), "bz_mlp_fused: layer %d: PReLU slope", i);
    if (s.act == BZ_ACT_DICE) BZ_REQUIRE(s.p0 && s.p1 && s.p2, "bz_mlp_fused: layer %d: Dice parameters", i);
    LayerP& L = P.l[i];
    L.w = (const char*)s.w;
    L.bias = s.bias;
    L.p0 = s.p0;
    L.p1 = s.p1;
    L.p2 = s.p2;
    L.n = s.n;
    L.k = s.k;
    L.ldw = s.ldw;
    L.act = s.act;
    L.act_size = s.act_size;
    L.nosqrt = s.dice_nosqrt;
    L.alpha = s.alpha;
    L.beta = s.beta;
    L.act_alpha = s.act_alpha;
    k_in = s.n;
  }
  BZ_REQUIRE(d.out_dtype == d.dtype || (skinny_last && d.out_dtype == BZ_F32), "bz_mlp_fused: out dtype %d", d.out_dtype);
  BZ_REQUIRE(d.ldy >= last.n, "bz_mlp_fused: ldy=%lld < n=%d", (long long)d.ldy, last.n);
  if (!skinny_last) BZ_REQUIRE((uintptr_t)d.y % 16 == 0 && d.ldy % 8 == 0, "bz_mlp_fused: y must be 16-byte aligned with ldy %% 8 == 0");
  if (d.m == 0) return BZ_OK;
  P.x = (const char*)d.x;
  P.y = (char*)d.y;
  P.ldx = d.ldx;
  P.ldy = d.ldy;
  P.m = d.m;
  P.n_layers = d.n_layers;
  P.out_dtype = d.out_dtype;
  P.skinny_last = skinny_last;
  // with fewer workgroups than two per XCD there is nobody to share the warm-up with
  P.warm_l2 = (d.m + bm - 1) / bm >= 16 ? 1 : 0;
  const int a_bytes = 2 * bm * kAPitch;
  P.h_off[0] = a_bytes;
  P.h_off[1] = a_bytes + h_size[0];
  P.head_off = a_bytes + h_size[0] + h_size[1];
  const int lds_bytes = P.head_off + (skinny_last ? last.n * last.k * 2 + 128 : 0);
  BZ_REQUIRE(lds_bytes <= 160 * 1024, "bz_mlp_fused: the stack needs %d bytes of LDS (limit 163840)", lds_bytes);
  hipStream_t st = bz::as_stream(stream);
  const int grid = (d.m + bm - 1) / bm;
  // (the opt-in to more than 64 KB of dynamic LDS is per kernel function and per device)
#define BZ_MLP_LAUNCH(DT, BM)                                                                                              \
  do {                                                                                                                     \
    static thread_local int set = 0;                                                                                       \
    if (set < lds_bytes) {                                                                                                 \
      BZ_HIP_OK(hipFuncSetAttribute((const void*)bz_mlp_kernel<DT, BM>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); \
      set = 160 * 1024;                                                                                                    \
    }                                                                                                                      \
    hipLaunchKernelGGL((bz_mlp_kernel<DT, BM>), dim3(grid), dim3(kThreads), lds_bytes, st, P);                             \
  } while (0)
  if (d.dtype == BZ_F16) {
    if (bm == kBM)
      BZ_MLP_LAUNCH(BZ_F16, kBM);
    else
      BZ_MLP_LAUNCH(BZ_F16, 32);
  } else {
    if (bm == kBM)
      BZ_MLP_LAUNCH(BZ_BF16, kBM);
    else
      BZ_MLP_LAUNCH(BZ_BF16, 32);
  }
#undef BZ_MLP_LAUNCH
  BZ_LAUNCH_OK("bz_mlp_kernel");
  return BZ_OK;
}
