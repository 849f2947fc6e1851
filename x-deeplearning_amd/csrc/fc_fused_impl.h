// fc_fused_impl.h -- FC layer = GEMM + bias + activation in one kernel, for gfx950 MFMA.
//
// Stands in for the reference's pair  Gemm op (blaze/operator/op/gemm_op.h:33-107:
// Y <- broadcast(bias); Y = alpha*A*B + beta*Y via cblas/cuBLAS, blaze/math/gemm.cc:13-27,
// gemm.cu:35-104)  +  the separate PRelu / Dice / LeakyRelu / Sigmoid / Softmax op that
// follows it (prelu_op.cc:11-30, dice_op.cc:15-34, leaky_relu_op.cc:15-21,
// sigmoid_op.cc:15-21, softmax_op.cc:21-78).  The result equals the composition
// Activation(Gemm(x, W, b)) evaluated in fp32.
//
// Main kernel: C tile BM x BN per workgroup, K stepped by BK through double-buffered LDS
// (global -> registers -> LDS, one barrier per step) with the global loads of the next D
// tiles in flight in D register sets while the current tile is multiplied.  Operands are both "K contiguous" (A row major, W packed [N,K]) so
// a lane's MFMA fragment is one 16-byte LDS read; rows are padded by 16 bytes, which
// spreads the 16 lanes of a ds_read_b128 phase over all 64 banks.  fp16/bf16 use
// v_mfma_f32_32x32x16 (K=16 per instruction, fp32 accumulate); fp32 uses
// v_mfma_f32_32x32x2 with a K permutation inside each 8-wide step so its fragments are
// 16-byte reads as well.  In the accumulator a lane owns one output column and 16
// rows, so per-column epilogue parameters (bias, PReLU slope, Dice gamma/mean/var) are
// lane constants.
//
// Skinny kernel (N <= 8: the 256->2 softmax head, the 40->1 attention score, the 256->1
// sigmoid head): bandwidth bound on A; a lane group of pow2(K/8) lanes owns a row, the
// weight fragments live in registers, the N dot products are reduced by shuffles.
//
// Compiled once per operand type (fc_fused_f16.hip, fc_fused_bf16.hip, fc_fused_f32.hip include this file and define
// that type's entry, bz::fc_run_*): three translation units that build side by side instead of one that takes three
// times as long.  bz_fc_fused itself (argument checks, the choice of path) is in fc_fused.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <mutex>
#include <type_traits>

#include "bz_common.h"
#include "fc_common.h"

namespace {

using namespace bz::fc;

// one 16-byte chunk of a K-contiguous operand row; zero beyond K; element-wise when unaligned
template <int DT>
__device__ __forceinline__ uint4 load_chunk(const char* base, int64_t row, int64_t ld, int k, int K, bool vec_ok) {
  constexpr int ES = In<DT>::kSize;
  constexpr int CH = In<DT>::kChunk;
  uint4 out = make_uint4(0, 0, 0, 0);
  if (k >= K) return out;
  const char* p = base + (row * ld + k) * ES;
  if (vec_ok && k + CH <= K) return *(const uint4*)p;
  if constexpr (ES == 2) {
    if (((uintptr_t)p & 3) == 0) {
      // rows that start on 4 bytes (an even row length, e.g. a Concat of 3 x 54 columns): pairs of elements
      uint32_t d[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        d[i] = 0u;
        if (k + 2 * i + 1 < K)
          d[i] = *(const uint32_t*)(p + 4 * i);
        else if (k + 2 * i < K)
          d[i] = *(const unsigned short*)(p + 4 * i);
      }
      return make_uint4(d[0], d[1], d[2], d[3]);
    }
    unsigned short e[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) e[i] = (k + i < K) ? *(const unsigned short*)(p + 2 * i) : (unsigned short)0;
    out.x = e[0] | ((uint32_t)e[1] << 16);
    out.y = e[2] | ((uint32_t)e[3] << 16);
    out.z = e[4] | ((uint32_t)e[5] << 16);
    out.w = e[6] | ((uint32_t)e[7] << 16);
  } else {
    uint32_t e[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = (k + i < K) ? *(const uint32_t*)(p + 4 * i) : 0u;
    out = make_uint4(e[0], e[1], e[2], e[3]);
  }
  return out;
}

// The same for operands whose rows are 16-byte aligned and K a multiple of the chunk (a chunk is either wholly inside
// K or absent): no branches and nothing done to the loaded value, so the loads of several K tiles can stay in
// flight.  A chunk beyond K is read from 16 bytes of zeros instead of being masked after the load: a mask is an
// instruction on the loaded register, and the scheduler is free to place it - and the wait for the load it implies -
// right behind the load (it did so in the 128x256 tile: one exposed trip to memory in every K tile).
__device__ uint4 kZeroChunk = {0u, 0u, 0u, 0u};  // never written; not const, so that it lives in the global address space like the operands (a select between a global and a constant-space pointer would be loaded through FLAT)

template <int DT>
__device__ __forceinline__ uint4 load_chunk_aligned(const char* base, int64_t row, int64_t ld, int k, int K) {
  constexpr int ES = In<DT>::kSize;
  const char* p = k < K ? base + (row * ld + k) * ES : (const char*)&kZeroChunk;
  return *(const uint4*)p;
}

// The variant that reads a clamped address and leaves the zeroing of chunks beyond K to the consumer.  The eight-wave
// tile with the skinny head keeps it: there the address select costs more (11.1 against 10.5 us on config 2's
// 512 -> 256 -> 2) than the mask, which the scheduler leaves at the LDS store in that kernel.
template <int DT>
__device__ __forceinline__ uint4 load_chunk_clamped(const char* base, int64_t row, int64_t ld, int k, int K) {
  constexpr int ES = In<DT>::kSize;
  constexpr int CH = In<DT>::kChunk;
  const int kc = k < K ? k : K - CH;
  return *(const uint4*)(base + (row * ld + kc) * ES);
}


template <int DT>
__device__ __forceinline__ void chunk_to_float(const uint4& c, float (&f)[In<DT>::kChunk]) {
  const uint32_t r[4] = {c.x, c.y, c.z, c.w};
  if constexpr (DT == BZ_F32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(r[i]);
  } else if constexpr (DT == BZ_F16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __half2float(__ushort_as_half((unsigned short)(r[i] & 0xffffu)));
      f[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(r[i] >> 16)));
    }
  } else {  // bf16: the upper 16 bits of the fp32 pattern
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(r[i] << 16);
      f[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
}

// the optional skinny second layer computed from the first layer's output tile while it is still in LDS
struct HeadArgs {
  const char* w;      // [n, ldw], K contiguous, the dtype of the first layer's operands
  const float* bias;  // [n] or null
  void* y;            // [M, ldy]
  int64_t ldw, ldy;
  int n, act, out_dtype;
};

// ---------------------------------------------------------------------------------------------
// tiled MFMA kernel
// ---------------------------------------------------------------------------------------------
template <int DT, typename OutT, int BM, int BN, int BK, int WM, int WN, int D, bool ALIGNED, bool HEAD>
__global__ __launch_bounds__(WM* WN * 64) void bz_fc_mfma_kernel(const char* __restrict__ A, const char* __restrict__ W,
                                                                  OutT* __restrict__ Y, int M, int N, int K, int64_t lda,
                                                                  int64_t ldw, int64_t ldy, bool vec_a, bool vec_w,
                                                                  bool vec_y, int tiles_m, Epilogue ep, HeadArgs head) {
  using T = In<DT>;
  constexpr int NT = WM * WN * 64;
  constexpr int ES = T::kSize;
  constexpr int ROWB = BK * ES;        // bytes of one tile row
  constexpr int PITCH = ROWB + 16;     // padded LDS pitch
  constexpr int CPR = ROWB / 16;       // 16-byte chunks per row
  constexpr int A_CHUNKS = BM * CPR, W_CHUNKS = BN * CPR;
  constexpr int A_PER = (A_CHUNKS + NT - 1) / NT, W_PER = (W_CHUNKS + NT - 1) / NT;
  constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
  constexpr int TM = WTM / 32, TN = WTN / 32;  // 32x32 blocks per wave
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % T::kStepK == 0, "tile shape");

  __shared__ __attribute__((aligned(16))) char lds[2][(BM + BN) * PITCH];
  // HEAD: the second layer's weight [kSkinnyMaxN, BN], requested now into registers, parked in LDS after the K loop
  constexpr int HW_ROW = BN * ES;  // bytes
  constexpr int HW_CHUNKS = HEAD ? kSkinnyMaxN * HW_ROW / 16 : 1;
  constexpr int HW_PER = (HW_CHUNKS + NT - 1) / NT;
  __shared__ __attribute__((aligned(16))) char lds_hw[HEAD ? kSkinnyMaxN * HW_ROW : 16];
  uint4 rhw[HW_PER];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  // consecutive workgroups walk down M within one N panel: the W panel stays hot in L2
  const int tile_m = blockIdx.x % tiles_m, tile_n = blockIdx.x / tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // D register sets: K tiles kt+1 .. kt+D are in flight from global memory while tile kt is multiplied out of
  // LDS.  The kernel is latency bound at CTR sizes (a tile's MFMAs take ~0.1 us, a round trip ~1 us), so the
  // number of exposed round trips, ceil(KT / D), is what sets its duration.
  // which aligned loader: the head tile (see load_chunk_clamped) and the 256x256 tile, whose 256 registers have no room
  // for the zero-chunk select's addresses (it spilled 75 of them)
  constexpr bool CLAMPED = HEAD || BM * BN >= 256 * 256;
  uint4 ra[D][A_PER], rw[D][W_PER];
  auto gload = [&](int set, int k0) {
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
      const int q = tid + i * NT;
      if (A_CHUNKS % NT == 0 || q < A_CHUNKS) {
        const int r = q / CPR, ch = q % CPR;
        int m = m0 + r;
        m = m < M ? m : M - 1;
        ra[set][i] = !ALIGNED ? load_chunk<DT>(A, m, lda, k0 + ch * T::kChunk, K, vec_a)
                     : CLAMPED ? load_chunk_clamped<DT>(A, m, lda, k0 + ch * T::kChunk, K)
                            : load_chunk_aligned<DT>(A, m, lda, k0 + ch * T::kChunk, K);
      }
    }
#pragma unroll
    for (int i = 0; i < W_PER; ++i) {
      const int q = tid + i * NT;
      if (W_CHUNKS % NT == 0 || q < W_CHUNKS) {
        const int r = q / CPR, ch = q % CPR;
        int n = n0 + r;
        n = n < N ? n : N - 1;
        rw[set][i] = !ALIGNED ? load_chunk<DT>(W, n, ldw, k0 + ch * T::kChunk, K, vec_w)
                     : CLAMPED ? load_chunk_clamped<DT>(W, n, ldw, k0 + ch * T::kChunk, K)
                            : load_chunk_aligned<DT>(W, n, ldw, k0 + ch * T::kChunk, K);
      }
    }
  };
  // registers -> LDS (chunks beyond K already arrived as zeros, except from the clamped loader)
  auto masked = [&](uint4 v, int k) {
    if (ALIGNED && CLAMPED) {
      const uint32_t keep = k < K ? 0xffffffffu : 0u;
      v.x &= keep;
      v.y &= keep;
      v.z &= keep;
      v.w &= keep;
    }
    return v;
  };
  auto lstore = [&](int set, int buf, int k0) {
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
      const int q = tid + i * NT;
      if (A_CHUNKS % NT == 0 || q < A_CHUNKS)
        *(uint4*)&lds[buf][(q / CPR) * PITCH + (q % CPR) * 16] = masked(ra[set][i], k0 + (q % CPR) * T::kChunk);
    }
#pragma unroll
    for (int i = 0; i < W_PER; ++i) {
      const int q = tid + i * NT;
      if (W_CHUNKS % NT == 0 || q < W_CHUNKS)
        *(uint4*)&lds[buf][(BM + q / CPR) * PITCH + (q % CPR) * 16] = masked(rw[set][i], k0 + (q % CPR) * T::kChunk);
    }
  };

  if constexpr (HEAD) {
    const int present = N * ES / 16;  // chunks of a weight row that exist (N is a whole number of chunks)
#pragma unroll
    for (int i = 0; i < HW_PER; ++i) {
      const int q = tid + i * NT;
      const int j = q / (HW_ROW / 16), ch = q % (HW_ROW / 16);
      rhw[i] = make_uint4(0, 0, 0, 0);
      if (q < HW_CHUNKS && j < head.n && ch < present) rhw[i] = *(const uint4*)(head.w + (int64_t)j * head.ldw * ES + ch * 16);
    }
  }

  // with a single 32x32 block per wave, back-to-back MFMAs into one accumulator would each wait for the
  // previous result; alternate K steps between two accumulators and add them at the end
  constexpr int KACC = (TM * TN == 1 && BK / T::kStepK >= 2) ? 2 : 1;
  floatx16 acc[KACC][TM][TN];
#pragma unroll
  for (int a = 0; a < KACC; ++a)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][i][j][r] = 0.f;

  // per-column epilogue parameters, requested before anything else so their latency hides under the K loop; nothing
  // is computed from them before the epilogue (an instruction on a loaded value here is a wait for memory here)
  float cbias[TN], cp0[TN], cp1[TN], cp2[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    int n = n0 + wn * WTN + j * 32 + (lane & 31);
    n = n < N ? n : N - 1;
    cbias[j] = ep.bias_rows == 1 ? ep.bias[n] : 0.f;
    cp0[j] = cp1[j] = cp2[j] = 0.f;
    if (ep.act == BZ_ACT_PRELU) cp0[j] = ep.p0[ep.act_size == 1 ? 0 : n];
    if (ep.act == BZ_ACT_DICE) {
      cp0[j] = ep.p0[n];
      cp1[j] = ep.p1[n];
      cp2[j] = ep.p2[n];
    }
  }

  // The K loop runs over KT rounded up to a multiple of D with no conditionals inside: tiles beyond K are
  // loaded from a clamped address and zeroed by the mask, so they add nothing.  Straight-line code lets the
  // compiler count outstanding loads exactly (s_waitcnt vmcnt(n) waits for the oldest set only).
  const int KT = (K + BK - 1) / BK;
  const int KTR = (KT + D - 1) / D * D;
#pragma unroll
  for (int d = 0; d < D; ++d) gload(d, d * BK);
  lstore(0, 0, 0);
  __syncthreads();
  const int frag_row = lane & 31, frag_half = lane >> 5;
  // Tiles are bound by how well LDS traffic hides behind the MFMAs, and a barrier lines all waves up in the same
  // phase: a burst of fragment reads right after it (matrix pipes idle), a burst of tile stores right before it.  PIPE
  // reorders a K tile: the next tile goes to the other LDS buffer first (its registers arrived long ago), fragments
  // are read one sub-step ahead of the MFMAs that use them, and the barrier sits before the last sub-step's MFMAs,
  // which then cover the read of the next tile's first fragments.
  // (not the 256x256 tile: with 128 accumulator registers a wave has no room for a second set of fragments; measured on
  // the other tiles: 128x256 245 -> 238 us on 8192x12800x1024, 64x64 9.6 -> 9.2 us on config 2's first layer)
  constexpr bool PIPE = !HEAD && BM * BN >= 64 * 64 && BM * BN < 256 * 256;
  constexpr int KS = BK / T::kStepK;
  if constexpr (PIPE) {
    static_assert(KS % 2 == 0, "fragment double buffer needs an even number of sub-steps");
    uint4 fa[2][TM], fw[2][TN];
    auto fread = [&](int slot, int buf, int ks) {
      const char* la = &lds[buf][(wm * WTM + frag_row) * PITCH + frag_half * 16];
      const char* lw = &lds[buf][(BM + wn * WTN + frag_row) * PITCH + frag_half * 16];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[slot][i] = *(const uint4*)(la + i * 32 * PITCH + ks * 32);
#pragma unroll
      for (int j = 0; j < TN; ++j) fw[slot][j] = *(const uint4*)(lw + j * 32 * PITCH + ks * 32);
    };
    auto fmma = [&](int slot, int ks) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) T::mma(fa[slot][i], fw[slot][j], acc[ks % KACC][i][j]);
    };
    fread(0, 0, 0);
    for (int kt0 = 0; kt0 < KTR; kt0 += D) {
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const int kt = kt0 + d;
        const int buf = kt & 1;
        gload(d, (kt + D) * BK);  // set d held tile kt, which already sits in LDS
        // the other buffer was last read before the previous barrier: tile kt+1 can go there now
        lstore((d + 1) % D, buf ^ 1, (kt + 1) * BK);
#pragma unroll
        for (int ks = 0; ks + 1 < KS; ++ks) {
          fread((ks + 1) & 1, buf, ks + 1);
          fmma(ks & 1, ks);
        }
        __syncthreads();           // tile kt+1 is complete; every read of this buffer has returned
        fread(0, buf ^ 1, 0);      // KS is even: the next tile's first fragments take slot 0 again
        fmma((KS - 1) & 1, KS - 1);
      }
    }
    __syncthreads();  // the fragments read ahead for a tile that does not exist are dropped; LDS is free for the epilogue
  } else {
  for (int kt0 = 0; kt0 < KTR; kt0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int kt = kt0 + d;
      const int buf = kt & 1;
      gload(d, (kt + D) * BK);  // set d held tile kt, which already sits in LDS
      const char* la = &lds[buf][(wm * WTM + frag_row) * PITCH + frag_half * 16];
      const char* lw = &lds[buf][(BM + wn * WTN + frag_row) * PITCH + frag_half * 16];
#pragma unroll
      for (int ks = 0; ks < BK / T::kStepK; ++ks) {
        uint4 fa[TM], fw[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = *(const uint4*)(la + i * 32 * PITCH + ks * 32);
#pragma unroll
        for (int j = 0; j < TN; ++j) fw[j] = *(const uint4*)(lw + j * 32 * PITCH + ks * 32);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) T::mma(fa[i], fw[j], acc[ks % KACC][i][j]);
      }
      lstore((d + 1) % D, buf ^ 1, (kt + 1) * BK);
      __syncthreads();
    }
  }
  }

  if (KACC == 2) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][i][j][r] += acc[KACC - 1][i][j][r];
  }
  // epilogue: lane owns column n, rows 8*(r/4) + 4*(lane/32) + r%4 of each 32x32 block.  The activated tile
  // goes through LDS (free after the K loop) so that global stores are 16 bytes per lane along rows.
  constexpr int OS = (int)sizeof(OutT);
  constexpr int OPITCH = BN * OS + 16;
  static_assert(BM * OPITCH <= (int)sizeof(lds), "output tile must fit the operand buffers");
  char* lout = &lds[0][0];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    cbias[j] *= ep.beta;
    if (ep.act == BZ_ACT_DICE) cp2[j] = dice_inv_den(ep, cp2[j]);
  }
  // A bias of one row per sample, the rare form, is folded into the accumulators first, so that the element loop below
  // has no index to compute and nothing to decide per element.
  // (The 256x256 tile has no registers to spare for it and is not chosen for such a layer.)
  float alpha_e = ep.alpha;
  if (BM * BN < 256 * 256 && ep.bias_rows > 1) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * WTN + j * 32 + (lane & 31);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * WTM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          const float b = (m < M && n < N) ? ep.beta * ep.bias[full_bias_index(ep, m, n, M, N)] : 0.f;
          acc[0][i][j][r] = fmaf(ep.alpha, acc[0][i][j][r], b);
        }
      }
    }
    alpha_e = 1.f;
  }
  // The activation is a compile-time parameter of the element loop: a run-time switch per element would turn the
  // unrolled epilogue into a string of taken branches over far more code than the loop needs.  Every output goes
  // into the LDS tile, rows and columns beyond the matrix included (they are not copied out): a bounds check and a
  // 64-bit address per element cost several times the activation.
  auto epilogue = [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int nl = wn * WTN + j * 32 + (lane & 31);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int ml = wm * WTM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          float v = fmaf(alpha_e, acc[0][i][j][r], cbias[j]);  // (cbias: beta * bias of the column, or 0)
          v = apply_act_t<ACT>(v, ep, cp0[j], cp1[j], cp2[j]);
          store_out<OutT>((OutT*)(lout + ml * OPITCH) + nl, v);
        }
      }
    }
  };
  switch (ep.act) {
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
  if constexpr (HEAD) {
#pragma unroll
    for (int i = 0; i < HW_PER; ++i) {
      const int q = tid + i * NT;
      if (q < HW_CHUNKS) *(uint4*)&lds_hw[q * 16] = rhw[i];
    }
  }
  __syncthreads();
  if (vec_y) {
    constexpr int OCPR = BN * OS / 16;  // 16-byte chunks per tile row
    for (int q = tid; q < BM * OCPR; q += NT) {
      const int ml = q / OCPR, ch = q % OCPR;
      const int m = m0 + ml, n = n0 + ch * (16 / OS);
      if (m < M && n < N) *(uint4*)((char*)(Y + out_index(ep, m, n, ldy))) = *(const uint4*)(lout + ml * OPITCH + ch * 16);
    }
  } else if (Y != nullptr) {  // an output that takes no 16-byte stores: element by element, along rows
    for (int q = tid; q < BM * BN; q += NT) {
      const int ml = q / BN, nl = q % BN;
      if (m0 + ml < M && n0 + nl < N) Y[out_index(ep, m0 + ml, n0 + nl, ldy)] = ((const OutT*)(lout + ml * OPITCH))[nl];
    }
  }
  if constexpr (HEAD) {
    // z[m, j] = head_act(sum_n y[m, n] * w2[j, n] + b2[j]) from the rounded tile, as the separate skinny launch
    // computes it from the stored tensor.  NT / BM lanes share a row; this workgroup owns whole rows (n0 == 0).
    static_assert(OS == ES, "the head reads the tile with the operand type");
    constexpr int LPRH = NT / BM;
    constexpr int CH = In<DT>::kChunk;
    const int r = tid / LPRH, hl = tid % LPRH;
    const int m = m0 + r;
    const int nch = N / CH;
    float hacc[kSkinnyMaxN];
#pragma unroll
    for (int j = 0; j < kSkinnyMaxN; ++j) hacc[j] = 0.f;
    for (int ch = hl; ch < nch; ch += LPRH) {
      float a[CH];
      chunk_to_float<DT>(*(const uint4*)(lout + r * OPITCH + ch * 16), a);
#pragma unroll
      for (int j = 0; j < kSkinnyMaxN; ++j) {
        if (j < head.n) {
          float w[CH];
          chunk_to_float<DT>(*(const uint4*)(lds_hw + j * HW_ROW + ch * 16), w);
#pragma unroll
          for (int i = 0; i < CH; ++i) hacc[j] = fmaf(a[i], w[i], hacc[j]);
        }
      }
    }
#pragma unroll
    for (int d = LPRH >> 1; d > 0; d >>= 1) {
#pragma unroll
      for (int j = 0; j < kSkinnyMaxN; ++j) hacc[j] += __shfl_xor(hacc[j], d, 64);
    }
    if (hl == 0 && m < M) {
      float v[kSkinnyMaxN];
#pragma unroll
      for (int j = 0; j < kSkinnyMaxN; ++j) v[j] = (j < head.n) ? hacc[j] + (head.bias ? head.bias[j] : 0.f) : 0.f;
      if (head.act == BZ_ACT_SOFTMAX) {  // softmax_op.cc:21-78: subtract max, exp, sum in order, divide
        float mx = v[0];
#pragma unroll
        for (int j = 1; j < kSkinnyMaxN; ++j)
          if (j < head.n) mx = v[j] > mx ? v[j] : mx;
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < kSkinnyMaxN; ++j)
          if (j < head.n) {
            v[j] = expf(v[j] - mx);
            sum += v[j];
          }
#pragma unroll
        for (int j = 0; j < kSkinnyMaxN; ++j)
          if (j < head.n) v[j] = v[j] / sum;
      } else if (head.act == BZ_ACT_SIGMOID) {
#pragma unroll
        for (int j = 0; j < kSkinnyMaxN; ++j) {
          const float t = expf(v[j]);
          v[j] = t / (1.f + t);
        }
      }
#pragma unroll
      for (int j = 0; j < kSkinnyMaxN; ++j) {
        if (j < head.n) {
          const int64_t at = (int64_t)m * head.ldy + j;
          if (head.out_dtype == BZ_F32)
            store_out<float>((float*)head.y + at, v[j]);
          else if (head.out_dtype == BZ_F16)
            store_out<__half>((__half*)head.y + at, v[j]);
          else
            store_out<__hip_bfloat16>((__hip_bfloat16*)head.y + at, v[j]);
        }
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------
// streaming kernel: large layers (a 256x128 tile per CU fills the chip, K deep)
// ---------------------------------------------------------------------------------------------
// At this size the limit is how fast operands reach a CU, not latency: a 256x128x64 step is 1024 MFMA cycles per SIMD
// and 48 KB of operands, which the path from L2 into a CU (64 bytes a clock) needs 768 cycles for.  So the tile is the
// largest one that still gives every CU a workgroup with one wave per SIMD multiplying (128x64 per wave, 128 accumulator
// registers), and nothing else may stand in the loads' way:
//  - operands go from global memory straight into LDS (global_load_lds_dwordx4: no registers, no LDS store
//    instructions), three stages of 48 KB, two tiles in flight;
//  - four more waves, one per SIMD, do nothing but issue those loads and wait for them; the multiplying waves issue
//    only LDS reads and MFMAs and meet the loaders at one barrier per K tile (the same wave doing both measured 237 us
//    on 8192 x 12800 -> 1024 bf16, this split 203 us);
//  - a tile row is 128 bytes, half of the 64 banks; chunk c of row r is stored at position c ^ ((r >> 1) & 7), so the
//    16 lanes of a ds_read_b128 phase (16 rows, one logical chunk) hit 16 different bank groups (203 -> 195 us: with
//    the 32-bank pattern c ^ (r & 7) every other cycle of the LDS was a conflict);
//  - the scheduler is told to alternate MFMA and fragment read, and not to move either across a phase (195 -> 192 us).
constexpr int kStreamBM = 256, kStreamBN = 128, kStreamBK = 64, kStreamStages = 3;
constexpr int kStreamRowB = kStreamBK * 2;
constexpr int kStreamStageBytes = (kStreamBM + kStreamBN) * kStreamRowB;  // 49152
constexpr int kStreamLds = kStreamStages * kStreamStageBytes;            // 147456 of the CU's 160 KB
constexpr int kStreamCompute = 256;                                       // threads that multiply; as many again load

typedef __attribute__((address_space(3))) char lds_char;

// 16 bytes per lane from global memory to LDS at lds_addr + 16 * lane (lds_addr is the same in all lanes)
__device__ __forceinline__ void load_to_lds(const char* g, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_addr) : "memory", "m0");
}

// one phase = 6 fragment reads for the phase after next and 8 MFMAs on fragments read a phase ago
#define BZ_PIN_PHASE()                                     \
  do {                                                     \
    _Pragma("unroll") for (int q_ = 0; q_ < 6; ++q_) {     \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   \
    }                                                      \
    __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);     \
    __builtin_amdgcn_sched_barrier(0);                     \
  } while (0)

template <int DT, typename OutT>
__global__ __launch_bounds__(2 * kStreamCompute, 1) void bz_fc_stream_kernel(const char* __restrict__ A,
                                                                              const char* __restrict__ W, OutT* __restrict__ Y,
                                                                              int M, int N, int K, int64_t lda, int64_t ldw,
                                                                              int64_t ldy, int tiles_m, int tiles_n, Epilogue ep) {
  using T = In<DT>;
  static_assert(T::kSize == 2 && sizeof(OutT) == 2, "2-byte operands and outputs");
  constexpr int BM = kStreamBM, BN = kStreamBN, ROWB = kStreamRowB, STAGES = kStreamStages, NT = kStreamCompute;
  constexpr int STAGE_BYTES = kStreamStageBytes;
  constexpr int LOADS = (BM + BN) * (ROWB / 16) / NT;  // 12 chunks per loader thread per stage
  constexpr int TM = 4, TN = 2;                        // 32x32 blocks per wave tile (128 x 64)
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const bool loader = threadIdx.x >= NT;
  const int tid = threadIdx.x & (NT - 1), lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // The 8 XCDs take turns at consecutive workgroup ids.  XCD x walks its own band of M tiles, the N tiles of an M tile
  // next to each other in time: an A tile is fetched into that XCD's L2 once, the W panel streams through it.
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int per_xcd = (tiles_m + 7) / 8;
  const int tile_m = xcd * per_xcd + j / tiles_n, tile_n = j % tiles_n;
  if (tile_m >= tiles_m) return;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_char*)smem;
  const int KT = K / kStreamBK;

  if (loader) {
    // chunk p = i*256 + tid of a stage: row p >> 3 (A rows, then W rows), position p & 7
    const char* src[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int p = i * NT + tid;
      const int r = p >> 3, c = (p & 7) ^ ((r >> 1) & 7);
      if (r < BM) {
        int m = m0 + r;
        m = m < M ? m : M - 1;
        src[i] = A + ((int64_t)m * lda) * 2 + c * 16;
      } else {
        int n = n0 + (r - BM);
        n = n < N ? n : N - 1;
        src[i] = W + ((int64_t)n * ldw) * 2 + c * 16;
      }
    }
    auto issue = [&](int kt) {
      const uint32_t base = __builtin_amdgcn_readfirstlane(lds0 + (kt % STAGES) * STAGE_BYTES + wave * 1024);
      const int64_t koff = (int64_t)kt * ROWB;
#pragma unroll
      for (int i = 0; i < LOADS; ++i) load_to_lds(src[i] + koff, base + i * (NT * 16));
    };
    // Barrier kt (counted from 0) says: tile kt has landed, and nobody reads the stage tile kt+2 goes to any more.
    // The waits are written out because only this code knows how many loads may stay in flight.
    issue(0);
    if (KT > 1) issue(1);
    if (KT > 1)
      asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    for (int kt = 0; kt < KT; ++kt) {
      if (kt + 2 < KT) {
        issue(kt + 2);
        asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
      }
    }
    __syncthreads();  // the two barriers of the epilogue
    __syncthreads();
    return;
  }

  // per-column epilogue parameters, requested before the K loop
  float cbias[TN], cp0[TN], cp1[TN], cp2[TN];
#pragma unroll
  for (int jn = 0; jn < TN; ++jn) {
    int n = n0 + wn * 64 + jn * 32 + (lane & 31);
    n = n < N ? n : N - 1;
    cbias[jn] = ep.bias_rows == 1 ? ep.bias[n] : 0.f;
    cp0[jn] = cp1[jn] = cp2[jn] = 0.f;
    if (ep.act == BZ_ACT_PRELU) cp0[jn] = ep.p0[ep.act_size == 1 ? 0 : n];
    if (ep.act == BZ_ACT_DICE) {
      cp0[jn] = ep.p0[n];
      cp1[jn] = ep.p1[n];
      cp2[jn] = ep.p2[n];  // (finished in the epilogue: an instruction on a loaded value here is a wait for memory here)
    }
  }

  floatx16 acc[TM][TN];
#pragma unroll
  for (int a = 0; a < TM; ++a)
#pragma unroll
    for (int b = 0; b < TN; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // lane (row = lane & 31, half = lane >> 5) reads logical chunk 2*ks + half of its row
  const int frow = lane & 31, fhalf = lane >> 5;
  int foff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) foff[ks] = frow * ROWB + (((2 * ks + fhalf) ^ ((frow >> 1) & 7)) << 4);
  const int a_base = (wm * 128) * ROWB, w_base = (BM + wn * 64) * ROWB;
  uint4 fa[2][TM], fw[2][TN];
  auto fread = [&](int slot, int stage, int ks) {
    const char* s = smem + stage * STAGE_BYTES + foff[ks];
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[slot][i] = *(const uint4*)(s + a_base + i * 32 * ROWB);
#pragma unroll
    for (int jn = 0; jn < TN; ++jn) fw[slot][jn] = *(const uint4*)(s + w_base + jn * 32 * ROWB);
  };
  auto fmma = [&](int slot) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int jn = 0; jn < TN; ++jn) T::mma(fa[slot][i], fw[slot][jn], acc[i][jn]);
  };

  asm volatile("s_barrier" ::: "memory");  // tile 0 landed
  fread(0, 0, 0);
  for (int kt = 0; kt < KT; ++kt) {
    const int stage = kt % STAGES;
    fread(1, stage, 1);
    fmma(0);
    BZ_PIN_PHASE();
    fread(0, stage, 2);
    fmma(1);
    BZ_PIN_PHASE();
    fread(1, stage, 3);
    fmma(0);
    BZ_PIN_PHASE();
    // every read of this stage has returned (the last were issued 8 MFMAs ago); past the barrier tile kt+1 is complete
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (kt + 1 < KT) fread(0, (kt + 1) % STAGES, 0);
    fmma(1);
    BZ_PIN_PHASE();
  }

  // epilogue: lane owns column n of each 32x32 block, rows 8*(r/4) + 4*(lane/32) + r%4; the activated tile goes through
  // LDS so that global stores are 16 bytes per lane along rows
  __syncthreads();
#pragma unroll
  for (int jn = 0; jn < TN; ++jn) {
    cbias[jn] *= ep.beta;
    if (ep.act == BZ_ACT_DICE) cp2[jn] = dice_inv_den(ep, cp2[jn]);
  }
  constexpr int OPITCH = BN * 2 + 16;
  char* lout = smem;
  auto epilogue = [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int jn = 0; jn < TN; ++jn) {
      const int nl = wn * 64 + jn * 32 + (lane & 31);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int ml = wm * 128 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          float v = fmaf(ep.alpha, acc[i][jn][r], cbias[jn]);  // (cbias: beta * bias of the column, or 0)
          v = apply_act_t<ACT>(v, ep, cp0[jn], cp1[jn], cp2[jn]);
          store_out<OutT>((OutT*)(lout + ml * OPITCH) + nl, v);
        }
      }
    }
  };
  switch (ep.act) {
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
  __syncthreads();
  constexpr int OCPR = BN * 2 / 16;
  for (int q = tid; q < BM * OCPR; q += NT) {
    const int ml = q / OCPR, ch = q % OCPR;
    const int m = m0 + ml, n = n0 + ch * 8;
    if (m < M && n < N) *(uint4*)((char*)(Y + out_index(ep, m, n, ldy))) = *(const uint4*)(lout + ml * OPITCH + ch * 16);
  }
}
#undef BZ_PIN_PHASE

// ---------------------------------------------------------------------------------------------
// skinny kernel: N <= 8
// ---------------------------------------------------------------------------------------------
template <int DT, typename OutT>
__global__ __launch_bounds__(256) void bz_fc_skinny_kernel(const char* __restrict__ A, const char* __restrict__ W,
                                                           OutT* __restrict__ Y, int M, int N, int K, int64_t lda,
                                                           int64_t ldw, int64_t ldy, bool vec_a, bool vec_w, int lpr,
                                                           Epilogue ep) {
  constexpr int CH = In<DT>::kChunk;
  const int tid = threadIdx.x;
  const int g = tid / lpr, l = tid - g * lpr;
  const int rows_per_wg = 256 / lpr;
  const int nchunks = (K + CH - 1) / CH;
  // per-column parameters first: their latency hides under the row loads
  float cb[kSkinnyMaxN], q0[kSkinnyMaxN], q1[kSkinnyMaxN], q2[kSkinnyMaxN];
#pragma unroll
  for (int n = 0; n < kSkinnyMaxN; ++n) {
    const int nn = n < N ? n : N - 1;
    cb[n] = ep.bias_rows == 1 ? ep.bias[nn] : 0.f;
    q0[n] = q1[n] = q2[n] = 0.f;
    if (ep.act == BZ_ACT_PRELU) q0[n] = ep.p0[ep.act_size == 1 ? 0 : nn];
    if (ep.act == BZ_ACT_DICE) {
      q0[n] = ep.p0[nn];
      q1[n] = ep.p1[nn];
      q2[n] = ep.p2[nn];
    }
  }
  for (int64_t m = (int64_t)blockIdx.x * rows_per_wg + g; m < M; m += (int64_t)gridDim.x * rows_per_wg) {
    float acc[kSkinnyMaxN];
#pragma unroll
    for (int n = 0; n < kSkinnyMaxN; ++n) acc[n] = 0.f;
    for (int c = l; c < nchunks; c += lpr) {
      float a[CH];
      chunk_to_float<DT>(load_chunk<DT>(A, m, lda, c * CH, K, vec_a), a);
#pragma unroll
      for (int n = 0; n < kSkinnyMaxN; ++n) {
        if (n < N) {
          float w[CH];
          chunk_to_float<DT>(load_chunk<DT>(W, n, ldw, c * CH, K, vec_w), w);
#pragma unroll
          for (int i = 0; i < CH; ++i) acc[n] = fmaf(a[i], w[i], acc[n]);
        }
      }
    }
    // reduce over the lane group (lpr is a power of two <= 64, groups are lane aligned)
    for (int d = lpr >> 1; d > 0; d >>= 1) {
#pragma unroll
      for (int n = 0; n < kSkinnyMaxN; ++n) acc[n] += __shfl_xor(acc[n], d, 64);
    }
    if (l == 0) {
      float v[kSkinnyMaxN];
#pragma unroll
      for (int n = 0; n < kSkinnyMaxN; ++n) {
        v[n] = 0.f;
        if (n < N) {
          float x = ep.alpha * acc[n];
          if (ep.bias_rows == 1)
            x += ep.beta * cb[n];
          else if (ep.bias_rows > 1)
            x += ep.beta * ep.bias[full_bias_index(ep, m, n, M, N)];
          v[n] = x;
        }
      }
      if (ep.act == BZ_ACT_SOFTMAX) {  // softmax_op.cc:21-78: subtract max, exp, sum in order, divide
        float mx = v[0];
#pragma unroll
        for (int n = 1; n < kSkinnyMaxN; ++n)
          if (n < N) mx = v[n] > mx ? v[n] : mx;
        float sum = 0.f;
#pragma unroll
        for (int n = 0; n < kSkinnyMaxN; ++n)
          if (n < N) {
            v[n] = expf(v[n] - mx);
            sum += v[n];
          }
#pragma unroll
        for (int n = 0; n < kSkinnyMaxN; ++n)
          if (n < N) v[n] = v[n] / sum;
      } else {
#pragma unroll
        for (int n = 0; n < kSkinnyMaxN; ++n)
          if (n < N) v[n] = apply_act_regs(v[n], ep, q0[n], q1[n], q2[n]);
      }
#pragma unroll
      for (int n = 0; n < kSkinnyMaxN; ++n)
        if (n < N) store_out<OutT>(Y + out_index(ep, m, n, ldy), v[n]);
    }
  }
}


template <int DT, typename OutT, int BM, int BN, int BK, int WM, int WN, int D, bool ALIGNED, bool HEAD = false>
int launch_mfma(const bz_fc_desc& d, const Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st) {
  const int tiles_m = (d.m + BM - 1) / BM, tiles_n = (d.n + BN - 1) / BN;
  // output rows 16-byte aligned and N a whole number of 16-byte chunks: coalesced stores through LDS
  // (with split outputs every slice must start on a chunk boundary as well)
  const bool vec_y = d.y != nullptr && ((uintptr_t)d.y % 16 == 0) && ((d.ldy * (int64_t)sizeof(OutT)) % 16 == 0) &&
                     (d.n % (16 / (int)sizeof(OutT)) == 0) &&
                     (d.n_split == 0 || (d.n_split % (16 / (int)sizeof(OutT)) == 0 && (d.y_split_stride * (int64_t)sizeof(OutT)) % 16 == 0));
  HeadArgs head = {};
  if (HEAD) {
    head.w = (const char*)d.head_w;
    head.bias = d.head_bias;
    head.y = d.head_y;
    head.ldw = d.head_ldw;
    head.ldy = d.head_ldy;
    head.n = d.head_n;
    head.act = d.head_act;
    head.out_dtype = d.head_out_dtype;
  }
  hipLaunchKernelGGL((bz_fc_mfma_kernel<DT, OutT, BM, BN, BK, WM, WN, D, ALIGNED, HEAD>), dim3(tiles_m * tiles_n), dim3(WM * WN * 64), 0,
                     st, (const char*)d.a, (const char*)d.w, (OutT*)d.y, d.m, d.n, d.k, d.lda, d.ldw, d.ldy, vec_a, vec_w, vec_y,
                     tiles_m, ep, head);
  BZ_LAUNCH_OK("bz_fc_mfma_kernel");
  return BZ_OK;
}


// 2-byte operands and outputs, 16-byte aligned rows on all three, K a whole number of 64-wide tiles
template <int DT, typename OutT>
int launch_stream(const bz_fc_desc& d, const Epilogue& ep, hipStream_t st) {
  const int tiles_m = (d.m + kStreamBM - 1) / kStreamBM, tiles_n = (d.n + kStreamBN - 1) / kStreamBN;
  const int grid = (tiles_m + 7) / 8 * 8 * tiles_n;
  // more dynamic LDS than the default limit: raised once per kernel and device
  static std::mutex mu;
  static bool raised[64] = {};
  int dev = 0;
  BZ_HIP_OK(hipGetDevice(&dev));
  {
    std::lock_guard<std::mutex> lock(mu);
    if (dev >= 0 && dev < 64 && !raised[dev]) {
      BZ_HIP_OK(hipFuncSetAttribute((const void*)bz_fc_stream_kernel<DT, OutT>, hipFuncAttributeMaxDynamicSharedMemorySize, kStreamLds));
      raised[dev] = true;
    }
  }
  hipLaunchKernelGGL((bz_fc_stream_kernel<DT, OutT>), dim3(grid), dim3(2 * kStreamCompute), kStreamLds, st, (const char*)d.a,
                     (const char*)d.w, (OutT*)d.y, d.m, d.n, d.k, d.lda, d.ldw, d.ldy, tiles_m, tiles_n, ep);
  BZ_LAUNCH_OK("bz_fc_stream_kernel");
  return BZ_OK;
}


// Layer + skinny head in one launch: a workgroup owns whole rows of the first layer's output (N <= 256).
template <int DT, typename OutT>
int dispatch_head(const bz_fc_desc& d, const Epilogue& ep, hipStream_t st) {
  constexpr int BK = In<DT>::kSize == 2 ? 64 : 32;
  if (d.n <= 64) {
    if ((d.m + 63) / 64 >= 256) return launch_mfma<DT, OutT, 64, 64, BK, 2, 2, 4, true, true>(d, ep, true, true, st);
    return launch_mfma<DT, OutT, 32, 64, BK, 1, 2, 4, true, true>(d, ep, true, true, st);
  }
  if (d.n <= 128) return launch_mfma<DT, OutT, 32, 128, BK, 1, 4, 4, true, true>(d, ep, true, true, st);
  // eight waves: with one workgroup per 32 rows only M / 32 CUs work, and each has 288 KB of operands to pull in
  // (two K tiles in flight: with eight waves taking turns that hides the loads, and it is faster than four both alone,
  // 10.5 against 11.3 us on config 2's 512 -> 256 -> 2, and next to other kernels)
  return launch_mfma<DT, OutT, 32, 256, BK, 1, 8, 2, true, true>(d, ep, true, true, st);
}

template <int DT, typename OutT>
int dispatch_tiles(const bz_fc_desc& d, const Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st) {
  constexpr int BK = In<DT>::kSize == 2 ? 64 : 32;
  const int64_t wg128 = (int64_t)((d.m + 127) / 128) * ((d.n + 127) / 128);
  const int64_t wg64 = (int64_t)((d.m + 63) / 64) * ((d.n + 63) / 64);
  // rows 16-byte aligned and K a whole number of chunks: branch-free loads, several tiles in flight
  const bool aligned = vec_a && vec_w && d.k % In<DT>::kChunk == 0;
  if (!aligned) return launch_mfma<DT, OutT, 64, 64, BK, 2, 2, 1, false>(d, ep, vec_a, vec_w, st);
  // Largest first, and never a tile much wider than N.  128x256 with eight waves and three K tiles in flight fills the
  // chip once it has a workgroup per CU (its fp32 output tile would not fit the operand buffers it is staged in, so
  // 2-byte outputs only); below that, 128x128; then 64x128 while that still gives two workgroups per CU; then the
  // latency-bound small tiles.
  const int64_t wg128x256 = (int64_t)((d.m + 127) / 128) * ((d.n + 255) / 256);
  const int64_t wg64x128 = (int64_t)((d.m + 63) / 64) * ((d.n + 127) / 128);
  if constexpr (sizeof(OutT) == 2 && In<DT>::kSize == 2) {
    // the streaming kernel once its 256x128 tiles keep most CUs busy and K is deep enough to pay for filling its ring
    // (8192 x 12800 -> 1024 bf16: 192 against 238 us; 4096^3: 128 against 139 us)
    const int64_t wg_stream = (int64_t)((d.m + kStreamBM - 1) / kStreamBM) * ((d.n + kStreamBN - 1) / kStreamBN);
    const bool vec_y = d.y != nullptr && ((uintptr_t)d.y % 16 == 0) && ((d.ldy * 2) % 16 == 0) && d.n % 8 == 0 &&
                       (d.n_split == 0 || (d.n_split % 8 == 0 && (d.y_split_stride * 2) % 16 == 0));
    // (a bias of one row per sample stays with the tile kernels: the streaming kernel's epilogue handles 128 outputs a
    // lane, and an index and a bounds check per output for that rare form cost every layer ten times the activation)
    if (wg_stream >= 200 && d.k % kStreamBK == 0 && d.k >= 8 * kStreamBK && vec_y && d.bias_rows <= 1)
      return launch_stream<DT, OutT>(d, ep, st);
  }
  if constexpr (sizeof(OutT) == 2 && In<DT>::kSize == 2) {
    // (256x256 once even that fills the chip: 4096^3 bf16 987 against 885 TFLOP/s; with fp32 operands these two tiles
    // do not fit the registers)
    const int64_t wg256 = (int64_t)((d.m + 255) / 256) * ((d.n + 255) / 256);
    if (wg256 >= 256 && d.bias_rows <= 1) return launch_mfma<DT, OutT, 256, 256, BK, 4, 2, 2, true>(d, ep, vec_a, vec_w, st);
    if (d.n > 128 && wg128x256 >= 256) return launch_mfma<DT, OutT, 128, 256, BK, 2, 4, 3, true>(d, ep, vec_a, vec_w, st);
  }
  // tall and narrow (the attention MLP over batch x history rows): one 96-wide tile reads A once
  if (d.n > 64 && d.n <= 96 && (d.m + 127) / 128 >= 256)
    return launch_mfma<DT, OutT, 128, 96, BK, 4, 1, 2, true>(d, ep, vec_a, vec_w, st);
  if (d.n > 64 && wg128 >= 512) return launch_mfma<DT, OutT, 128, 128, BK, 2, 2, 3, true>(d, ep, vec_a, vec_w, st);
  if (d.n > 64 && wg64x128 >= 512) return launch_mfma<DT, OutT, 64, 128, BK, 2, 2, 4, true>(d, ep, vec_a, vec_w, st);
  if (wg64 >= 256) {
    // Four K tiles in flight (120 VGPRs, three waves per SIMD).  Seven save a round trip on config 2's 896-deep layer
    // when the kernel runs alone (9.2 against 9.8 us) but hold 182 VGPRs, and next to the kernels of other serving
    // threads the leaner one wins: 127.5 against 121 M samples/s at the same forward latency.
    return launch_mfma<DT, OutT, 64, 64, BK, 2, 2, 4, true>(d, ep, vec_a, vec_w, st);
  }
  return launch_mfma<DT, OutT, 32, 64, BK, 1, 2, 4, true>(d, ep, vec_a, vec_w, st);
}

template <int DT, typename OutT>
int dispatch_skinny(const bz_fc_desc& d, const Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st) {
  const int nchunks = (d.k + In<DT>::kChunk - 1) / In<DT>::kChunk;
  int lpr = 1;
  while (lpr < nchunks && lpr < 64) lpr <<= 1;
  const int rows_per_wg = 256 / lpr;
  int64_t grid = ((int64_t)d.m + rows_per_wg - 1) / rows_per_wg;
  if (grid > 256 * 32) grid = 256 * 32;
  hipLaunchKernelGGL((bz_fc_skinny_kernel<DT, OutT>), dim3((int)grid), dim3(256), 0, st, (const char*)d.a,
                     (const char*)d.w, (OutT*)d.y, d.m, d.n, d.k, d.lda, d.ldw, d.ldy, vec_a, vec_w, lpr, ep);
  BZ_LAUNCH_OK("bz_fc_skinny_kernel");
  return BZ_OK;
}

template <int DT>
int dispatch_out(const bz_fc_desc& d, const Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st) {
  const bool skinny = d.n <= kSkinnyMaxN;
  switch (d.out_dtype) {
    case BZ_F32:
      return skinny ? dispatch_skinny<DT, float>(d, ep, vec_a, vec_w, st) : dispatch_tiles<DT, float>(d, ep, vec_a, vec_w, st);
    case BZ_F16:
      return skinny ? dispatch_skinny<DT, __half>(d, ep, vec_a, vec_w, st)
                    : dispatch_tiles<DT, __half>(d, ep, vec_a, vec_w, st);
    case BZ_BF16:
      return skinny ? dispatch_skinny<DT, __hip_bfloat16>(d, ep, vec_a, vec_w, st)
                    : dispatch_tiles<DT, __hip_bfloat16>(d, ep, vec_a, vec_w, st);
    default:
      return bz::fail(BZ_EINVAL, "bz_fc_fused: unsupported out dtype %d", d.out_dtype);
  }
}


// one operand type's entry: the layer with a head, or the plain layer (skinny / tile / streaming kernel)
template <int DT, typename T>
int run_typed(const bz_fc_desc& d, const Epilogue& ep, bool vec_a, bool vec_w, hipStream_t st) {
  if (d.head_n != 0) return dispatch_head<DT, T>(d, ep, st);
  return dispatch_out<DT>(d, ep, vec_a, vec_w, st);
}

}  // namespace
