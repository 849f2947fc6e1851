// fc_pieces.hip -- an FC layer whose A operand is computed on the fly from pieces (bz_fc_desc.a_pieces), for gfx950.
// Stands in for the reference's Concat of elementwise results followed by a 3-D Gemm (+ the activation after it) in the
// attention unit of a DIN model (tools/example_model/din/model/graph_ulf.txt; blaze/operator/op/concat_op.h:46-121,
// elementwise_op.cc:28-165, gemm_op.h:52-58,77-91) without the tensor between them.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <mutex>
#include <type_traits>

#include "bz_common.h"
#include "bz_pieces.h"
#include "fc_common.h"

namespace {

using namespace bz::fc;

// ---------------------------------------------------------------------------------------------
// pieces kernel: a tall layer of few columns and small K whose A operand is computed on the fly
// ---------------------------------------------------------------------------------------------
// A row of A is the concatenation of up to NP pieces x | x op y (bz_concat_ew's model, bz_pieces.h): the attention unit's
// [q, k, q-k, q*k] with q broadcast over the history.  Stored first and read back, that tensor is 22 MB each way on a
// batch of 1024 x 50 positions x 216 columns; here a workgroup writes its 128 rows of it into LDS and nowhere else.
// The rest follows from K being small (<= 224) and N narrow (<= 96):
//  - all of K is on chip at once, so there is no K loop over memory: one trip for the pieces' operands, one barrier,
//    then MFMAs only;
//  - the whole weight is kept in registers as MFMA fragments (N/32 x K/16 fragments of 4 registers: 168 for 96 x 224),
//    loaded straight from global memory while the pieces are computed; LDS holds only the A tile (59 KB for K = 216), two
//    workgroups a CU;
//  - after the barrier a wave touches only its own 32 rows, so it stages its outputs in those rows' LDS without
//    another barrier.
// The elements of A are rounded to the tensor type as the concat kernel would have stored them (bz::cew_piece), so the
// result is the two-launch form's up to the order of the K sum.
constexpr int kPiecesBM = 128, kPiecesKS = 14, kPiecesMaxN = 96;

// the layers that follow in the same launch (bz_fc_desc.next, head_*)
struct ChainArgs {
  const char* w2;      // [n2, ldw2]
  void* y2;            // [M, ldy2] or null
  int64_t ldw2, ldy2;
  int n2;              // 9..64
  Epilogue ep2;
  const char* w3;      // [n3, ldw3] or null
  const float* bias3;
  void* y3;            // [M, ldy3]
  int64_t ldw3, ldy3;
  int n3, act3, y3_dtype;  // n3 = 0: no third layer
};
constexpr int kChainKS = kPiecesMaxN / 16;  // K steps of the second layer (its K is the first layer's N)
constexpr int kChainPitch = kPiecesMaxN * 2 + 16;  // bytes between the rows of the second layer's weight in LDS

// Row pitch of the A tile in LDS.  A wave stages its outputs in its own 32 rows of the tile once the MFMAs have read
// them: a row of tn column blocks of the first layer, and of 64 two-byte columns of a chained second layer, must fit.
__host__ __device__ inline int pieces_pitch(int k, int tn, int out_size, bool chain) {
  int pitch = (k + 15) / 16 * 16 * 2 + 16;
  const int o1 = tn * 32 * out_size + 16, o2 = chain ? 64 * 2 + 16 : 0;
  pitch = pitch > o1 ? pitch : o1;
  return pitch > o2 ? pitch : o2;
}
// dynamic LDS of a workgroup: the tile, the first layer's column parameters and, for a chain, the third layer's weight,
// the second layer's column parameters and its weight
__host__ __device__ inline int pieces_lds(int k, int tn, int out_size, bool chain) {
  return kPiecesBM * pieces_pitch(k, tn, out_size, chain) + 4 * kPiecesMaxN * 4 +
         (chain ? kSkinnyMaxN * 64 * 4 + 4 * 64 * 4 + 64 * kChainPitch : 0);
}

// XY4: the pieces are exactly [x, y, x - y, x * y] of two operands (the attention input): a lane loads x and y once and
// makes all four from them, instead of addressing and loading eight operands.
// CHAIN: a wave goes on with its 32 rows through a second layer of at most 64 columns and a skinny third one; what the
// layers hand each other is rounded to the tensor type and staged in the wave's rows of LDS, where the separate launches
// would have stored it and read it back.
template <int DT, typename OutT, int VEC, int NP, int TN, bool XY4, bool CHAIN>
__global__ __launch_bounds__(256, 2) void bz_fc_pieces_kernel(bz::CewP p, const char* __restrict__ W, OutT* __restrict__ Y, int M,
                                                              int N, int K, int64_t ldw, int64_t ldy, bool stage_y, Epilogue ep,
                                                              ChainArgs ch) {
  using T = In<DT>;
  using ET = typename std::conditional<DT == BZ_F16, __half, __hip_bfloat16>::type;
  using Pack = bz::CewPack<ET, VEC>;
  constexpr int BM = kPiecesBM, NT = 256;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int KP = (K + 15) / 16 * 16;   // K as the MFMAs see it; columns K.. are zero
  const int KS = KP / 16;
  // bytes between the tile's rows: the 16 spread the 16 rows of a ds_read_b128 phase over all banks; at least what a row
  // of the outputs staged there takes (pieces_pitch() on the host)
  const int pitch = pieces_pitch(K, TN, (int)sizeof(OutT), CHAIN);
  const int m0 = blockIdx.x * BM;
  const int frow = lane & 31, fhalf = lane >> 5;

  // LDS behind the A tile: the layers' per-column epilogue parameters as finished floats ([4][96]: beta * bias, slope or
  // gamma, mean, log2(e) / den; [4][64] for a second layer), a third layer's weight as floats [8][64] (zero beyond its n3
  // rows and n2 columns) and a second layer's weight as the tile the fragment reads expect ([64] rows of kChainPitch
  // bytes).  pieces_lds() on the host.
  float* ps1 = (float*)(smem + BM * pitch);
  float* w3s = ps1 + 4 * kPiecesMaxN;
  float* ps2 = w3s + kSkinnyMaxN * 64;
  char* w2s = (char*)(ps2 + 4 * 64);

  // Everything the workgroup needs from memory is asked for here, at once, and nothing waits before all of it is in
  // flight: first what comes from L2 and is needed first (the weights, the parameters), then the A tile's operands from
  // HBM.  Loads return in the order they were issued, so the weights can be put into LDS while the operands travel.
  //
  // The first layer's weight goes through LDS: row n of the tile = column n of the layer, coalesced 16-byte loads, and
  // every wave then reads its fragments (lane: column frow of block j, k = 16*ks + 8*fhalf .. +7) from there.  Loaded
  // straight from memory as fragments, a load instruction touched 32 different 128-byte lines, and a workgroup's four
  // waves asked L1 for the same 43 KB four times: 10 000 cycles of a workgroup's 40 000.
  constexpr int kWPasses = TN * 4;  // 32 lanes a row (28 chunks of 16 bytes at most), 8 rows a pass
  const int wc = tid & 31, wr = tid >> 5;
  uint4 wreg[kWPasses];
  {
    const bool have = wc * 8 < KP && wc * 8 < ldw;  // (rows are zero from K up to ldw, a multiple of 8)
#pragma unroll
    for (int i = 0; i < kWPasses; ++i) {
      int n = wr + 8 * i;
      n = n < N ? n : N - 1;
      wreg[i] = *(const uint4*)(W + ((int64_t)n * ldw + (have ? wc * 8 : 0)) * 2);
      if (!have) wreg[i] = make_uint4(0, 0, 0, 0);
    }
  }
  // a second layer's weight the same way: 16 lanes a row (12 chunks at most), 16 rows a pass
  constexpr int kW2Passes = CHAIN ? 4 : 0;
  uint4 w2reg[kW2Passes + 1];
  if constexpr (CHAIN) {
    const int c2 = tid & 15;
    const bool have = c2 * 8 < kPiecesMaxN && c2 * 8 < ch.ldw2;
#pragma unroll
    for (int i = 0; i < kW2Passes; ++i) {
      int n2 = (tid >> 4) + 16 * i;
      n2 = n2 < ch.n2 ? n2 : ch.n2 - 1;
      w2reg[i] = *(const uint4*)(ch.w2 + ((int64_t)n2 * ch.ldw2 + (have ? c2 * 8 : 0)) * 2);
      if (!have) w2reg[i] = make_uint4(0, 0, 0, 0);
    }
  }
  // the parameters: thread t makes entries t and t + 256 of ps1 and entry t of ps2.  Here only the loads, with no branch
  // round them (the compiler would wait there for everything asked so far; an entry that does not exist reads the
  // weight's first word instead) and nothing computed from them yet (that would be a wait for memory as well).
  auto param_use = [&](const Epilogue& e, int which) {
    const bool dice = e.act == BZ_ACT_DICE, prelu = e.act == BZ_ACT_PRELU;
    return which == 0 ? e.bias_rows == 1 : (which == 1 ? (dice || prelu) : dice);
  };
  auto param_load = [&](const Epilogue& e, int which, int n) -> float {
    const float* src = which == 0 ? e.bias : (which == 1 ? e.p0 : (which == 2 ? e.p1 : e.p2));
    const int at = (which == 1 && e.act == BZ_ACT_PRELU && e.act_size == 1) ? 0 : n;
    return *(param_use(e, which) ? src + at : (const float*)W);
  };
  auto param_finish = [&](const Epilogue& e, int which, float v) -> float {
    const float r = which == 0 ? e.beta * v : (which == 3 ? dice_inv_den(e, v) : v);
    return param_use(e, which) ? r : 0.f;
  };
  int which1[2];
  float pv1[2], pv2 = 0.f, w3v[2] = {0.f, 0.f};
  bool w3use[2] = {false, false};
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    int q = tid + h * NT;
    q = q < 4 * kPiecesMaxN ? q : 0;
    which1[h] = q / kPiecesMaxN;
    const int n = q - which1[h] * kPiecesMaxN;
    pv1[h] = param_load(ep, which1[h], n < N ? n : N - 1);
  }
  if constexpr (CHAIN) {
    const int n2 = tid & 63;
    pv2 = param_load(ch.ep2, tid >> 6, n2 < ch.n2 ? n2 : ch.n2 - 1);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int q = tid + h * NT, j = q >> 6, c = q & 63;
      w3use[h] = j < ch.n3 && c < ch.n2;
      w3v[h] = bz::ldv<ET>(w3use[h] ? (const ET*)ch.w3 + (int64_t)j * ch.ldw3 + c : (const ET*)W);
    }
  }
  // into LDS: the first layer's weight into the A tile's own rows (it is gone from there before the tile is written)
  uint4 wf[TN][kPiecesKS];
  auto stage_and_read_w = [&]() {
    if (wc * 8 < KP) {
#pragma unroll
      for (int i = 0; i < kWPasses; ++i) *(uint4*)(smem + (wr + 8 * i) * pitch + wc * 16) = wreg[i];
    }
    if constexpr (CHAIN) {
      const int c2 = tid & 15;
      if (c2 * 8 < kPiecesMaxN) {
#pragma unroll
        for (int i = 0; i < kW2Passes; ++i) *(uint4*)(w2s + ((tid >> 4) + 16 * i) * kChainPitch + c2 * 16) = w2reg[i];
      }
      ps2[tid] = param_finish(ch.ep2, tid >> 6, pv2);
      w3s[tid] = w3use[0] ? w3v[0] : 0.f;
      w3s[tid + NT] = w3use[1] ? w3v[1] : 0.f;
    }
    ps1[tid] = param_finish(ep, which1[0], pv1[0]);
    if (tid + NT < 4 * kPiecesMaxN) ps1[tid + NT] = param_finish(ep, which1[1], pv1[1]);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int ks = 0; ks < kPiecesKS; ++ks)
        wf[j][ks] = ks < KS ? *(const uint4*)(smem + (j * 32 + frow) * pitch + ks * 32 + fhalf * 16) : make_uint4(0, 0, 0, 0);
    __syncthreads();  // every wave has its fragments: the rows are free for the A tile
  };

  // the A tile: a lane owns VEC columns of a piece and walks the pieces; 64 / (W / VEC) rows share a wave.  kGenRows rows
  // of a lane are in flight at once (no branch round the loads: a row beyond M reads row M-1 and is not stored; one
  // beyond the tile reads the lane's first row again, a cache hit), so the tile costs BM / (4 * rows_per_wave * kGenRows)
  // trips to memory, not one per row: one for the attention input of 4 x 54 columns.  kGenRows keeps the rows in flight
  // within 32 registers where x and y are loaded once and within 64 otherwise (8 columns a lane mean at most 8 lanes a row,
  // so 4 rows in flight already cover the tile); the weight's 168 registers are live at the same time.
  {
    constexpr int kGenRows = XY4 ? (VEC == 8 ? 4 : 16) : (TN == 3 ? (VEC == 8 ? 1 : 4) : (VEC == 8 ? 2 : 8));
    constexpr int NL = XY4 ? 2 : NP;  // operands loaded a row: x and y once, or x and y of every piece
    const int per_piece = p.col0[1] / VEC;
    const int rows_per_wave = 64 / per_piece;
    const int sub = lane / per_piece, cv = lane - sub * per_piece;
    const uint32_t r1 = (uint32_t)p.r1;
    // row -> (row / r1, row % r1): one division for the tile's first row (the same for every lane); a row of the tile is
    // less than BM rows further, and a quotient that small is exact in fp32 up to a correction by one
    const uint32_t q0_ = (uint32_t)m0 / r1, rem0 = (uint32_t)m0 - q0_ * r1;
    const float inv_r1 = 1.f / (float)r1;
    auto split_row = [&](uint32_t row, uint32_t* i0, uint32_t* i1) {
      const uint32_t t = row - (uint32_t)m0 + rem0;  // < r1 + BM; (a row clamped to M - 1 is not before m0)
      uint32_t q = (uint32_t)((float)t * inv_r1);
      q -= (q * r1 > t);
      q += ((q + 1) * r1 <= t);
      *i0 = q0_ + q;
      *i1 = t - q * r1;
    };
    const int step = 4 * rows_per_wave;
    const int base0 = wave * rows_per_wave + sub;
    Pack xs[kGenRows][NL], ys[kGenRows][XY4 ? 1 : NP];
    auto gen_load = [&](int base) {
#pragma unroll
      for (int u = 0; u < kGenRows; ++u) {
        const int rl = base + u * step;
        uint32_t row = (uint32_t)(m0 + (rl < BM ? rl : base));
        row = row < (uint32_t)M ? row : (uint32_t)M - 1;
        uint32_t i0, i1;
        split_row(row, &i0, &i1);
        if constexpr (XY4) {
          xs[u][0] = *(const Pack*)((const ET*)p.x[0] + (int64_t)i0 * p.xs[0][0] + (int64_t)i1 * p.xs[0][1] + cv * VEC);
          xs[u][1] = *(const Pack*)((const ET*)p.x[1] + (int64_t)i0 * p.xs[1][0] + (int64_t)i1 * p.xs[1][1] + cv * VEC);
        } else {
#pragma unroll
          for (int k = 0; k < NP; ++k) {
            const int kk = k < p.n ? k : 0;
            const bool two = p.op[kk] != BZ_EW_ASSIGN;
            const ET* yb = two ? (const ET*)p.y[kk] : (const ET*)p.x[kk];
            const int64_t ys0 = two ? p.ys[kk][0] : p.xs[kk][0], ys1 = two ? p.ys[kk][1] : p.xs[kk][1];
            xs[u][k] = *(const Pack*)((const ET*)p.x[kk] + (int64_t)i0 * p.xs[kk][0] + (int64_t)i1 * p.xs[kk][1] + cv * VEC);
            ys[u][k] = *(const Pack*)(yb + (int64_t)i0 * ys0 + (int64_t)i1 * ys1 + cv * VEC);
          }
        }
      }
    };
    auto gen_store = [&](int base) {
      // (an opaque copy: what the loads computed per row - offsets, predicates - is worked out again here instead of
      // being kept in registers across the weight's loads, where there are none to spare)
      asm volatile("" : "+v"(base));
#pragma unroll
      for (int u = 0; u < kGenRows; ++u) {
        const int rl = base + u * step;
        if constexpr (XY4) {
          if (rl < BM && m0 + rl < M) {
            char* dst = smem + rl * pitch + cv * VEC * 2;
            const int wb = p.col0[1] * 2;  // bytes of a piece
            *(Pack*)dst = xs[u][0];
            *(Pack*)(dst + wb) = xs[u][1];
            *(Pack*)(dst + 2 * wb) = bz::cew_piece<ET, VEC>(BZ_EW_SUB, xs[u][0], xs[u][1]);
            *(Pack*)(dst + 3 * wb) = bz::cew_piece<ET, VEC>(BZ_EW_MUL, xs[u][0], xs[u][1]);
          }
        } else {
#pragma unroll
          for (int k = 0; k < NP; ++k) {
            const Pack o = bz::cew_piece<ET, VEC>(p.op[k < p.n ? k : 0], xs[u][k], ys[u][k]);
            if (k < p.n && rl < BM && m0 + rl < M) *(Pack*)(smem + rl * pitch + (p.col0[k] + cv * VEC) * 2) = o;
          }
        }
      }
    };
    // (the lanes left over when the piece's width does not divide 64 load what their neighbours load and store nothing:
    // no branch round the loads)
    const bool mine = sub < rows_per_wave;
    gen_load(base0);
    stage_and_read_w();
    if (mine) gen_store(base0);
    for (int base = base0 + step * kGenRows; base < BM; base += step * kGenRows) {
      gen_load(base);
      if (mine) gen_store(base);
    }
    // columns K .. KP-1 of every row (at most 15)
    if (tid < BM)
      for (int c = K; c < KP; ++c) *(unsigned short*)(smem + tid * pitch + c * 2) = 0;
  }
  __syncthreads();

  floatx16 acc[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  const char* arow = smem + (wave * 32 + frow) * pitch + fhalf * 16;
  uint4 fa = *(const uint4*)arow;
#pragma unroll
  for (int ks = 0; ks < kPiecesKS; ++ks) {
    if (ks < KS) {
      const uint4 cur = fa;
      if (ks + 1 < KS) fa = *(const uint4*)(arow + (ks + 1) * 32);
#pragma unroll
      for (int j = 0; j < TN; ++j) T::mma(cur, wf[j][ks], acc[j]);
    }
  }

  // the epilogues' column parameters and the second layer's weight fragments, from LDS (the first layer's fragments are
  // dead from here on)
  float cbias[TN], cp0[TN], cp1[TN], cp2[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = j * 32 + frow;
    cbias[j] = ps1[n];
    cp0[j] = ps1[kPiecesMaxN + n];
    cp1[j] = ps1[2 * kPiecesMaxN + n];
    cp2[j] = ps1[3 * kPiecesMaxN + n];
  }
  constexpr int TN2 = CHAIN ? 2 : 0, KS2MAX = CHAIN ? kChainKS : 0;
  const int KS2 = (N + 15) / 16;
  uint4 wf2[TN2 + 1][KS2MAX + 1];
  float b2[TN2 + 1], q0[TN2 + 1], q1[TN2 + 1], q2[TN2 + 1];
#pragma unroll
  for (int j = 0; j < TN2; ++j) {
    const int n2 = j * 32 + frow;
#pragma unroll
    for (int ks = 0; ks < KS2MAX; ++ks)
      wf2[j][ks] = ks < KS2 ? *(const uint4*)(w2s + n2 * kChainPitch + ks * 32 + fhalf * 16) : make_uint4(0, 0, 0, 0);
    b2[j] = ps2[n2];
    q0[j] = ps2[64 + n2];
    q1[j] = ps2[128 + n2];
    q2[j] = ps2[192 + n2];
  }
  // epilogue: lane owns column n of each block, rows 8*(r/4) + 4*(lane/32) + r%4 of the wave's 32
  constexpr int OS = (int)sizeof(OutT);
  constexpr int OPITCH = TN * 32 * OS + 16;
  char* lout = smem + wave * 32 * pitch;  // this wave's own rows of the A tile
  auto epilogue = [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = j * 32 + frow;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int ml = 8 * (r >> 2) + 4 * fhalf + (r & 3);
        const int m = m0 + wave * 32 + ml;
        float v = fmaf(ep.alpha, acc[j][r], cbias[j]);  // (cbias: beta * bias of the column, or 0)
        v = apply_act_t<ACT>(v, ep, cp0[j], cp1[j], cp2[j]);
        // always through LDS: an address and a bounds check per element here cost more than the whole activation
        store_out<OutT>((OutT*)(lout + ml * OPITCH) + n, (!CHAIN || n < N) ? v : 0.f);  // (a next layer's operand: zero beyond N)
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
  if (stage_y && Y != nullptr) {
    const int ocpr = N * OS / 16;  // 16-byte chunks per output row (N * OS is a multiple of 16 when stage_y)
    for (int q = lane; q < 32 * ocpr; q += 64) {
      const int ml = q / ocpr, c16 = q - ml * ocpr;
      const int m = m0 + wave * 32 + ml;
      if (m < M) *(uint4*)((char*)(Y + (int64_t)m * ldy) + c16 * 16) = *(const uint4*)(lout + ml * OPITCH + c16 * 16);
    }
  } else if (Y != nullptr) {  // rows that do not start on 16 bytes: element by element
    for (int q = lane; q < 32 * N; q += 64) {
      const int ml = q / N, n = q - ml * N;
      const int m = m0 + wave * 32 + ml;
      if (m < M) Y[(int64_t)m * ldy + n] = ((const OutT*)(lout + ml * OPITCH))[n];
    }
  }
  if constexpr (CHAIN) {
    static_assert(!CHAIN || sizeof(OutT) == 2, "the layers hand each other the operand type");
    // ---- second layer: A = the staged rows [32, N] (K2 = N), at most two column blocks
    floatx16 acc2[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc2[j][r] = 0.f;
    const char* a2 = lout + frow * OPITCH + fhalf * 16;
#pragma unroll
    for (int ks = 0; ks < kChainKS; ++ks) {
      if (ks < KS2) {
        const uint4 cur = *(const uint4*)(a2 + ks * 32);
#pragma unroll
        for (int j = 0; j < 2; ++j) T::mma(cur, wf2[j][ks], acc2[j]);
      }
    }
    // its activated output, staged over the first layer's (every read of that has been consumed by the MFMAs above)
    constexpr int OPITCH2 = 64 * 2 + 16;
    auto epilogue2 = [&](auto act_c) {
      constexpr int ACT = decltype(act_c)::value;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n2 = j * 32 + frow;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int ml = 8 * (r >> 2) + 4 * fhalf + (r & 3);
          float v = fmaf(ch.ep2.alpha, acc2[j][r], b2[j]);
          v = apply_act_t<ACT>(v, ch.ep2, q0[j], q1[j], q2[j]);
          store_out<OutT>((OutT*)(lout + ml * OPITCH2) + n2, n2 < ch.n2 ? v : 0.f);
        }
      }
    };
    switch (ch.ep2.act) {
      case BZ_ACT_PRELU:
        epilogue2(std::integral_constant<int, BZ_ACT_PRELU>());
        break;
      case BZ_ACT_DICE:
        epilogue2(std::integral_constant<int, BZ_ACT_DICE>());
        break;
      case BZ_ACT_LEAKY_RELU:
        epilogue2(std::integral_constant<int, BZ_ACT_LEAKY_RELU>());
        break;
      case BZ_ACT_SIGMOID:
        epilogue2(std::integral_constant<int, BZ_ACT_SIGMOID>());
        break;
      default:
        epilogue2(std::integral_constant<int, BZ_ACT_NONE>());
        break;
    }
    if (ch.y2 != nullptr) {
      for (int q = lane; q < 32 * ch.n2; q += 64) {
        const int ml = q / ch.n2, n2 = q - ml * ch.n2;
        const int m = m0 + wave * 32 + ml;
        if (m < M) ((OutT*)ch.y2)[(int64_t)m * ch.ldy2 + n2] = ((const OutT*)(lout + ml * OPITCH2))[n2];
      }
    }
    // ---- skinny third layer: two lanes a row, 32 columns each, from the rounded staged tile
    if (ch.n3 > 0) {
      const int ml = lane >> 1, hx = lane & 1;
      const int m = m0 + wave * 32 + ml;
      float hacc[kSkinnyMaxN];
#pragma unroll
      for (int j = 0; j < kSkinnyMaxN; ++j) hacc[j] = 0.f;
      // the lane's 32 columns of its row in four 16-byte reads (columns from n2 up are zero, in the tile and in w3s);
      // the weights come from LDS, where the workgroup put them at the start: a load from memory per column here made
      // every wave wait 32 times
      float yv[32];
      const uint4* yrow = (const uint4*)(lout + ml * OPITCH2 + hx * 64);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint4 raw = yrow[q];
        const uint32_t r[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (DT == BZ_F16) {
            yv[8 * q + 2 * e] = __half2float(__ushort_as_half((unsigned short)(r[e] & 0xffffu)));
            yv[8 * q + 2 * e + 1] = __half2float(__ushort_as_half((unsigned short)(r[e] >> 16)));
          } else {  // bf16: the upper 16 bits of the fp32 pattern
            yv[8 * q + 2 * e] = __uint_as_float(r[e] << 16);
            yv[8 * q + 2 * e + 1] = __uint_as_float(r[e] & 0xffff0000u);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kSkinnyMaxN; ++j) {
        if (j < ch.n3) {
          const float4* wj = (const float4*)(w3s + j * 64 + hx * 32);
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const float4 w = wj[q];
            hacc[j] = fmaf(yv[4 * q], w.x, hacc[j]);
            hacc[j] = fmaf(yv[4 * q + 1], w.y, hacc[j]);
            hacc[j] = fmaf(yv[4 * q + 2], w.z, hacc[j]);
            hacc[j] = fmaf(yv[4 * q + 3], w.w, hacc[j]);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < kSkinnyMaxN; ++j) hacc[j] += __shfl_xor(hacc[j], 1, 64);
      if (hx == 0 && m < M) {
        float v[kSkinnyMaxN];
#pragma unroll
        for (int j = 0; j < kSkinnyMaxN; ++j) v[j] = (j < ch.n3) ? hacc[j] + (ch.bias3 ? ch.bias3[j] : 0.f) : 0.f;
        if (ch.act3 == BZ_ACT_SOFTMAX) {  // softmax_op.cc:21-78: subtract max, exp, sum in order, divide
          float mx = v[0];
#pragma unroll
          for (int j = 1; j < kSkinnyMaxN; ++j)
            if (j < ch.n3) mx = v[j] > mx ? v[j] : mx;
          float sum = 0.f;
#pragma unroll
          for (int j = 0; j < kSkinnyMaxN; ++j)
            if (j < ch.n3) {
              v[j] = expf(v[j] - mx);
              sum += v[j];
            }
#pragma unroll
          for (int j = 0; j < kSkinnyMaxN; ++j)
            if (j < ch.n3) v[j] = v[j] / sum;
        } else if (ch.act3 == BZ_ACT_SIGMOID) {
#pragma unroll
          for (int j = 0; j < kSkinnyMaxN; ++j) {
            const float t = expf(v[j]);
            v[j] = t / (1.f + t);
          }
        }
#pragma unroll
        for (int j = 0; j < kSkinnyMaxN; ++j) {
          if (j < ch.n3) {
            const int64_t at = (int64_t)m * ch.ldy3 + j;
            if (ch.y3_dtype == BZ_F32)
              store_out<float>((float*)ch.y3 + at, v[j]);
            else if (ch.y3_dtype == BZ_F16)
              store_out<__half>((__half*)ch.y3 + at, v[j]);
            else
              store_out<__hip_bfloat16>((__hip_bfloat16*)ch.y3 + at, v[j]);
          }
        }
      }
    }
  }
}

// A from pieces (bz_fc_desc.a_pieces).  BZ_ENOTSUP, with nothing launched, for anything outside the kernel's model.
template <int DT, typename OutT, int VEC, int NP, bool XY4, bool CHAIN>
int launch_pieces_tn(const bz_fc_desc& d, const bz::CewP& p, const Epilogue& ep, bool stage_y, int smem, const ChainArgs& ch,
                     hipStream_t st) {
  const int grid = (d.m + kPiecesBM - 1) / kPiecesBM;
  const int tn = (d.n + 31) / 32;
#define BZ_PIECES(TN)                                                                                                          \
  do {                                                                                                                         \
    static std::mutex mu;                                                                                                      \
    static bool raised[64] = {};                                                                                               \
    int dev = 0;                                                                                                               \
    BZ_HIP_OK(hipGetDevice(&dev));                                                                                             \
    {                                                                                                                          \
      std::lock_guard<std::mutex> lock(mu);                                                                                    \
      if (dev >= 0 && dev < 64 && !raised[dev]) {                                                                              \
        BZ_HIP_OK(hipFuncSetAttribute((const void*)bz_fc_pieces_kernel<DT, OutT, VEC, NP, TN, XY4, CHAIN>,                                 \
                                      hipFuncAttributeMaxDynamicSharedMemorySize,                                                  \
                                      pieces_lds(kPiecesKS * 16, 3, 4, true)));     \
        raised[dev] = true;                                                                                                    \
      }                                                                                                                        \
    }                                                                                                                          \
    hipLaunchKernelGGL((bz_fc_pieces_kernel<DT, OutT, VEC, NP, TN, XY4, CHAIN>), dim3(grid), dim3(256), smem, st, p, (const char*)d.w,     \
                       (OutT*)d.y, d.m, d.n, d.k, d.ldw, d.ldy, stage_y, ep, ch);                                              \
  } while (0)
  if (tn == 1)
    BZ_PIECES(1);
  else if (tn == 2)
    BZ_PIECES(2);
  else
    BZ_PIECES(3);
#undef BZ_PIECES
  BZ_LAUNCH_OK("bz_fc_pieces_kernel");
  return BZ_OK;
}

template <int DT, typename OutT>
int launch_pieces(const bz_fc_desc& d, const Epilogue& ep, hipStream_t st) {
  const bz_concat_ew_desc& c = *d.a_pieces;
  bz::CewP p;
  int vec = 1;
  const int rc = bz::cew_build(c, false, &p, &vec, "bz_fc_fused (a_pieces)");
  if (rc != BZ_OK) return rc;
  BZ_REQUIRE(c.dtype == d.in_dtype, "bz_fc_fused: a_pieces of dtype %d for a layer of dtype %d", c.dtype, d.in_dtype);
  BZ_REQUIRE(p.rows == d.m && p.col0[p.n] == d.k, "bz_fc_fused: a_pieces describe [%lld, %d], the layer takes [%d, %d]",
             (long long)p.rows, p.col0[p.n], d.m, d.k);
  const int kp = (d.k + 15) / 16 * 16;
  const int os = (int)sizeof(OutT);
  if (!bz::cew_uniform(p) || p.col0[1] / (vec == 4 ? 2 : vec) > 64 || p.n > 4 || kp / 16 > kPiecesKS || d.n > kPiecesMaxN || d.n <= kSkinnyMaxN ||
      d.m >= (1ll << 31) - kPiecesBM)
    return bz::fail(BZ_ENOTSUP, "bz_fc_fused: a_pieces take at most 4 pieces of one width without division, k <= %d, %d < n <= %d",
                    kPiecesKS * 16, kSkinnyMaxN, kPiecesMaxN);
  const int tn = (d.n + 31) / 32;
  const int pitch = pieces_pitch(d.k, tn, os, d.next != nullptr);
  // 16-byte stores of whole output rows when they are aligned for them (the outputs always go through LDS)
  const bool stage_y = d.y != nullptr && ((uintptr_t)d.y % 16 == 0) && ((d.ldy * os) % 16 == 0) && ((d.n * os) % 16 == 0);
  const int smem = pieces_lds(d.k, tn, os, d.next != nullptr);
  ChainArgs ch = {};
  const bool chain = d.next != nullptr;
  if (chain) {
    const bz_fc_next& x = *d.next;
    BZ_REQUIRE(x.w != nullptr && (uintptr_t)x.w % 16 == 0 && x.ldw >= d.n && (x.ldw * 2) % 16 == 0,
               "bz_fc_fused: next.w null or misaligned, or next.ldw=%lld below n=%d", (long long)x.ldw, d.n);
    BZ_REQUIRE(x.y == nullptr || x.ldy >= x.n, "bz_fc_fused: next.ldy=%lld below next.n=%d", (long long)x.ldy, x.n);
    BZ_REQUIRE(x.act != BZ_ACT_PRELU || (x.act_p0 && (x.act_size == 1 || x.act_size == x.n)), "bz_fc_fused: next: PRelu slope size %d", x.act_size);
    BZ_REQUIRE(x.act != BZ_ACT_DICE || (x.act_p0 && x.act_p1 && x.act_p2), "bz_fc_fused: next: Dice needs gamma, mean and var");
    BZ_REQUIRE(d.y != nullptr || x.y != nullptr || d.head_n > 0, "bz_fc_fused: a chain that stores nothing");
    if (sizeof(OutT) != 2 || x.n <= kSkinnyMaxN || x.n > 64 || x.act == BZ_ACT_SOFTMAX || x.act < BZ_ACT_NONE)
      return bz::fail(BZ_ENOTSUP, "bz_fc_fused: next takes a 2-byte layer of %d < n <= 64 columns without softmax", kSkinnyMaxN);
    ch.w2 = (const char*)x.w;
    ch.y2 = x.y;
    ch.ldw2 = x.ldw;
    ch.ldy2 = x.ldy;
    ch.n2 = x.n;
    ch.ep2.bias = x.bias;
    ch.ep2.bias_rows = x.bias ? 1 : 0;
    ch.ep2.p0 = x.act_p0;
    ch.ep2.p1 = x.act_p1;
    ch.ep2.p2 = x.act_p2;
    ch.ep2.act = x.act;
    ch.ep2.act_size = x.act_size;
    ch.ep2.dice_nosqrt = x.dice_nosqrt;
    ch.ep2.alpha = x.alpha;
    ch.ep2.beta = x.beta;
    ch.ep2.act_alpha = x.act_alpha;
    ch.ep2.split_n = 0;
    ch.ep2.split_stride = 0;
    if (d.head_n > 0) {
      BZ_REQUIRE(d.head_n <= kSkinnyMaxN && d.head_w && d.head_y && d.head_ldw >= x.n && d.head_ldy >= d.head_n,
                 "bz_fc_fused: head of %d outputs (1..%d), null head_w / head_y, or a leading dimension below its row", d.head_n, kSkinnyMaxN);
      BZ_REQUIRE(d.head_act == BZ_ACT_NONE || d.head_act == BZ_ACT_SIGMOID || d.head_act == BZ_ACT_SOFTMAX, "bz_fc_fused: head activation %d", d.head_act);
      BZ_REQUIRE(d.head_out_dtype == BZ_F32 || d.head_out_dtype == BZ_F16 || d.head_out_dtype == BZ_BF16, "bz_fc_fused: head out dtype %d", d.head_out_dtype);
      ch.w3 = (const char*)d.head_w;
      ch.bias3 = d.head_bias;
      ch.y3 = d.head_y;
      ch.ldw3 = d.head_ldw;
      ch.ldy3 = d.head_ldy;
      ch.n3 = d.head_n;
      ch.act3 = d.head_act;
      ch.y3_dtype = d.head_out_dtype;
    }
  } else if (d.y == nullptr) {
    return bz::fail(BZ_EINVAL, "bz_fc_fused: null y");
  }
  // (8 or 2 columns a lane; a width that allows 4 takes 2, an odd one is left to the two-launch form)
  // [x, y, x - y, x * y]: pieces 2 and 3 read exactly what pieces 0 and 1 copy
  auto same = [&](int k, bool second, int src) {
    const void* ptr = second ? p.y[k] : p.x[k];
    const int64_t* s = second ? p.ys[k] : p.xs[k];
    return ptr == p.x[src] && s[0] == p.xs[src][0] && s[1] == p.xs[src][1];
  };
  const bool xy4 = p.n == 4 && p.op[0] == BZ_EW_ASSIGN && p.op[1] == BZ_EW_ASSIGN && p.op[2] == BZ_EW_SUB && p.op[3] == BZ_EW_MUL &&
                   same(2, false, 0) && same(2, true, 1) && same(3, false, 0) && same(3, true, 1);
#define BZ_PIECES_V(V)                                                                                         \
  do {                                                                                                         \
    if constexpr (sizeof(OutT) == 2) {                                                                         \
      if (chain)                                                                                               \
        return xy4 ? launch_pieces_tn<DT, OutT, V, 4, true, true>(d, p, ep, stage_y, smem, ch, st)             \
                   : launch_pieces_tn<DT, OutT, V, 4, false, true>(d, p, ep, stage_y, smem, ch, st);           \
    }                                                                                                          \
    return xy4 ? launch_pieces_tn<DT, OutT, V, 4, true, false>(d, p, ep, stage_y, smem, ch, st)                \
               : launch_pieces_tn<DT, OutT, V, 4, false, false>(d, p, ep, stage_y, smem, ch, st);              \
  } while (0)
  if (vec == 8) BZ_PIECES_V(8);
  if (vec >= 2) BZ_PIECES_V(2);
#undef BZ_PIECES_V
  return bz::fail(BZ_ENOTSUP, "bz_fc_fused: a_pieces of odd width");
}

}  // namespace

int bz::fc_pieces_launch(const bz_fc_desc& d, const bz::fc::Epilogue& ep, hipStream_t st) {
  if (d.in_dtype == BZ_F16) {
    if (d.out_dtype == BZ_F32) return launch_pieces<BZ_F16, float>(d, ep, st);
    if (d.out_dtype == BZ_F16) return launch_pieces<BZ_F16, __half>(d, ep, st);
  } else if (d.in_dtype == BZ_BF16) {
    if (d.out_dtype == BZ_F32) return launch_pieces<BZ_BF16, float>(d, ep, st);
    if (d.out_dtype == BZ_BF16) return launch_pieces<BZ_BF16, __hip_bfloat16>(d, ep, st);
  }
  return bz::fail(BZ_ENOTSUP, "bz_fc_fused: a_pieces: in dtype %d, out dtype %d", d.in_dtype, d.out_dtype);
}
