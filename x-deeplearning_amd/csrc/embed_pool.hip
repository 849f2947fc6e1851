// embed_pool.hip -- Embedding gather + segmented pooling for gfx950 (MI355X).
//
// Replaces, for device-resident tables, the CPU loop of
// blaze/store/quick_embedding/quick_embedding_dict.cc:89-148 (QuickEmbeddingDict::Get)
// with its pooling processors blaze/store/quick_embedding/udf_processor.h:43-133 and
// the key lookup blaze/store/quick_embedding/hashtable.cc:45-64.
//
// Work decomposition.  The workload is memory bound: per id one random table row
// (36..256 bytes) plus 12 bytes of id/value.  A row is cut into 16-byte chunks
// (one 128-bit load); a *lane group* of `lpr` = pow2(chunks per row) lanes owns one
// (sample, slot) segment and walks its ids in order, so every output element is
// summed in exactly the reference's order (bit-identical fp32).  A 512-thread
// workgroup holds 512/lpr segments of consecutive samples of one slot.  One launch
// covers every slot of the operator; the linear workgroup id is remapped so that
// each of the 8 XCDs (each with its own L2) serves a contiguous range of slots and
// therefore caches the hot rows of only those tables.
//
// The kernel is latency bound before it is bandwidth bound (a batch-2048 launch moves
// ~36 MB), so the dependent chain is kept at: slot record -> segments -> ids -> rows.
//   * segments -> offsets is fused: a workgroup sums the counts before its first
//     sample and scans its own 512/lpr counts in LDS (no separate scan launch, no
//     offsets round trip);
//   * with equal work per slot the slot index is a division, not a search;
//   * the specialised ksum/kavg kernel walks a segment kBlockIds ids at a time: the lanes
//     of a group load disjoint ids/values (one coalesced read), resolve them to rows,
//     pass rows and values around with ds_bpermute, then issue the row loads before
//     the first add.  The block is short on purpose: the memory-level parallelism
//     comes from eight resident waves per SIMD, not from a deep unroll in each.
// A generic kernel covers kassign, mixed slot shapes, rows wider than 64 chunks and
// precomputed offsets.
//
// The memory system fetches 128-byte lines: a table whose rows sit inside lines
// (bz_table_pitch) costs one request per id, and an int8 row's scale lives in the
// row's own line.  Counts come from the caller and are not trusted: negative counts
// are zero and offsets stop at the slot's nnz.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <string.h>

#include <mutex>

#include "bz_common.h"

#include <limits.h>

namespace {

constexpr int kThreads = 512;  // measured at 128 / 256 / 512 / 1024 on config 2: 14.7 / 13.5 / 13.3 / 13.4 us per launch,
                               // 127 / 131 / 135 / 129 M samples/s with eight serving threads
constexpr int kUnroll = 4;  // rows in flight per lane group in the generic kernel (8 held 118 VGPRs and was no faster)

// ---------------------------------------------------------------------------------------------
// segments -> offsets (exclusive scan), one workgroup per array
// ---------------------------------------------------------------------------------------------
constexpr int kScanItems = 8;  // counts per thread per tile -> 4096 per workgroup tile
constexpr int kScanTile = kThreads * kScanItems;
// a thread's kScanItems consecutive entries sit kScanItems + 1 apart from the next thread's: its walk over them does
// not hit its neighbours' LDS banks
__device__ __forceinline__ int scan_slot(int i) { return i + i / kScanItems; }

__device__ __forceinline__ int64_t wave_incl_scan(int64_t v, int lane) {
#pragma unroll
  for (int d = 1; d < bz::kWave; d <<= 1) {
    int64_t t = __shfl_up(v, d, bz::kWave);
    if (lane >= d) v += t;
  }
  return v;
}

// Counts below zero are taken as zero and the running offset stops at `limit` (the length of the ids / values arrays),
// so no offset this scan produces points outside them.
// Global memory is read and written one element per lane, consecutive lanes consecutive elements; the thread-owns-a-run
// layout the scan wants exists only in LDS.  (With every thread loading and storing its own run directly, a wave's
// access touched 64 lines for 256 or 512 bytes: 200 slots x 8192 counts took 19.5 us.)
// Tiles [first_tile, first_tile + n_tiles) of the array (n_tiles < 0: all of them from first_tile on).  A workgroup that
// does not start at tile 0 first adds up the counts before its first tile - all those loads are independent, so a slot's
// scan split over several workgroups takes one tile's time, not the array's.
__device__ void scan_segments(const int32_t* __restrict__ seg, int64_t* __restrict__ off, int64_t n, int64_t limit,
                              int64_t first_tile = 0, int64_t n_tiles = -1) {
  __shared__ int64_t wave_tot[kThreads / bz::kWave];
  __shared__ int64_t carry_s;
  __shared__ int32_t cnt_s[kScanTile + kThreads];
  __shared__ int64_t off_s[kScanTile + kThreads];
  const int tid = threadIdx.x;
  const int lane = tid & (bz::kWave - 1);
  const int wave = tid / bz::kWave;
  const int64_t begin = first_tile * kScanTile;
  const int64_t end = (n_tiles < 0 || begin + n_tiles * kScanTile > n) ? n : begin + n_tiles * kScanTile;
  if (begin > n || (begin == n && n != 0)) return;  // nothing here; whoever scans the last tile writes off[n]
  {
    int64_t part = 0;
    for (int64_t i = tid; i < begin; i += kThreads) part += max(seg[i], 0);
    part = wave_incl_scan(part, lane);
    if (lane == bz::kWave - 1) wave_tot[wave] = part;
    __syncthreads();
    if (tid == 0) {
      int64_t c = 0;
      for (int w = 0; w < kThreads / bz::kWave; ++w) c += wave_tot[w];
      carry_s = c;
    }
    __syncthreads();
  }
  for (int64_t base = begin; base < end; base += kScanTile) {
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      const int j = k * kThreads + tid;
      cnt_s[scan_slot(j)] = (base + j < n) ? max(seg[base + j], 0) : 0;
    }
    __syncthreads();
    int32_t v[kScanItems];
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) v[k] = cnt_s[tid * (kScanItems + 1) + k];
    int64_t local = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) local += v[k];
    int64_t incl = wave_incl_scan(local, lane);
    if (lane == bz::kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    int64_t before = carry_s;
    for (int w = 0; w < wave; ++w) before += wave_tot[w];
    int64_t run = before + incl - local;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      off_s[tid * (kScanItems + 1) + k] = run < limit ? run : limit;
      run += v[k];
    }
    __syncthreads();
    if (tid == kThreads - 1) carry_s = run;  // last thread's running total = total so far
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      const int j = k * kThreads + tid;
      if (base + j < n) off[base + j] = off_s[scan_slot(j)];
    }
    __syncthreads();
  }
  if (tid == 0 && end == n) off[n] = carry_s < limit ? carry_s : limit;
}

__global__ __launch_bounds__(kThreads) void bz_scan_segments_kernel(const int32_t* __restrict__ seg,
                                                                    int64_t* __restrict__ off, int64_t n) {
  scan_segments(seg, off, n, INT64_MAX);
}

// ext_off != nullptr: slot i's offsets go to ext_off + i * ext_stride instead of slot.offsets (at most ext_stride - 1
// samples of a slot are scanned, so a record whose batch disagrees with the plan cannot write past its share)
// Grid (slots, parts): part p of a slot scans tiles p, or, for the last part, every tile from p on.
__global__ __launch_bounds__(kThreads) void bz_scan_segments_slots_kernel(const bz_embed_slot* __restrict__ slots,
                                                                          int64_t* __restrict__ ext_off, int64_t ext_stride) {
  const bz_embed_slot* s = &slots[blockIdx.x];
  const int64_t first = blockIdx.y, count = blockIdx.y + 1 == gridDim.y ? -1 : 1;
  if (ext_off != nullptr) {
    const int64_t n = s->batch < ext_stride - 1 ? s->batch : ext_stride - 1;
    scan_segments(s->segments, ext_off + (int64_t)blockIdx.x * ext_stride, n, s->nnz, first, count);
  } else {
    scan_segments(s->segments, s->offsets, s->batch, s->nnz, first, count);
  }
}

// parts a slot's scan is split into: one per tile of the largest batch, at most 8 (a part re-reads the counts before it)
inline int scan_parts(int64_t max_batch) {
  const int64_t tiles = (max_batch + kScanTile - 1) / kScanTile;
  return (int)(tiles < 1 ? 1 : (tiles > 8 ? 8 : tiles));
}

// ---------------------------------------------------------------------------------------------
// pooling
// ---------------------------------------------------------------------------------------------
template <int DT>
struct RowTraits;
template <>
struct RowTraits<BZ_F32> {
  static constexpr int kElems = 4;  // per 16-byte chunk
};
template <>
struct RowTraits<BZ_F16> {
  static constexpr int kElems = 8;
};
template <>
struct RowTraits<BZ_I8> {
  static constexpr int kElems = 16;
};

// widen one 16-byte chunk to fp32 weights.  int8: w = scale * (float)q, one rounding.
template <int DT>
__device__ __forceinline__ void widen(const uint4& raw, float scale, float (&w)[RowTraits<DT>::kElems]) {
  const uint32_t r[4] = {raw.x, raw.y, raw.z, raw.w};
  if constexpr (DT == BZ_F32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = __uint_as_float(r[i]);
  } else if constexpr (DT == BZ_F16) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      w[2 * i] = __half2float(__ushort_as_half((unsigned short)(r[i] & 0xffffu)));
      w[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(r[i] >> 16)));
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        int q = (int)(int8_t)((r[i] >> (8 * b)) & 0xffu);
        w[4 * i + b] = __fmul_rn(scale, (float)q);
      }
    }
  }
}

// scale of row r of an int8 table (a dense float array, or a field inside the table's rows)
__device__ __forceinline__ float load_scale(const bz_embed_slot& s, int64_t r) {
  return *(const float*)((const char*)s.row_scale + r * (int64_t)(s.scale_pitch != 0 ? s.scale_pitch : 4));
}

// acc += value * (the weights of one 16-byte chunk), the product rounded, then the sum rounded (udf_processor.h:66: never
// one fused operation).  For fp16 rows the widening rides in the multiply: fma(widen(h), value, +0) is the correctly
// rounded product (a product of -0 comes out as +0, which adds the same).  UNIT: the caller knows value == 1, so the
// product is the weight itself and acc + w is a single rounding, fma(widen(h), 1, acc) -- one instruction per element
// where the general form takes three.
template <int DT, bool UNIT>
__device__ __forceinline__ void accum_chunk(float (&acc)[RowTraits<DT>::kElems], const uint4& raw, float scale, float value) {
  const uint32_t r[4] = {raw.x, raw.y, raw.z, raw.w};
  if constexpr (DT == BZ_F32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float w = __uint_as_float(r[i]);
      acc[i] = __fadd_rn(acc[i], UNIT ? w : __fmul_rn(value, w));
    }
  } else if constexpr (DT == BZ_F16) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float w = __half2float(__ushort_as_half((unsigned short)((r[i / 2] >> (16 * (i & 1))) & 0xffffu)));
      // (UNIT: `value` is a 1.0 the compiler cannot see through, so that the widening and the add stay one
      // v_fma_mix_f32; with a literal 1 it splits them into a convert and an add)
      acc[i] = UNIT ? __builtin_fmaf(w, value, acc[i]) : __fadd_rn(acc[i], __builtin_fmaf(w, value, 0.0f));
    }
  } else {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float w = __fmul_rn(scale, (float)(int)(int8_t)((r[i / 4] >> (8 * (i & 3))) & 0xffu));
      acc[i] = __fadd_rn(acc[i], UNIT ? w : __fmul_rn(value, w));
    }
  }
}

// key / id -> table row, or -1 when absent.  Hash path = HashTable::Lookup
// (hashtable.cc:45-64): bucket record {offset:40, size:24}, (key,row) pairs.
__device__ __forceinline__ int64_t resolve_row(const bz_embed_slot& s, int64_t id) {
  if (s.hash_buckets != nullptr) {
    const uint64_t key = (uint64_t)id;
    const uint32_t h = (uint32_t)key;
    const uint64_t rec = s.hash_buckets[h % s.hash_bucket_size];
    const uint32_t cnt = (uint32_t)(rec >> 40);
    const uint64_t* p = s.hash_pairs + ((rec & 0xffffffffffull) >> 3);
    for (uint32_t i = 0; i < cnt; ++i) {
      if (p[2 * i] == key) {
        const uint64_t row = p[2 * i + 1];
        return row < (uint64_t)s.rows ? (int64_t)row : -1;
      }
    }
    return -1;
  }
  return (id >= 0 && id < s.rows) ? id : -1;
}

// fp32 -> bf16 bit pattern, round to nearest even; NaN stays a quiet NaN
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

// Store `nvalid` fp32 results as the slot's output dtype at element pointer `dst` using the widest store the address
// allows - the widest every active lane of the wave allows: lanes of one wave that picked different widths would run
// the paths one after the other (three kassign items sharing 108-byte rows start on 0, 4, 8 and 12 bytes mod 16, and
// their stores were 40 % of that kernel).
template <int N>
__device__ __forceinline__ void store_elems(void* dst_base, int64_t elem_off, const float (&v)[N], int nvalid,
                                            int out_dtype) {
  if (out_dtype == BZ_F32) {
    float* dst = (float*)dst_base + elem_off;
    if (__all(nvalid == N && (((uintptr_t)dst) & 15) == 0)) {
#pragma unroll
      for (int i = 0; i < N; i += 4) *(float4*)(dst + i) = make_float4(v[i], v[i + 1], v[i + 2], v[i + 3]);
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i)
        if (i < nvalid) dst[i] = v[i];
    }
  } else {  // BZ_F16 / BZ_BF16, round to nearest even
    __half* dst = (__half*)dst_base + elem_off;  // (a 16-bit slot; bf16 bits travel through the same stores)
    uint32_t pk[N / 2];
#pragma unroll
    for (int i = 0; i < N / 2; ++i) {
      uint32_t lo, hi;
      if (out_dtype == BZ_F16) {
        lo = __half_as_ushort(__float2half_rn(v[2 * i]));
        hi = __half_as_ushort(__float2half_rn(v[2 * i + 1]));
      } else {
        lo = f32_to_bf16_bits(v[2 * i]);
        hi = f32_to_bf16_bits(v[2 * i + 1]);
      }
      pk[i] = lo | (hi << 16);
    }
    const uintptr_t a = (uintptr_t)dst;
    const bool full = nvalid == N;
    if (N >= 8 && __all(full && (a & 15) == 0)) {
#pragma unroll
      for (int i = 0; i + 4 <= N / 2; i += 4) *(uint4*)((uint32_t*)dst + i) = make_uint4(pk[i], pk[i + 1], pk[i + 2], pk[i + 3]);
    } else if (__all(full && (a & 7) == 0)) {
#pragma unroll
      for (int i = 0; i < N / 2; i += 2) *(uint2*)((uint32_t*)dst + i) = make_uint2(pk[i], pk[i + 1]);
    } else if (__all((a & 3) == 0)) {
      if (__all(full)) {
#pragma unroll
        for (int i = 0; i < N / 2; ++i) ((uint32_t*)dst)[i] = pk[i];
      } else {
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
          if (2 * i + 1 < nvalid)
            ((uint32_t*)dst)[i] = pk[i];
          else if (2 * i < nvalid)
            dst[2 * i] = __ushort_as_half((unsigned short)(pk[i] & 0xffffu));
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i)
        if (i < nvalid) dst[i] = __ushort_as_half((unsigned short)((pk[i / 2] >> (16 * (i & 1))) & 0xffffu));
    }
  }
}

// elements between the output positions of a kassign sample
__device__ __forceinline__ int assign_pitch(const bz_embed_slot& s) { return s.assign_pitch != 0 ? s.assign_pitch : s.dim; }

// ksum / kavg for one lane: chunk `c` of the segment [start, end) of sample b.
template <int DT>
__device__ __forceinline__ void pool_sum(const bz_embed_slot& s, int64_t start, int64_t end, int c, int64_t b) {
  constexpr int CE = RowTraits<DT>::kElems;
  float acc[CE];
#pragma unroll
  for (int i = 0; i < CE; ++i) acc[i] = 0.f;
  const char* table = (const char*)s.table + (int64_t)c * 16;
  for (int64_t j = start; j < end; j += kUnroll) {
    const int n = (int)((end - j) < kUnroll ? (end - j) : kUnroll);
    int64_t row[kUnroll];
    float val[kUnroll];
    uint4 raw[kUnroll];
    float sc[kUnroll];
    // clamp instead of branching: the tail repeats the last id (cache hit), results ignored
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t jj = (u < n) ? j + u : end - 1;
      row[u] = resolve_row(s, s.ids[jj]);
      val[u] = s.values[jj];
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t r = row[u] < 0 ? 0 : row[u];
      raw[u] = *(const uint4*)(table + r * (int64_t)s.pitch);
      sc[u] = (DT == BZ_I8) ? load_scale(s, r) : 1.f;
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (u < n && row[u] >= 0) {
        float w[CE];
        widen<DT>(raw[u], sc[u], w);
        // out = out + value * w: two roundings, never an FMA (udf_processor.h:66)
#pragma unroll
        for (int i = 0; i < CE; ++i) acc[i] = __fadd_rn(acc[i], __fmul_rn(val[u], w[i]));
      }
    }
  }
  if (s.udf == BZ_AVG) {
    const int64_t num = end - start;
    if (num != 0) {
      const float inv = (float)(1.0 / (double)num);  // ValueType(1.0 / size), udf_processor.h:88
#pragma unroll
      for (int i = 0; i < CE; ++i) acc[i] = __fmul_rn(acc[i], inv);
    }
  }
  const int e0 = c * CE;
  const int nvalid = (s.dim - e0) < CE ? (s.dim - e0) : CE;
  store_elems<CE>(s.out, b * s.out_stride + e0, acc, nvalid, s.out_dtype);
}

// kassign: position p of the output holds id j = p (in order) or num - trunc + p (reverse);
// positions without an id, and ids absent from the table, are zero (udf_processor.h:103-131).
// One call fills chunk c of positions p0 .. p0 + kAssignRun - 1 of sample b: the positions of a sample are independent
// of each other, so the kernel spreads them over lane groups instead of walking them one dependent load after the
// other, and a group keeps kAssignRun of them in flight (their ids are neighbours in memory): with one position a
// group, DIN's 50-position histories were bounded by the four dependent trips to memory each group makes for a
// single 36-byte row.
constexpr int kAssignRun = 4;
__host__ __device__ inline int64_t items_per_sample(const bz_embed_slot& s) {
  return s.udf == BZ_ASSIGN ? (s.trunc_num + kAssignRun - 1) / kAssignRun : 1;
}

template <int DT>
__device__ __forceinline__ void pool_assign(const bz_embed_slot& s, int64_t start, int64_t end, int c, int64_t b, int p0) {
  constexpr int CE = RowTraits<DT>::kElems;
  constexpr int R = kAssignRun;
  const int64_t num = end - start;
  const int e0 = c * CE;
  const int nvalid = (s.dim - e0) < CE ? (s.dim - e0) : CE;
  const char* table = (const char*)s.table + (int64_t)c * 16;
  const int64_t shift = (s.trunc_dir == BZ_ORDER) ? 0 : num - (int64_t)s.trunc_num;
  // no branch round the loads: a position without an id reads id 0 of the slot (there is one whenever any position
  // has an id) and row 0 of the table, and the result is dropped
  bool live[R];
  int64_t row[R];
  float val[R];
  uint4 raw[R];
  float sc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t j = shift + p0 + r;
    live[r] = p0 + r < s.trunc_num && j >= 0 && j < num;
    const int64_t at = live[r] ? start + j : 0;
    row[r] = -1;
    val[r] = 0.f;
    if (num > 0) {  // (uniform over the group's positions: they belong to one sample)
      row[r] = resolve_row(s, s.ids[at]);
      val[r] = s.values[at];
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    live[r] = live[r] && row[r] >= 0;
    const int64_t rr = live[r] ? row[r] : 0;
    raw[r] = *(const uint4*)(table + rr * (int64_t)s.pitch);
    sc[r] = (DT == BZ_I8) ? load_scale(s, rr) : 1.f;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (p0 + r < s.trunc_num) {
      float out[CE];
      float w[CE];
      widen<DT>(raw[r], sc[r], w);
#pragma unroll
      for (int i = 0; i < CE; ++i) out[i] = live[r] ? __fmul_rn(val[r], w[i]) : 0.f;
      store_elems<CE>(s.out, b * s.out_stride + (int64_t)(p0 + r) * assign_pitch(s) + e0, out, nvalid, s.out_dtype);
    }
  }
}

// zero fill of one item's columns (unknown table name: quick_embedding_dict.cc:95 leaves the
// memset block untouched)
__device__ __forceinline__ void pool_zero(const bz_embed_slot& s, int64_t b, int p0, int l, int lpr) {
  const int run = s.udf == BZ_ASSIGN ? kAssignRun : 1;  // p0 = 0 unless kassign
  for (int p = p0; p < p0 + run && (p == 0 || p < s.trunc_num); ++p) {
    const int64_t base = b * s.out_stride + (int64_t)p * assign_pitch(s);
    for (int e = l; e < s.dim; e += lpr) {
      if (s.out_dtype == BZ_F32)
        ((float*)s.out)[base + e] = 0.f;
      else
        ((__half*)s.out)[base + e] = __ushort_as_half(0);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// offsets of one workgroup's samples, derived from the segment counts
// ---------------------------------------------------------------------------------------------
// s_off[0..groups] <- exclusive offsets of samples b0 .. b0+groups (clipped to batch).
// Every thread of the workgroup calls it; ends with a barrier.
// `offsets`: the slot's precomputed offsets (slot.offsets, or its share of a buffer the launch brings), or nullptr.
__device__ __forceinline__ void stage_offsets(const bz_embed_slot& s, const int64_t* __restrict__ offsets, int64_t b0,
                                              int groups, int64_t* s_off, int64_t* s_part) {
  const int tid = threadIdx.x;
  const int lane = tid & (bz::kWave - 1), wave = tid / bz::kWave;
  if (offsets != nullptr) {
    for (int t = tid; t <= groups; t += kThreads)
      if (b0 + t <= s.batch) {
        const int64_t o = offsets[b0 + t];
        s_off[t] = o < 0 ? 0 : (o < s.nnz ? o : s.nnz);  // caller-made offsets get the same bounds as the scan's
      }
    __syncthreads();
    return;
  }
  // base = sum of the counts before b0 (independent coalesced reads), local = this thread's sample
  // (8 loads in flight per thread: a rolled loop would wait for each load before issuing the next)
  // this thread's own count is requested first so that it travels with the counts summed below
  // (a negative count is taken as 0 and the offsets below stop at nnz: see bz_embed_slot.nnz)
  const int64_t mine = (tid < groups && b0 + tid < s.batch) ? (int64_t)max(s.segments[b0 + tid], 0) : 0;
  int64_t part = 0;
  for (int64_t i0 = 0; i0 < b0; i0 += 8 * kThreads) {
    int32_t c[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int64_t i = i0 + k * kThreads + tid;
      c[k] = i < b0 ? max(s.segments[i], 0) : 0;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) part += c[k];
  }
  int64_t base = part;
#pragma unroll
  for (int d = bz::kWave / 2; d > 0; d >>= 1) base += __shfl_xor(base, d, bz::kWave);
  const int64_t incl = wave_incl_scan(mine, lane);
  if (lane == bz::kWave - 1) {
    s_part[wave] = base;
    s_part[kThreads / bz::kWave + wave] = incl;
  }
  __syncthreads();
  int64_t before = 0;
#pragma unroll
  for (int w = 0; w < kThreads / bz::kWave; ++w) {
    before += s_part[w];
    if (w < wave) before += s_part[kThreads / bz::kWave + w];
  }
  if (tid < groups) s_off[tid + 1] = (before + incl) < s.nnz ? (before + incl) : s.nnz;
  if (tid == 0) s_off[0] = before < s.nnz ? before : s.nnz;
  __syncthreads();
}

// ---------------------------------------------------------------------------------------------
// the same for the specialised kernel, where lane group g of the workgroup owns sample b0 + g: every lane ends up with
// its own segment [start, end) in registers
// ---------------------------------------------------------------------------------------------
// All sums saturate at cap = nnz (< 2^31 here; larger arrays take stage_offsets): every term is >= 0, so
// min(a + b, cap) is associative and gives the clamped offsets whatever the order of the additions, in 32 bits.
__device__ __forceinline__ uint32_t sat_add(uint32_t a, uint32_t b, uint32_t cap) {
  const uint32_t t = a + b;  // a, b <= cap < 2^31: no wrap
  return t < cap ? t : cap;
}

// Inclusive scan over the 64 lanes with data-parallel primitives (row_shr within rows of 16 lanes, then lane 15 and
// lane 31 handed on to the following rows): a dozen VALU instructions, where the same scan through ds_bpermute
// (__shfl_up) is six dependent trips to LDS per 32 bits.
__device__ __forceinline__ uint32_t wave_scan_sat(uint32_t v, uint32_t cap) {
  v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false), cap);  // row_shr:1
  v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false), cap);  // row_shr:2
  v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false), cap);  // row_shr:4
  v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false), cap);  // row_shr:8
  v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false), cap);  // row_bcast:15 -> rows 1, 3
  v = sat_add(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false), cap);  // row_bcast:31 -> rows 2, 3
  return v;
}

// start / end of sample b = b0 + g for every lane of lane group g (LPR lanes, g = tid / LPR); lanes of samples beyond
// the batch get an empty segment.  Every thread of the workgroup calls it; one barrier.
template <int LPR>
__device__ __forceinline__ void own_segment(const bz_embed_slot& s, int64_t b0, uint32_t* s_tot, int64_t* start, int64_t* end) {
  constexpr int WAVES = kThreads / bz::kWave;
  const int tid = threadIdx.x;
  const int lane = tid & (bz::kWave - 1), wave = tid / bz::kWave;
  const int g = tid / LPR, l = tid % LPR;
  const int64_t b = b0 + g;
  const uint32_t cap = (uint32_t)s.nnz;
  // this group's own count first (all its lanes ask for the same word), then the counts before b0, 8 loads in flight a
  // thread: everything is requested before anything is used
  const int32_t own = b < s.batch ? s.segments[b] : 0;
  // (b0 is below 2^31: batch is an int32.  A workgroup near the head of its slot has few counts before it: the rounds
  // of 8 loads stop, for the whole workgroup, where b0 ends)
  const uint32_t nb = (uint32_t)b0;
  uint64_t part = 0;
  for (uint32_t i0 = 0; i0 < nb; i0 += 8 * kThreads) {
    int32_t c[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const uint32_t i = i0 + k * kThreads + tid;
      c[k] = 0;
      if (i0 + k * kThreads < nb) c[k] = s.segments[i < nb ? i : nb - 1];  // (uniform test; a lane past b0 reads the last count, masked below)
      if (i >= nb) c[k] = 0;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) part += (uint32_t)max(c[k], 0);
  }
  const uint32_t mine = min((uint32_t)max(own, 0), cap);
  // the group's count sits in its last lane: after the scan that lane holds the inclusive sum and the group's other
  // lanes the exclusive one (they add nothing)
  const uint32_t scan = wave_scan_sat(l == LPR - 1 ? mine : 0u, cap);
  const uint32_t before_b0 = wave_scan_sat((uint32_t)(part < cap ? part : cap), cap);
  if (lane == bz::kWave - 1) {
    s_tot[wave] = before_b0;
    s_tot[WAVES + wave] = scan;
  }
  __syncthreads();
  // what lies before this wave: all the waves' sums of earlier counts and the totals of the waves before it -- entry
  // WAVES - 1 + wave of the inclusive (saturating) scan over the 2 * WAVES values, done in one row of 16 lanes
  static_assert(2 * WAVES <= 16, "the waves' totals are scanned within one row of lanes");
  uint32_t t = (lane & 15) < 2 * WAVES ? s_tot[lane & 15] : 0u;
  t = sat_add(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x111, 0xf, 0xf, false), cap);  // row_shr:1
  t = sat_add(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x112, 0xf, 0xf, false), cap);  // row_shr:2
  t = sat_add(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x114, 0xf, 0xf, false), cap);  // row_shr:4
  t = sat_add(t, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)t, 0x118, 0xf, 0xf, false), cap);  // row_shr:8
  const uint32_t before = (uint32_t)__builtin_amdgcn_readlane((int)t, WAVES - 1 + wave);
  const uint32_t x = sat_add(before, scan, cap);
  if constexpr (LPR == 1) {
    uint32_t excl = (uint32_t)__shfl_up((int)scan, 1, bz::kWave);
    if (lane == 0) excl = 0;
    *start = (int64_t)sat_add(before, excl, cap);
    *end = (int64_t)x;
  } else {
    const int gbase = lane - l;
    *start = (int64_t)(uint32_t)__shfl((int)x, gbase, bz::kWave);
    *end = (int64_t)(uint32_t)__shfl((int)x, gbase + LPR - 1, bz::kWave);
  }
}

// ---------------------------------------------------------------------------------------------
// specialised ksum / kavg kernel: every slot has table dtype DT and LPR lanes per row
// ---------------------------------------------------------------------------------------------
constexpr int kBlockIds = 4;  // ids walked per step (measured at 2, 4, 8, 16: 4 is best or equal on segments of 1-4, 8 and 20 ids)
// Above this many bytes of repeated count reads a separate scan launch (about 15 us with its gap) is cheaper than the
// fused one: config 5 (200 slots x 256 workgroups x batch 8192: 840 MB) pools in 155 + 16 us with offsets against
// 261 us fused; config 4 (26 MB) and config 2 (3 MB) stay fused.
constexpr int64_t kScanFirstBytes = 128ll << 20;

// Slot records handed over as kernel arguments: a workgroup then has its record after the one scalar load every
// kernel starts with, instead of after a second trip to memory for slots[si] (measured on config 2: 1050 cycles from
// the start of a wave to its kernel arguments, 2200 more to the record).
struct SlotPack {
  bz_embed_slot s[BZ_EMBED_ARG_SLOTS];
};
static_assert(sizeof(SlotPack) + 4 * 16 + 32 <= 4096, "the records and the other arguments fit the 4 KB kernel-argument segment");

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr uint32_t kBeyondTable = 0xF0000000u;  // a byte offset no table read through a buffer resource reaches

template <int DT, int LPR>
__device__ __forceinline__ void pool_samples(const bz_embed_slot& s, int64_t b0, const int64_t* __restrict__ offsets) {
  constexpr int CE = RowTraits<DT>::kElems;
  constexpr int GROUPS = kThreads / LPR;
  constexpr int SRC = LPR < kBlockIds ? LPR : kBlockIds;  // lanes of a group that fetch ids
  constexpr int KPL = kBlockIds / SRC;                    // ids fetched per such lane
  __shared__ int64_t s_off[GROUPS + 1];
  __shared__ int64_t s_part[2 * kThreads / bz::kWave];
  const int tid = threadIdx.x;
  const int g = tid / LPR, l = tid % LPR;
  int64_t start, end;
  if (offsets == nullptr && s.nnz < (1ll << 31)) {
    own_segment<LPR>(s, b0, (uint32_t*)s_part, &start, &end);
  } else if (offsets != nullptr) {
    // every lane of a group asks for its sample's two offsets itself (one address a group): nothing goes through LDS
    // and no wave waits for another's.  Caller-made offsets get the same bounds as the scan's.
    const int64_t bb = b0 + g < s.batch ? b0 + g : s.batch - 1;  // (lanes past the batch return below)
    const int64_t o0 = offsets[bb], o1 = offsets[bb + 1];
    start = o0 < 0 ? 0 : (o0 < s.nnz ? o0 : s.nnz);
    end = o1 < 0 ? 0 : (o1 < s.nnz ? o1 : s.nnz);
  } else {
    stage_offsets(s, offsets, b0, GROUPS, s_off, s_part);
    start = s_off[g];
    end = s_off[g + 1];
  }
  const int64_t b = b0 + g;
  if (b >= s.batch) return;
  const int nchunks = (s.dim + CE - 1) / CE;
  const bool has_chunk = l < nchunks;
  const int gbase = (tid & (bz::kWave - 1)) - l;  // first lane of this group within the wave
  const char* table = (const char*)s.table + (int64_t)l * 16;
  float acc[CE];
#pragma unroll
  for (int i = 0; i < CE; ++i) acc[i] = 0.f;
  float one = 1.f;  // (opaque: see accum_chunk)
  asm volatile("" : "+v"(one));
  // fp32 / fp16 tables of up to 2^24 rows and 3.75 GB are read through a buffer resource: the hardware checks every
  // access against the table's size and returns zeros beyond it, which is what a missing row contributes.  (Measured:
  // config 2's launch 11.9 -> 11.7 us.  Not for int8 tables: with the rows and their scales through buffer resources
  // config 4's launch took 97-110 us against 90-92 with plain loads under a branch.)
  const bool by_buffer = DT != BZ_I8 && s.rows <= (1ll << 24) && (uint64_t)s.rows * (uint64_t)s.pitch <= (uint64_t)kBeyondTable &&
                         s.pitch < (1 << 24);
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)s.table, 0, by_buffer ? (int)(uint32_t)(s.rows * (int64_t)s.pitch) : 0, 0x00020000);
  // each fetching lane takes ids j + k*SRC + l: one coalesced read per k for the whole group.  The
  // next step's ids are requested before this step's rows, so the two round trips overlap.
  int64_t id_next[KPL];  // raw ids: resolved to rows only when consumed, so the wait lands after the row loads
  float val_next[KPL];
  auto fetch_ids = [&](int64_t j) {
    const int cnt = (int)((end - j) < kBlockIds ? (end - j) : kBlockIds);
#pragma unroll
    for (int k = 0; k < KPL; ++k) {
      const int idx = k * SRC + l;
      id_next[k] = -1;  // resolves to "absent" on both the direct and (as a never-stored key) the hash path
      val_next[k] = 0.f;
      if (l < SRC && idx < cnt) {
        id_next[k] = s.ids[j + idx];
        val_next[k] = s.values[j + idx];
      }
    }
  };
  if (start < end) fetch_ids(start);
  for (int64_t j = start; j < end; j += kBlockIds) {
    const int cnt = (int)((end - j) < kBlockIds ? (end - j) : kBlockIds);
    int row_own[KPL];
    float val_own[KPL];
#pragma unroll
    for (int k = 0; k < KPL; ++k) {
      row_own[k] = (l < SRC && k * SRC + l < cnt) ? (int)resolve_row(s, id_next[k]) : -1;
      // an id without a row contributes a zero row (times the value 1): adding +0 leaves the running sum as it is
      // (the sum starts at +0 and so is never -0), which lets the accumulation below run without the row numbers
      val_own[k] = row_own[k] >= 0 ? val_next[k] : 1.f;
    }
    if (j + kBlockIds < end) fetch_ids(j + kBlockIds);
    // ids that carry no weight (value 1, the usual case) take the one-rounding form, when that holds for every lane of
    // the wave: decided on the lanes' own values, before anything is handed round, so that the values need not be
    bool unit_own = true;
#pragma unroll
    for (int k = 0; k < KPL; ++k) unit_own &= val_own[k] == 1.f;
    const bool unit = __all(unit_own);
    int row[kBlockIds];
    float val[kBlockIds];
    uint4 raw[kBlockIds];
    float sc[kBlockIds];
#pragma unroll
    for (int u = 0; u < kBlockIds; ++u) row[u] = __shfl(row_own[u / SRC], gbase + (u % SRC), bz::kWave);
    if (!unit) {
#pragma unroll
      for (int u = 0; u < kBlockIds; ++u) val[u] = __shfl(val_own[u / SRC], gbase + (u % SRC), bz::kWave);
    }
    if (by_buffer) {
      // no branch round a load, no zero fill, one multiply-add per address: a row that is not there (row[u] is -1 beyond
      // cnt and for ids without a row) is asked for beyond the table's end and comes back as zeros
#pragma unroll
      for (int u = 0; u < kBlockIds; ++u) {
        const uint32_t off = (has_chunk && row[u] >= 0) ? __umul24((uint32_t)row[u], (uint32_t)s.pitch) + (uint32_t)l * 16u : kBeyondTable;
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)off, 0, 0);
        raw[u] = make_uint4(v.x, v.y, v.z, v.w);
        sc[u] = 1.f;
      }
    } else {
#pragma unroll
      for (int u = 0; u < kBlockIds; ++u) {
        raw[u] = make_uint4(0, 0, 0, 0);
        sc[u] = 1.f;
        if (has_chunk && row[u] >= 0) {
          raw[u] = *(const uint4*)(table + (int64_t)row[u] * s.pitch);
          if (DT == BZ_I8) sc[u] = load_scale(s, row[u]);
        }
      }
    }
    if (unit) {
#pragma unroll
      for (int u = 0; u < kBlockIds; ++u) accum_chunk<DT, true>(acc, raw[u], sc[u], one);
    } else {
#pragma unroll
      for (int u = 0; u < kBlockIds; ++u) accum_chunk<DT, false>(acc, raw[u], sc[u], val[u]);
    }
  }
  if (s.udf == BZ_AVG) {
    const int64_t num = end - start;
    if (num != 0) {
      const float inv = (float)(1.0 / (double)num);  // ValueType(1.0 / size), udf_processor.h:88
#pragma unroll
      for (int i = 0; i < CE; ++i) acc[i] = __fmul_rn(acc[i], inv);
    }
  }
  if (has_chunk) {
    const int e0 = l * CE;
    const int nvalid = (s.dim - e0) < CE ? (s.dim - e0) : CE;
    store_elems<CE>(s.out, b * s.out_stride + e0, acc, nvalid, s.out_dtype);
  }
}

template <int DT, int LPR>
__global__ __launch_bounds__(kThreads) void bz_embed_pool_kernel(const bz_embed_slot* __restrict__ slots, int n_slots,
                                                                 int total_wg, int wg_per_xcd, int wg_per_slot,
                                                                 const int64_t* __restrict__ ext_off, int64_t ext_stride) {
  constexpr int GROUPS = kThreads / LPR;
  const int v = (int)(blockIdx.x % bz::kNumXcd) * wg_per_xcd + (int)(blockIdx.x / bz::kNumXcd);
  if (v >= total_wg) return;
  const int si = v / wg_per_slot;
  const bz_embed_slot s = slots[si];
  const int64_t b0 = (int64_t)(v - si * wg_per_slot) * GROUPS;
  pool_samples<DT, LPR>(s, b0, ext_off != nullptr ? ext_off + (int64_t)si * ext_stride : s.offsets);
}

template <int DT, int LPR>
__global__ __launch_bounds__(kThreads) void bz_embed_pool_args_kernel(const SlotPack pack, int total_wg, int wg_per_xcd,
                                                                      int wg_per_slot) {
  constexpr int GROUPS = kThreads / LPR;
  const int v = (int)(blockIdx.x % bz::kNumXcd) * wg_per_xcd + (int)(blockIdx.x / bz::kNumXcd);
  if (v >= total_wg) return;
  const int si = v / wg_per_slot;
  const bz_embed_slot s = pack.s[si];
  const int64_t b0 = (int64_t)(v - si * wg_per_slot) * GROUPS;
  pool_samples<DT, LPR>(s, b0, s.offsets);
}

__device__ __forceinline__ int chunk_elems(int dt) { return dt == BZ_F32 ? 4 : (dt == BZ_F16 ? 8 : 16); }

// one workgroup of the generic path: workgroup v of the launch, owned by slot s
__device__ __forceinline__ void pool_generic(const bz_embed_slot& s, int v, const int64_t* __restrict__ offsets, int64_t* s_off,
                                             int64_t* s_part) {
  const int ce = chunk_elems(s.table_dtype);
  const int nchunks = (s.dim + ce - 1) / ce;
  // lpr, a power of two: shifts, not divisions (a 64-bit division is some 150 instructions, and this kernel's threads
  // each do little else than one or four row gathers)
  int lpr_log = 0;
  while ((1 << lpr_log) < nchunks && (1 << lpr_log) < bz::kWave) ++lpr_log;
  const int lpr = 1 << lpr_log;
  const int groups = kThreads >> lpr_log;
  const int tid = threadIdx.x;
  const int g = tid >> lpr_log;
  const int l = tid - (g << lpr_log);
  // a lane group owns one item: a sample (ksum / kavg) or kAssignRun output positions of a sample (kassign)
  const int64_t per = items_per_sample(s);
  const int64_t n_items = (int64_t)s.batch * per;
  const int64_t i0 = (int64_t)(v - s.wg_begin) * groups;
  int64_t i_last = i0 + groups - 1;
  if (i_last >= n_items) i_last = n_items - 1;
  // item -> sample: no division for pooled slots (per == 1), a 32-bit one while the item count allows it
  auto sample_of = [&](int64_t item) -> int64_t {
    if (per == 1) return item;
    if (n_items < (1ll << 31)) return (int64_t)((uint32_t)item / (uint32_t)per);
    return item / per;
  };
  const int64_t b_first = sample_of(i0);
  const int n_samples = (int)(sample_of(i_last) - b_first) + 1;  // <= groups
  stage_offsets(s, offsets, b_first, n_samples, s_off, s_part);
  const int64_t item = i0 + g;
  if (item >= n_items) return;
  const int64_t b = sample_of(item);
  const int p = (int)(item - b * per) * (s.udf == BZ_ASSIGN ? kAssignRun : 1);
  if (s.table == nullptr) {
    pool_zero(s, b, p, l, lpr);
    return;
  }
  const int64_t start = s_off[b - b_first], end = s_off[b - b_first + 1];
  for (int c = l; c < nchunks; c += lpr) {
    if (s.udf == BZ_ASSIGN) {
      switch (s.table_dtype) {
        case BZ_F32: pool_assign<BZ_F32>(s, start, end, c, b, p); break;
        case BZ_F16: pool_assign<BZ_F16>(s, start, end, c, b, p); break;
        default: pool_assign<BZ_I8>(s, start, end, c, b, p); break;
      }
    } else {
      switch (s.table_dtype) {
        case BZ_F32: pool_sum<BZ_F32>(s, start, end, c, b); break;
        case BZ_F16: pool_sum<BZ_F16>(s, start, end, c, b); break;
        default: pool_sum<BZ_I8>(s, start, end, c, b); break;
      }
    }
  }
}

__global__ __launch_bounds__(kThreads) void bz_embed_pool_generic_kernel(const bz_embed_slot* __restrict__ slots,
                                                                         int n_slots, int total_wg, int wg_per_xcd,
                                                                         int wg_per_slot, const int64_t* __restrict__ ext_off,
                                                                         int64_t ext_stride) {
  __shared__ int64_t s_off[kThreads + 1];
  __shared__ int64_t s_part[2 * kThreads / bz::kWave];
  // XCD-aware order: hardware deals consecutive workgroup ids round robin over the 8 XCDs; give
  // each XCD a contiguous range of the logical workgroup space (= a contiguous range of slots).
  const int v = (int)(blockIdx.x % bz::kNumXcd) * wg_per_xcd + (int)(blockIdx.x / bz::kNumXcd);
  if (v >= total_wg) return;
  // The slot that owns workgroup v = the last one with wg_begin <= v (empty slots share a begin with their successor).
  // Begins never decrease, so that is (number of begins <= v) - 1: every wave counts them 64 at a time with one load
  // and a ballot - one trip to memory where a binary search would make log2(n_slots) dependent ones.
  int lo;
  if (wg_per_slot > 0) {
    lo = v / wg_per_slot;
  } else {
    const int lane = threadIdx.x & (bz::kWave - 1);
    int cnt = 0;
    for (int base = 0; base < n_slots; base += bz::kWave) {
      const int i = base + lane;
      const bool le = i < n_slots && slots[i].wg_begin <= v;
      cnt += __popcll(__ballot(le));
    }
    lo = __builtin_amdgcn_readfirstlane(cnt - 1);
  }
  // slots with wg_count == 0 sharing this begin come before the one that owns the workgroup
  const bz_embed_slot s = slots[lo];
  pool_generic(s, v, ext_off != nullptr ? ext_off + (int64_t)lo * ext_stride : s.offsets, s_off, s_part);
}

// the same with the slot records as kernel arguments: no trip for the begins, none for the record
struct SlotBegins {
  int b[16];  // wg_begin of every slot, INT_MAX behind the last: read with one wide scalar load
};

__global__ __launch_bounds__(kThreads) void bz_embed_pool_generic_args_kernel(const SlotPack pack, const SlotBegins begins,
                                                                              int total_wg, int wg_per_xcd, int wg_per_slot) {
  __shared__ int64_t s_off[kThreads + 1];
  __shared__ int64_t s_part[2 * kThreads / bz::kWave];
  const int v = (int)(blockIdx.x % bz::kNumXcd) * wg_per_xcd + (int)(blockIdx.x / bz::kNumXcd);
  if (v >= total_wg) return;
  int lo;
  if (wg_per_slot > 0) {
    lo = v / wg_per_slot;
  } else {
    lo = -1;
#pragma unroll
    for (int i = 0; i < 16; ++i) lo += begins.b[i] <= v ? 1 : 0;  // uniform: scalar compares
  }
  const bz_embed_slot s = pack.s[lo];
  pool_generic(s, v, s.offsets, s_off, s_part);
}

int groups_per_wg(const bz_embed_slot& s) {
  const int ce = s.table_dtype == BZ_F32 ? 4 : (s.table_dtype == BZ_F16 ? 8 : 16);
  const int nchunks = (s.dim + ce - 1) / ce;
  int lpr = 1;
  while (lpr < nchunks && lpr < bz::kWave) lpr <<= 1;
  return kThreads / lpr;
}

// ---------------------------------------------------------------------------------------------
// scratch of the entry point that allocates nothing: every slot's offsets, inside the library's own device image
// ---------------------------------------------------------------------------------------------
constexpr int64_t kStaticScratchEntries = BZ_EMBED_STATIC_SCRATCH_BYTES / sizeof(int64_t);
static __device__ __align__(256) int64_t scratch[kStaticScratchEntries];

// Device address of `scratch` on the current device.  In host code the array's name is only a handle: the address
// comes from hipGetSymbolAddress, asked once per device with that device current (every GPU holds its own copy of the
// array at its own address), and only that pointer is ever handed to a kernel.
constexpr int kMaxDevices = 64;
int static_scratch_ptr(int64_t** out) {
  static std::mutex mu;
  static int64_t* ptr[kMaxDevices] = {};
  int dev = -1;
  BZ_HIP_OK(hipGetDevice(&dev));
  BZ_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(mu);
  if (ptr[dev] == nullptr) {
    void* p = nullptr;
    BZ_HIP_OK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    BZ_REQUIRE(p != nullptr, "hipGetSymbolAddress gave no address for the scratch buffer on device %d", dev);
    ptr[dev] = static_cast<int64_t*>(p);
  }
  *out = ptr[dev];
  return BZ_OK;
}

}  // namespace

extern "C" {

int32_t bz_table_pitch(int64_t row_bytes, int scale_bytes) {
  if (row_bytes <= 0 || row_bytes > (1 << 24)) return 0;
  int64_t need = (row_bytes + 3) / 4 * 4 + (scale_bytes > 0 ? 4 : 0);
  need = (need + 15) / 16 * 16;
  if (need <= 128) {
    int64_t p = 16;
    while (p < need) p <<= 1;
    return (int32_t)p;
  }
  const int64_t lines = (need + 127) / 128 * 128;
  return (int32_t)(lines * 3 <= need * 4 ? lines : need);
}

int bz_embed_plan(bz_embed_slot* slots, int n_slots, bz_embed_launch* launch) {
  BZ_REQUIRE(slots != nullptr && launch != nullptr && n_slots > 0, "bz_embed_plan: null argument or n_slots=%d", n_slots);
  int64_t total = 0;
  bool uniform_wg = true, uniform_shape = true, any_offsets = false, all_offsets = true;
  int lpr0 = 0;
  for (int i = 0; i < n_slots; ++i) {
    bz_embed_slot& s = slots[i];
    BZ_REQUIRE(s.table_dtype == BZ_F32 || s.table_dtype == BZ_F16 || s.table_dtype == BZ_I8,
               "slot %d: unsupported table dtype %d", i, s.table_dtype);
    BZ_REQUIRE(s.out_dtype == BZ_F32 || s.out_dtype == BZ_F16 || s.out_dtype == BZ_BF16, "slot %d: unsupported out dtype %d", i,
               s.out_dtype);
    BZ_REQUIRE(s.udf == BZ_SUM || s.udf == BZ_AVG || s.udf == BZ_ASSIGN, "slot %d: Unsupported udf type: %d", i, s.udf);
    BZ_REQUIRE(s.dim > 0 && s.batch >= 0 && s.nnz >= 0, "slot %d: dim=%d batch=%d nnz=%lld", i, s.dim, s.batch, (long long)s.nnz);
    if (s.udf == BZ_ASSIGN)
      BZ_REQUIRE(s.trunc_num > 0 && (s.trunc_dir == BZ_ORDER || s.trunc_dir == BZ_REVERSE),
                 "slot %d: kAssign needs trunc_num > 0 and a trunc direction (trunc_num=%d dir=%d)", i, s.trunc_num,
                 s.trunc_dir);
    BZ_REQUIRE(s.assign_pitch == 0 || (s.udf == BZ_ASSIGN && s.assign_pitch >= s.dim),
               "slot %d: assign_pitch=%d is for kAssign items and at least dim=%d", i, s.assign_pitch, s.dim);
    BZ_REQUIRE(s.out != nullptr && (s.batch == 0 || s.segments != nullptr), "slot %d: null out/segments", i);
    if (s.table != nullptr) {
      const int esz = bz::dtype_size(s.table_dtype);
      BZ_REQUIRE(s.pitch % 16 == 0 && s.pitch >= ((s.dim * esz + 15) / 16) * 16,
                 "slot %d: row pitch %d must be a multiple of 16 covering dim*elem=%d", i, s.pitch, s.dim * esz);
      BZ_REQUIRE(((uintptr_t)s.table & 15) == 0, "slot %d: table base not 16-byte aligned", i);
      BZ_REQUIRE(s.table_dtype != BZ_I8 || s.row_scale != nullptr, "slot %d: int8 table without row_scale", i);
      BZ_REQUIRE(s.scale_pitch >= 0 && s.scale_pitch % 4 == 0 && ((uintptr_t)s.row_scale & 3) == 0,
                 "slot %d: scale_pitch=%d / row_scale must be multiples of 4", i, s.scale_pitch);
      BZ_REQUIRE(s.rows > 0 && s.rows < (1ll << 31), "slot %d: rows=%lld outside (0, 2^31)", i, (long long)s.rows);
      BZ_REQUIRE(s.nnz == 0 || (s.ids != nullptr && s.values != nullptr), "slot %d: null ids/values", i);
      if (s.hash_buckets != nullptr)
        BZ_REQUIRE(s.hash_pairs != nullptr && s.hash_bucket_size > 0, "slot %d: incomplete hash index", i);
    }
    any_offsets |= s.offsets != nullptr;
    all_offsets &= s.offsets != nullptr;
    const int g = groups_per_wg(s);
    const int lpr = kThreads / g;
    const int ce = s.table_dtype == BZ_F32 ? 4 : (s.table_dtype == BZ_F16 ? 8 : 16);
    s.wg_begin = (int32_t)total;
    const int64_t items = (int64_t)s.batch * items_per_sample(s);  // lane groups needed
    BZ_REQUIRE((items + g - 1) / g < (1ll << 30), "slot %d: too many workgroups", i);
    s.wg_count = (int32_t)((items + g - 1) / g);
    total += s.wg_count;
    BZ_REQUIRE(total < (1ll << 30), "too many workgroups");
    if (i == 0) lpr0 = lpr;
    uniform_wg &= s.wg_count == slots[0].wg_count;
    uniform_shape &= s.table != nullptr && s.udf != BZ_ASSIGN && lpr == lpr0 && s.table_dtype == slots[0].table_dtype &&
                     (s.dim + ce - 1) / ce <= lpr;
  }
  BZ_REQUIRE(all_offsets || !any_offsets, "either every slot carries offsets or none does");
  launch->n_slots = n_slots;
  launch->total_wg = (int32_t)total;
  launch->wg_per_slot = (uniform_wg && slots[0].wg_count > 0) ? slots[0].wg_count : 0;
  launch->variant = (uniform_shape && launch->wg_per_slot > 0) ? ((slots[0].table_dtype << 8) | lpr0) : 0;
  launch->fused_scan = any_offsets ? 0 : 1;
  // the fused scan reads, per workgroup, the counts before its first sample: on average batch/2 counts of 4 bytes
  int64_t prefix_bytes = 0;
  for (int i = 0; i < n_slots; ++i) prefix_bytes += (int64_t)slots[i].wg_count * slots[i].batch * 2;
  launch->scan_first = (launch->fused_scan && prefix_bytes > kScanFirstBytes) ? 1 : 0;
  int32_t max_batch = 0;
  for (int i = 0; i < n_slots; ++i) max_batch = slots[i].batch > max_batch ? slots[i].batch : max_batch;
  launch->max_batch = max_batch;
  launch->reserved_ = 0;
  return BZ_OK;
}

int bz_segments_to_offsets(const int32_t* segments, int64_t* offsets, int64_t n, bz_stream_t stream) {
  BZ_REQUIRE(offsets != nullptr && n >= 0 && (n == 0 || segments != nullptr), "bz_segments_to_offsets: null argument");
  BZ_REQUIRE(n <= (1ll << 24), "bz_segments_to_offsets: n=%lld exceeds 2^24", (long long)n);
  hipLaunchKernelGGL(bz_scan_segments_kernel, dim3(1), dim3(kThreads), 0, bz::as_stream(stream), segments, offsets, n);
  BZ_LAUNCH_OK("bz_scan_segments_kernel");
  return BZ_OK;
}

int bz_segments_to_offsets_slots(const bz_embed_slot* slots_dev, int n_slots, bz_stream_t stream) {
  BZ_REQUIRE(slots_dev != nullptr && n_slots > 0, "bz_segments_to_offsets_slots: null argument or n_slots=%d", n_slots);
  // the batch sizes are in device memory: always 8 parts a slot; a part beyond its slot's batch returns at once
  hipLaunchKernelGGL(bz_scan_segments_slots_kernel, dim3(n_slots, 8), dim3(kThreads), 0, bz::as_stream(stream), slots_dev,
                     (int64_t*)nullptr, (int64_t)0);
  BZ_LAUNCH_OK("bz_scan_segments_slots_kernel");
  return BZ_OK;
}

// launches the pooling kernel the plan chose; ext_off (may be nullptr) replaces slot.offsets as described at the kernels
static int launch_pool(const bz_embed_slot* slots_dev, const bz_embed_launch& L, const int64_t* ext_off, int64_t ext_stride,
                       hipStream_t st) {
  BZ_REQUIRE(L.n_slots > 0 && L.total_wg >= 0 && L.wg_per_slot >= 0, "bz_embed_pool: bad launch record (n_slots=%d total_wg=%d)",
             L.n_slots, L.total_wg);
  if (L.total_wg == 0) return BZ_OK;
  const int per_xcd = (L.total_wg + bz::kNumXcd - 1) / bz::kNumXcd;
  const dim3 grid(per_xcd * bz::kNumXcd), block(kThreads);
  if (L.variant == 0) {
    hipLaunchKernelGGL(bz_embed_pool_generic_kernel, grid, block, 0, st, slots_dev, L.n_slots, L.total_wg, per_xcd,
                       ((int64_t)L.wg_per_slot * L.n_slots == L.total_wg) ? L.wg_per_slot : 0, ext_off, ext_stride);
    BZ_LAUNCH_OK("bz_embed_pool_generic_kernel");
    return BZ_OK;
  }
  BZ_REQUIRE(L.wg_per_slot > 0 && (int64_t)L.wg_per_slot * L.n_slots == L.total_wg,
             "bz_embed_pool: variant %#x needs equal work per slot", L.variant);
  const int dt = L.variant >> 8, lpr = L.variant & 0xff;
#define BZ_POOL(DT, LPR)                                                                                             \
  hipLaunchKernelGGL((bz_embed_pool_kernel<DT, LPR>), grid, block, 0, st, slots_dev, L.n_slots, L.total_wg, per_xcd, \
                     L.wg_per_slot, ext_off, ext_stride)
#define BZ_POOL_LPR(DT)                                                                      \
  switch (lpr) {                                                                             \
    case 1: BZ_POOL(DT, 1); break;                                                           \
    case 2: BZ_POOL(DT, 2); break;                                                           \
    case 4: BZ_POOL(DT, 4); break;                                                           \
    case 8: BZ_POOL(DT, 8); break;                                                           \
    case 16: BZ_POOL(DT, 16); break;                                                         \
    case 32: BZ_POOL(DT, 32); break;                                                         \
    case 64: BZ_POOL(DT, 64); break;                                                         \
    default: return bz::fail(BZ_EINVAL, "bz_embed_pool: bad lanes-per-row %d in variant", lpr); \
  }
  switch (dt) {
    case BZ_F32: BZ_POOL_LPR(BZ_F32); break;
    case BZ_F16: BZ_POOL_LPR(BZ_F16); break;
    case BZ_I8: BZ_POOL_LPR(BZ_I8); break;
    default: return bz::fail(BZ_EINVAL, "bz_embed_pool: bad table dtype %d in variant", dt);
  }
#undef BZ_POOL_LPR
#undef BZ_POOL
  BZ_LAUNCH_OK("bz_embed_pool_kernel");
  return BZ_OK;
}

int bz_embed_pool(const bz_embed_slot* slots_dev, const bz_embed_launch* launch, bz_stream_t stream) {
  BZ_REQUIRE(slots_dev != nullptr && launch != nullptr, "bz_embed_pool: null argument");
  return launch_pool(slots_dev, *launch, nullptr, 0, bz::as_stream(stream));
}

int bz_embed_pool_args(const bz_embed_slot* slots_host, const bz_embed_launch* launch, bz_stream_t stream) {
  BZ_REQUIRE(slots_host != nullptr && launch != nullptr, "bz_embed_pool_args: null argument");
  const bz_embed_launch& L = *launch;
  BZ_REQUIRE(L.n_slots > 0 && L.total_wg >= 0 && L.wg_per_slot >= 0, "bz_embed_pool_args: bad launch record (n_slots=%d total_wg=%d)",
             L.n_slots, L.total_wg);
  if (L.n_slots > BZ_EMBED_ARG_SLOTS || !L.fused_scan || L.scan_first)
    return bz::fail(BZ_ENOTSUP, "bz_embed_pool_args: takes plans with at most %d slots and the scan fused in", BZ_EMBED_ARG_SLOTS);
  BZ_REQUIRE(L.variant == 0 || (L.wg_per_slot > 0 && (int64_t)L.wg_per_slot * L.n_slots == L.total_wg),
             "bz_embed_pool_args: variant %#x needs equal work per slot", L.variant);
  if (L.total_wg == 0) return BZ_OK;
  SlotPack pack;
  memcpy(pack.s, slots_host, (size_t)L.n_slots * sizeof(bz_embed_slot));
  memset(pack.s + L.n_slots, 0, (size_t)(BZ_EMBED_ARG_SLOTS - L.n_slots) * sizeof(bz_embed_slot));
  const int per_xcd = (L.total_wg + bz::kNumXcd - 1) / bz::kNumXcd;
  const dim3 grid(per_xcd * bz::kNumXcd), block(kThreads);
  hipStream_t st = bz::as_stream(stream);
  if (L.variant == 0) {
    if (L.n_slots > 16) return bz::fail(BZ_ENOTSUP, "bz_embed_pool_args: a plan of mixed row shapes takes at most 16 slots");
    for (int i = 0; i < L.n_slots; ++i)
      BZ_REQUIRE(pack.s[i].offsets == nullptr, "bz_embed_pool_args: slot %d brings offsets, but the plan says the scan is fused in", i);
    SlotBegins begins;
    for (int i = 0; i < 16; ++i) begins.b[i] = i < L.n_slots ? pack.s[i].wg_begin : INT_MAX;
    hipLaunchKernelGGL(bz_embed_pool_generic_args_kernel, grid, block, 0, st, pack, begins, L.total_wg, per_xcd,
                       ((int64_t)L.wg_per_slot * L.n_slots == L.total_wg) ? L.wg_per_slot : 0);
    BZ_LAUNCH_OK("bz_embed_pool_generic_args_kernel");
    return BZ_OK;
  }
  const int dt = L.variant >> 8, lpr = L.variant & 0xff;
#define BZ_POOL(DT, LPR) \
  hipLaunchKernelGGL((bz_embed_pool_args_kernel<DT, LPR>), grid, block, 0, st, pack, L.total_wg, per_xcd, L.wg_per_slot)
#define BZ_POOL_LPR(DT)                                                                           \
  switch (lpr) {                                                                                  \
    case 1: BZ_POOL(DT, 1); break;                                                                \
    case 2: BZ_POOL(DT, 2); break;                                                                \
    case 4: BZ_POOL(DT, 4); break;                                                                \
    case 8: BZ_POOL(DT, 8); break;                                                                \
    case 16: BZ_POOL(DT, 16); break;                                                              \
    case 32: BZ_POOL(DT, 32); break;                                                              \
    case 64: BZ_POOL(DT, 64); break;                                                              \
    default: return bz::fail(BZ_EINVAL, "bz_embed_pool_args: bad lanes-per-row %d in variant", lpr); \
  }
  switch (dt) {
    case BZ_F32: BZ_POOL_LPR(BZ_F32); break;
    case BZ_F16: BZ_POOL_LPR(BZ_F16); break;
    case BZ_I8: BZ_POOL_LPR(BZ_I8); break;
    default: return bz::fail(BZ_EINVAL, "bz_embed_pool_args: bad table dtype %d in variant", dt);
  }
#undef BZ_POOL_LPR
#undef BZ_POOL
  BZ_LAUNCH_OK("bz_embed_pool_args_kernel");
  return BZ_OK;
}

int bz_embed_pool_static_scratch(const bz_embed_slot* slots_dev, const bz_embed_launch* launch, bz_stream_t stream) {
  BZ_REQUIRE(slots_dev != nullptr && launch != nullptr, "bz_embed_pool_static_scratch: null argument");
  const bz_embed_launch& L = *launch;
  BZ_REQUIRE(L.n_slots > 0 && L.max_batch >= 0, "bz_embed_pool_static_scratch: bad launch record (n_slots=%d max_batch=%d)",
             L.n_slots, L.max_batch);
  const int64_t stride = (int64_t)L.max_batch + 1;  // int64 entries per slot
  BZ_REQUIRE((int64_t)L.n_slots * stride <= kStaticScratchEntries,
             "bz_embed_pool_static_scratch: %d slots x (batch %d + 1) offsets = %lld bytes exceed the library's %u-byte buffer",
             L.n_slots, L.max_batch, (long long)((int64_t)L.n_slots * stride * 8), BZ_EMBED_STATIC_SCRATCH_BYTES);
  int64_t* off = nullptr;
  const int rc = static_scratch_ptr(&off);
  if (rc != BZ_OK) return rc;
  hipStream_t st = bz::as_stream(stream);
  // nothing to clear: the scan writes entries [0, batch] of every slot's share, the only ones the pooling kernel reads
  hipLaunchKernelGGL(bz_scan_segments_slots_kernel, dim3(L.n_slots, scan_parts(L.max_batch)), dim3(kThreads), 0, st, slots_dev, off,
                     stride);
  BZ_LAUNCH_OK("bz_scan_segments_slots_kernel");
  return launch_pool(slots_dev, L, off, stride, st);
}

const char* bz_embed_pool_kernel_name(void) { return "bz_embed_pool_kernel"; }

}  // extern "C"
