/*
 * blaze_oracle.c -- CPU restatement of Blaze's sparse CTR inference hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is the checker the GPU
 * kernels are compared against (tests, the smoke check and the cpu_baseline
 * leg of the benchmark).  Nothing in the shipped library links or calls it.
 *
 * Every function restates one reference function in plain C and cites it.
 * Paths are relative to the reference tree's blaze/ directory.
 *
 * Pin status (which independent evidence holds each function in place):
 *   orc_segments_to_offsets  reference fixtures (segments of embedding_v1.conf),
 *                            invariants off[0]=0, off[B]=nnz, brute force
 *   orc_hash_*               the compiled reference HashTable (oracle/_ref),
 *                            reference keys of quick_embedding_dict_test.cc
 *   orc_embed_get (fp32)     the compiled reference UdfProcessor + HashTable +
 *                            WeightBlob (oracle/_ref); udf_processor_test.cc and
 *                            quick_embedding_dict_test.cc known answers
 *   orc_embed_get (fp16)     binary16->binary32 widening is exact; checked against
 *                            numpy's float16 widening on all 65536 bit patterns
 *   orc_embed_get (int8)     NOT a reference feature (the reference store rejects
 *                            int8 tables, store/defines.h:29-50).  Semantics are
 *                            defined here; pinned by brute force in numpy only.
 *   orc_gemm & friends       reference known answers (gemm_net_v1, fused_parallel_
 *                            gemm v1..v5, matmul_net_v1, fused_parallel_matmul
 *                            v1..v3) + fp64 numpy matmul on random shapes
 *   orc_prelu/dice/...       reference known answers (prelu_net_v1, dice_net_v1,
 *                            leaky_relu_net_v1, sigmoid_net_v1, softmax_net_v1) +
 *                            closed-form limits
 *   3-D Gemm                 "parity unpinned" by reference fixtures (none exists);
 *                            pinned by the loop-of-2-D identity only
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* binary16 -> binary32, exact (reference: common/types.h:81 operator float(), */
/* which widens through F16C; widening is value-preserving by IEEE-754).       */
/* ------------------------------------------------------------------------- */
static float orc_half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        e++;
        man <<= 1;
      } while ((man & 0x400u) == 0);
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* binary32 -> binary16, round to nearest even (reference: common/types.cc:9-19,
 * _mm256_cvtps_ph(x, 0) / _cvtss_sh(x, 0) = RNE). */
static uint16_t orc_float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) { /* inf / nan */
    uint32_t man = absx & 0x7fffffu;
    return (uint16_t)(sign | 0x7c00u | (man ? (0x200u | (man >> 13)) : 0));
  }
  if (absx >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx < 0x33000001u) { /* < 2^-25 (or == 2^-25 ties to even 0) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u;
  uint32_t shift;
  uint32_t hexp;
  if (e < -14) { /* subnormal half */
    shift = (uint32_t)(13 + (-14 - e));
    hexp = 0;
  } else {
    shift = 13;
    hexp = (uint32_t)(e + 15);
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  uint32_t out;
  if (hexp == 0) {
    out = q; /* may carry into exponent 1: correct encoding */
  } else {
    out = ((hexp - 1) << 10) + q; /* q carries the implicit 1 at bit 10 */
  }
  return (uint16_t)(sign | out);
}

ORC_API void orc_half_to_float_n(const uint16_t* h, float* f, int64_t n) {
  for (int64_t i = 0; i < n; ++i) f[i] = orc_half_to_float(h[i]);
}

ORC_API void orc_float_to_half_n(const float* f, uint16_t* h, int64_t n) {
  for (int64_t i = 0; i < n; ++i) h[i] = orc_float_to_half(f[i]);
}

/* ------------------------------------------------------------------------- */
/* segments (per-sample id counts) -> exclusive offsets.                      */
/* The reference never materialises the offsets: it advances key/value         */
/* pointers by num after each sample (store/quick_embedding/                   */
/* quick_embedding_dict.cc:111-140).  The pointer position before sample i is  */
/* this exclusive prefix sum.  off has n+1 entries; off[n] = total id count.   */
/* ------------------------------------------------------------------------- */
ORC_API void orc_segments_to_offsets(const int32_t* segments, int64_t* off, int64_t n) {
  int64_t run = 0;
  for (int64_t i = 0; i < n; ++i) {
    off[i] = run;
    run += (int64_t)segments[i];
  }
  off[n] = run;
}

/* ------------------------------------------------------------------------- */
/* Hash index: key -> value.  Restates store/quick_embedding/hashtable.{h,cc}. */
/* ------------------------------------------------------------------------- */
typedef struct {
  uint32_t bucket_size;
  uint64_t* bucket_offset; /* byte offset into pairs (Bucket.offset, 40 bit) */
  uint32_t* bucket_count;  /* Bucket.size, 24 bit */
  uint64_t byte_size;
  unsigned char* bytes;    /* (u64 key, u64 value) pairs, hashtable.cc:171-187 */
} orc_hashtable;

/* prime ladder, hashtable.cc:12-32 */
static const uint32_t kOrcSteps[] = {
    53,       97,       193,       389,       769,       1543,     3079,
    6151,     12289,    24593,     49157,     98317,     196613,   393241,
    786433,   1572869,  3145739,   6291469,   12582917,  25165843, 50331653,
    100663319, 201326611, 402653189, 805306457};

ORC_API uint32_t orc_hash_bucket_size(uint32_t node_size) {
  uint32_t n = sizeof(kOrcSteps) / sizeof(kOrcSteps[0]);
  for (uint32_t i = 0; i < n; ++i)
    if (kOrcSteps[i] > node_size) return kOrcSteps[i];
  return kOrcSteps[n - 1];
}

typedef struct {
  uint64_t key, value;
  uint32_t bucket;
} orc_item;

static int orc_item_cmp(const void* a, const void* b) {
  const orc_item* x = (const orc_item*)a;
  const orc_item* y = (const orc_item*)b;
  if (x->bucket != y->bucket) return x->bucket < y->bucket ? -1 : 1;
  if (x->key != y->key) return x->key < y->key ? -1 : 1;
  return 0;
}

/* BulkLoadHashTable::PreInsert + BulkLoad, hashtable.cc:137-187.  Duplicate
 * keys are all stored; Lookup returns the first in (bucket, key) order. */
ORC_API orc_hashtable* orc_hash_build(const uint64_t* keys, const uint64_t* values, uint64_t n) {
  orc_hashtable* t = (orc_hashtable*)calloc(1, sizeof(*t));
  t->bucket_size = orc_hash_bucket_size((uint32_t)n);
  t->bucket_offset = (uint64_t*)calloc(t->bucket_size, sizeof(uint64_t));
  t->bucket_count = (uint32_t*)calloc(t->bucket_size, sizeof(uint32_t));
  orc_item* items = (orc_item*)malloc(sizeof(orc_item) * (n ? n : 1));
  for (uint64_t i = 0; i < n; ++i) {
    items[i].key = keys[i];
    items[i].value = values[i];
    items[i].bucket = (uint32_t)keys[i] % t->bucket_size; /* hashcode = (u32)key */
  }
  qsort(items, n, sizeof(orc_item), orc_item_cmp);
  t->byte_size = 16 * n;
  t->bytes = (unsigned char*)malloc(t->byte_size ? t->byte_size : 1);
  for (uint64_t i = 0; i < n; ++i) {
    uint32_t b = items[i].bucket;
    if (t->bucket_count[b] == 0) t->bucket_offset[b] = 16 * i;
    memcpy(t->bytes + 16 * i, &items[i].key, 8);
    memcpy(t->bytes + 16 * i + 8, &items[i].value, 8);
    t->bucket_count[b]++;
  }
  free(items);
  return t;
}

ORC_API void orc_hash_free(orc_hashtable* t) {
  if (!t) return;
  free(t->bucket_offset);
  free(t->bucket_count);
  free(t->bytes);
  free(t);
}

/* HashTable::Lookup, hashtable.cc:45-64 */
ORC_API int orc_hash_lookup(const orc_hashtable* t, uint64_t key, uint64_t* value) {
  if (!t || !t->bucket_size || !t->bytes) return 0;
  uint32_t hash_code = (uint32_t)key;
  uint32_t b = hash_code % t->bucket_size;
  uint32_t cnt = t->bucket_count[b];
  if (!cnt) return 0;
  const unsigned char* p = t->bytes + t->bucket_offset[b];
  for (uint32_t i = 0; i < cnt; ++i) {
    uint64_t k;
    memcpy(&k, p, 8);
    if (k == key) {
      memcpy(value, p + 8, 8);
      return 1;
    }
    p += 16;
  }
  return 0;
}

/* Serialised image of the index exactly as HashTable::Dump writes it
 * (hashtable.cc:73-94): u32 bucket_size; Bucket[bucket_size] where Bucket is
 * the 8-byte bitfield {offset:40, size:24} (hashtable.h:41-46); u64 byte_size;
 * pairs.  Returns the number of bytes; writes only if dst != NULL. */
ORC_API uint64_t orc_hash_dump(const orc_hashtable* t, unsigned char* dst) {
  uint64_t need = 4 + 8ull * t->bucket_size + 8 + t->byte_size;
  if (!dst) return need;
  memcpy(dst, &t->bucket_size, 4);
  dst += 4;
  for (uint32_t i = 0; i < t->bucket_size; ++i) {
    uint64_t rec = (t->bucket_offset[i] & 0xffffffffffull) | ((uint64_t)(t->bucket_count[i] & 0xffffffu) << 40);
    memcpy(dst, &rec, 8);
    dst += 8;
  }
  memcpy(dst, &t->byte_size, 8);
  dst += 8;
  memcpy(dst, t->bytes, t->byte_size);
  return need;
}

ORC_API void orc_hash_export(const orc_hashtable* t, uint32_t* bucket_size, const uint64_t** bucket_offset,
                             const uint32_t** bucket_count, const unsigned char** bytes, uint64_t* byte_size) {
  *bucket_size = t->bucket_size;
  *bucket_offset = t->bucket_offset;
  *bucket_count = t->bucket_count;
  *bytes = t->bytes;
  *byte_size = t->byte_size;
}

/* ------------------------------------------------------------------------- */
/* Embedding gather + pooling.                                                */
/* ------------------------------------------------------------------------- */
enum { ORC_FP32 = 0, ORC_FP16 = 1, ORC_INT8 = 2 };          /* table dtypes */
enum { ORC_SUM = 0, ORC_AVG = 1, ORC_ASSIGN = 2 };          /* store/store.h:21-25 */
enum { ORC_ORDER = 0, ORC_REVERSE = 1 };                    /* store/sparse_puller.h:35-38 */

typedef struct {
  int32_t dtype;       /* ORC_FP32 | ORC_FP16 | ORC_INT8 */
  int32_t dim;
  int64_t rows;
  int64_t pitch;       /* bytes between rows */
  const void* data;
  const float* scale;  /* per-row scale, ORC_INT8 only */
  const orc_hashtable* hash; /* NULL: ids are row numbers; else ids are keys, value = row number */
} orc_table;

typedef struct {
  int32_t udf;         /* ORC_SUM | ORC_AVG | ORC_ASSIGN */
  int32_t trunc_dir;   /* ORC_ORDER | ORC_REVERSE */
  int32_t trunc_num;
  int32_t pad_;
  float* out;          /* first sample's slot inside the block */
  int64_t stride;      /* elements between consecutive samples */
} orc_item_out;

/* resolve an id to its weight row; returns 0 when the id is not in the table
 * (quick_embedding_dict.h:55-71: hash miss, or blob offset past the end) */
static int orc_row_of(const orc_table* t, int64_t id, int64_t* row) {
  if (t->hash) {
    uint64_t v;
    if (!orc_hash_lookup(t->hash, (uint64_t)id, &v)) return 0;
    if (v >= (uint64_t)t->rows) return 0;
    *row = (int64_t)v;
    return 1;
  }
  if (id < 0 || id >= t->rows) return 0;
  *row = id;
  return 1;
}

/* dequantised fp32 weight k of a row */
static float orc_weight(const orc_table* t, int64_t row, int k) {
  const unsigned char* p = (const unsigned char*)t->data + row * t->pitch;
  switch (t->dtype) {
    case ORC_FP32: {
      float f;
      memcpy(&f, p + 4 * k, 4);
      return f;
    }
    case ORC_FP16: {
      uint16_t h;
      memcpy(&h, p + 2 * k, 2);
      return orc_half_to_float(h); /* (ValueType)(weights[i]), udf_processor.h:66 */
    }
    default: {
      /* extension (not in the reference): w = scale[row] * (float)q, one fp32 rounding */
      float q = (float)((const int8_t*)p)[k];
      return t->scale[row] * q;
    }
  }
}

/*
 * One feature group: restates QuickEmbeddingDict::Get(input, output)
 * (store/quick_embedding/quick_embedding_dict.cc:89-148) with the three
 * UdfProcessors of store/quick_embedding/udf_processor.h:43-133 inlined.
 *   ids/values: [nnz]; segments: [batch] counts; items: one per block the group feeds.
 * Arithmetic is fp32, multiply then add, never fused (udf_processor.h:66 built
 * without -mfma, CMakeLists.txt:78) -- volatile temporaries forbid contraction.
 * A NULL table (unknown table name) leaves the outputs untouched
 * (quick_embedding_dict.cc:95).
 */
ORC_API int orc_embed_get(const orc_table* t, const int64_t* ids, const float* values, const int32_t* segments,
                          int64_t batch, const orc_item_out* items, int32_t n_items) {
  if (!t) return 0;
  const int dim = t->dim;
  float** out = (float**)malloc(sizeof(float*) * (size_t)(n_items > 0 ? n_items : 1));
  for (int k = 0; k < n_items; ++k) out[k] = items[k].out;
  const int64_t* key = ids;
  const float* value = values;
  for (int64_t i = 0; i < batch; ++i) {
    size_t num = (size_t)segments[i];
    /* InitProcess: udf_processor.h:50-55 (sum/avg), :103-108 (assign) */
    for (int k = 0; k < n_items; ++k) {
      size_t n = items[k].udf == ORC_ASSIGN ? (size_t)dim * (size_t)items[k].trunc_num : (size_t)dim;
      memset(out[k], 0, n * sizeof(float));
    }
    for (size_t j = 0; j < num; ++j) {
      int64_t row;
      if (!orc_row_of(t, key[j], &row)) continue; /* quick_embedding_dict.cc:121-123 */
      for (int k = 0; k < n_items; ++k) {
        const orc_item_out* it = &items[k];
        if (it->udf == ORC_ASSIGN) { /* udf_processor.h:110-131 */
          if (it->trunc_dir == ORC_ORDER && j >= (size_t)it->trunc_num) continue;
          if (it->trunc_dir == ORC_REVERSE && (num - j) > (size_t)it->trunc_num) continue;
          float* o = out[k];
          if (it->trunc_dir == ORC_ORDER)
            o += (size_t)dim * j;
          else
            o += (size_t)dim * ((size_t)it->trunc_num - (num - j));
          for (int c = 0; c < dim; ++c) {
            volatile float prod = value[j] * orc_weight(t, row, c);
            o[c] = prod;
          }
        } else { /* udf_processor.h:57-70 */
          float* o = out[k];
          for (int c = 0; c < dim; ++c) {
            volatile float prod = value[j] * orc_weight(t, row, c);
            volatile float sum = o[c] + prod;
            o[c] = sum;
          }
        }
      }
    }
    /* ReduceProcess: udf_processor.h:82-91 (avg only; size==0 -> untouched) */
    for (int k = 0; k < n_items; ++k) {
      if (items[k].udf == ORC_AVG && num != 0) {
        float inv = (float)(1.0 / (double)num);
        for (int c = 0; c < dim; ++c) {
          volatile float r = out[k][c] * inv;
          out[k][c] = r;
        }
      }
      out[k] += items[k].stride; /* quick_embedding_dict.cc:135-136 */
    }
    key += num;
    value += num;
  }
  free(out);
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Dense: GEMM family.  Restates the row-major cblas_sgemm contract the         */
/* reference calls (math/gemm.cc:13-27): C = alpha*op(A)*op(B) + beta*C with     */
/* lda = K|M, ldb = N|K, ldc = N.  MKL's internal summation order is not         */
/* reproducible; this is the textbook k-ascending fp32 sum (and an fp64 twin     */
/* used to scale tolerances).                                                    */
/* ------------------------------------------------------------------------- */
ORC_API void orc_gemm_ex(int transa, int transb, int M, int N, int K, float alpha, const float* A, int lda,
                         const float* B, int ldb, float beta, float* C, int ldc) {
  for (int m = 0; m < M; ++m) {
    for (int n = 0; n < N; ++n) {
      float acc = 0.f;
      for (int k = 0; k < K; ++k) {
        float a = transa ? A[(size_t)k * lda + m] : A[(size_t)m * lda + k];
        float b = transb ? B[(size_t)n * ldb + k] : B[(size_t)k * ldb + n];
        acc += a * b;
      }
      float* c = &C[(size_t)m * ldc + n];
      *c = (beta == 0.f) ? alpha * acc : alpha * acc + beta * (*c); /* beta==0: C not read (BLAS rule) */
    }
  }
}

ORC_API void orc_gemm_ex_f64(int transa, int transb, int M, int N, int K, float alpha, const float* A, int lda,
                             const float* B, int ldb, float beta, const float* Cin, double* Cout, int ldc) {
  for (int m = 0; m < M; ++m) {
    for (int n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int k = 0; k < K; ++k) {
        double a = transa ? A[(size_t)k * lda + m] : A[(size_t)m * lda + k];
        double b = transb ? B[(size_t)n * ldb + k] : B[(size_t)k * ldb + n];
        acc += a * b;
      }
      double c = (beta == 0.f || !Cin) ? 0.0 : (double)beta * (double)Cin[(size_t)m * ldc + n];
      Cout[(size_t)m * ldc + n] = (double)alpha * acc + c;
    }
  }
}

/* Gemm<float,CPUContext>, math/gemm.cc:13-27 */
ORC_API void orc_gemm(int transa, int transb, int M, int N, int K, float alpha, const float* A, const float* B,
                      float beta, float* C) {
  orc_gemm_ex(transa, transb, M, N, K, alpha, A, transa ? M : K, B, transb ? K : N, beta, C, N);
}

/* GemmStridedBatched<float,CPUContext>, math/gemm.cc:82-139 (element strides; 0 = shared operand) */
ORC_API void orc_gemm_strided_batched(int transa, int transb, int M, int N, int K, float alpha, const float* A,
                                      long long stride_a, const float* B, long long stride_b, float beta, float* C,
                                      long long stride_c, int batch) {
  for (int i = 0; i < batch; ++i)
    orc_gemm(transa, transb, M, N, K, alpha, A + stride_a * i, B + stride_b * i, beta, C + stride_c * i);
}

/* DimEqualBroadcastAssign, math/broadcast.cc:15-29: y[off+z] = x[z] tiled over y */
ORC_API void orc_broadcast_assign(float* y, int64_t y_size, const float* x, int64_t x_size) {
  for (int64_t o = 0; o < y_size; o += x_size)
    for (int64_t z = 0; z < x_size; ++z) y[o + z] = x[z];
}

/*
 * GemmOp::RunOnDevice, operator/op/gemm_op.h:33-107.
 *   a_rank 2: A is [a0,a1];  a_rank 3: A is [a0,a1,a2].  B is [b0,b1].
 *   c_size: 0 = no bias, else number of bias elements ([N] or [M,N]).
 *   Y must hold the output ([M,N] or [a0,M,N]); y_shape (3 ints) receives it.
 */
ORC_API int orc_gemm_op(int transa, int transb, float alpha, float beta, const float* A, int a_rank, const int64_t* a_shape,
                        const float* B, const int64_t* b_shape, const float* Cb, int64_t c_size, float* Y,
                        int64_t* y_shape) {
  int64_t M = a_rank == 3 ? a_shape[1] : a_shape[0];
  int64_t K = a_rank == 3 ? a_shape[2] : a_shape[1];
  if (transa) {
    int64_t t = M;
    M = K;
    K = t;
  }
  int64_t N = transb ? b_shape[0] : b_shape[1];
  int64_t bk = transb ? b_shape[1] : b_shape[0];
  if (bk != K) return -1; /* CheckValid, gemm_op.h:134 */
  int is3d = 0;
  int64_t y_size;
  if (a_rank == 3) {
    y_shape[0] = a_shape[0];
    y_shape[1] = M;
    y_shape[2] = N;
    y_size = a_shape[0] * M * N;
    if (M == 1)
      M = a_shape[0]; /* gemm_op.h:54-55 */
    else
      is3d = 1;
  } else {
    y_shape[0] = M;
    y_shape[1] = N;
    y_shape[2] = 0;
    y_size = M * N;
  }
  if (!Cb || c_size == 0)
    beta = 0.f;
  else
    orc_broadcast_assign(Y, y_size, Cb, c_size); /* gemm_op.h:66-72 */
  if (is3d)
    orc_gemm_strided_batched(transa, transb, (int)M, (int)N, (int)K, alpha, A, M * K, B, 0, beta, Y, M * N,
                             (int)a_shape[0]);
  else
    orc_gemm(transa, transb, (int)M, (int)N, (int)K, alpha, A, B, beta, Y);
  return 0;
}

/*
 * FusedParallelGemmOp::RunOnDevice, operator/fused_op/fused_parallel_gemm_op.h:43-133
 * (2-D A only here; the 3-D branch is a loop of the 3-D GemmOp).  B is the P
 * weight matrices stacked on dim 0; bias is [P*N] or [P*M,N]; Y is [P*M,N].
 */
ORC_API int orc_fused_parallel_gemm_op(int P, int transa, int transb, float alpha, float beta, const float* A,
                                       const int64_t* a_shape, const float* B, const int64_t* b_shape, const float* Cb,
                                       int64_t c_size, float* Y) {
  int64_t M = a_shape[0], K = a_shape[1];
  if (transa) {
    int64_t t = M;
    M = K;
    K = t;
  }
  int64_t N = transb ? b_shape[0] / P : b_shape[1];
  int64_t bk = transb ? b_shape[1] : b_shape[0] / P;
  if (bk != K) return -1;
  if (!Cb || c_size == 0) {
    beta = 0.f;
  } else {
    /* DimEqualBatchedBroadcastAssign, math/broadcast.cc:52-66: per parallel slice */
    int64_t ys = M * N, xs = c_size / P;
    for (int p = 0; p < P; ++p) orc_broadcast_assign(Y + p * ys, ys, Cb + p * xs, xs);
  }
  orc_gemm_strided_batched(transa, transb, (int)M, (int)N, (int)K, alpha, A, 0, B, K * N, beta, Y, M * N, P);
  return 0;
}

/*
 * MatMulOp via BroadcastGemm_NxN, operator/op/matmul_op.h:31-92 and
 * math/broadcast.h:157-222: a_batch / b_batch are the products of the outer
 * dims (1 = broadcast that operand); alpha=1, beta=0.  C is [max(batch),M,N].
 */
ORC_API int orc_matmul_op(int transa, int transb, int M, int N, int K, const float* A, int64_t a_batch, const float* B,
                          int64_t b_batch, float* C) {
  if (a_batch == 1 && b_batch == 1) {
    orc_gemm(transa, transb, M, N, K, 1.f, A, B, 0.f, C);
  } else if (a_batch != 1 && b_batch != 1) {
    if (a_batch != b_batch) return -1;
    orc_gemm_strided_batched(transa, transb, M, N, K, 1.f, A, (long long)M * K, B, (long long)K * N, 0.f, C,
                             (long long)M * N, (int)a_batch);
  } else {
    orc_gemm_strided_batched(transa, transb, M, N, K, 1.f, A, a_batch == 1 ? 0 : (long long)M * K, B,
                             b_batch == 1 ? 0 : (long long)K * N, 0.f, C, (long long)M * N,
                             (int)(a_batch == 1 ? b_batch : a_batch));
  }
  return 0;
}

/*
 * FusedParallelMatMulOp via BatchedBroadcastGemm_NxN,
 * operator/fused_op/fused_parallel_matmul_op.h:36-93, math/broadcast.h:267-381.
 * a_batch / b_batch are per-parallel-slice outer sizes.  The reference's
 * N==1 shortcut (broadcast.h:319-338) is an algebraic rewrite of the same
 * products, so the plain nested loop below has the same value.
 */
ORC_API int orc_fused_parallel_matmul_op(int P, int transa, int transb, int M, int N, int K, const float* A,
                                         int64_t a_batch, const float* B, int64_t b_batch, float* C) {
  int64_t cb = a_batch > b_batch ? a_batch : b_batch;
  if (a_batch != b_batch && a_batch != 1 && b_batch != 1) return -1;
  for (int p = 0; p < P; ++p) {
    const float* Ap = A + (int64_t)p * a_batch * M * K;
    const float* Bp = B + (int64_t)p * b_batch * K * N;
    float* Cp = C + (int64_t)p * cb * M * N;
    for (int64_t i = 0; i < cb; ++i) {
      const float* Ai = Ap + (a_batch == 1 ? 0 : i * M * K);
      const float* Bi = Bp + (b_batch == 1 ? 0 : i * K * N);
      orc_gemm(transa, transb, M, N, K, 1.f, Ai, Bi, 0.f, Cp + i * M * N);
    }
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Activations                                                                */
/* ------------------------------------------------------------------------- */

/* PRelu: operator/op/prelu_op.cc:11-30 with Activation<kPRelu>, math/activation.h:37-42:
 * y = x * ((x>0) + (x<0)*w[j]),  j = flat index % w_size */
ORC_API void orc_prelu(const float* x, const float* w, float* y, int64_t size, int64_t w_size) {
  for (int64_t i = 0; i < size; ++i) {
    float xv = x[i];
    float wv = w[i % w_size];
    y[i] = xv * ((float)(xv > 0) + (float)(xv < 0) * wv);
  }
}

/* Dice (inference form): operator/op/dice_op.cc:15-34; kDiceEpsilon is the
 * float 1e-8 of operator/common_helper.h:90; exp is std::exp on float when
 * MKL's vmsExp is not used (math/vml.cc:105). */
ORC_API void orc_dice(const float* x, const float* gamma, const float* mean, const float* var, float* y, int64_t size,
                      int64_t c, int nosqrt) {
  const float eps = 1e-8f;
  int64_t rows = size / c;
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * c;
    float* yr = y + r * c;
    for (int64_t j = 0; j < c; ++j) {
      float den = nosqrt ? var[j] : sqrtf(var[j] + eps);
      float t = -1 * (xr[j] - mean[j]) / den;
      t = expf(t);
      float p = 1 / (1 + t);
      yr[j] = (1 - p) * gamma[j] * xr[j] + p * xr[j];
    }
  }
}

/* LeakyRelu: operator/op/leaky_relu_op.cc:15-21 with Activation<kRelu>, math/activation.h:29-34 */
ORC_API void orc_leaky_relu(const float* x, float* y, int64_t size, float alpha) {
  for (int64_t i = 0; i < size; ++i) y[i] = x[i] >= 0 ? x[i] : alpha * x[i];
}

/* Sigmoid: operator/op/sigmoid_op.cc:15-21: y = e^x / (1 + e^x) (overflows to NaN for x > ~88.7) */
ORC_API void orc_sigmoid(const float* x, float* y, int64_t size) {
  for (int64_t i = 0; i < size; ++i) {
    float e = expf(x[i]);
    y[i] = e / (1 + e);
  }
}

/* Softmax over axis with shape [n, c, w]: operator/op/softmax_op.cc:21-78
 * (max-subtracted; sum accumulated in channel order) */
ORC_API void orc_softmax(const float* x, float* y, int64_t n, int64_t c, int64_t w) {
  for (int64_t i = 0; i < n; ++i) {
    for (int64_t z = 0; z < w; ++z) {
      const float* xs = x + i * c * w + z;
      float* ys = y + i * c * w + z;
      float mx = xs[0];
      for (int64_t j = 1; j < c; ++j) mx = xs[j * w] > mx ? xs[j * w] : mx;
      float sum = 0.f;
      for (int64_t j = 0; j < c; ++j) {
        ys[j * w] = expf(xs[j * w] - mx);
        sum += ys[j * w];
      }
      for (int64_t j = 0; j < c; ++j) ys[j * w] /= sum;
    }
  }
}

/* ReduceSum over the middle axis of [outer, dim, inner]: math/reduce.cc:13-29 (y zeroed, then rows of
 * `inner` added in ascending j). */
ORC_API void orc_reduce_sum(const float* x, int64_t outer, int64_t dim, int64_t inner, float* y) {
  for (int64_t i = 0; i < outer; ++i) {
    for (int64_t k = 0; k < inner; ++k) y[k] = 0.f;
    for (int64_t j = 0; j < dim; ++j) {
      for (int64_t k = 0; k < inner; ++k) y[k] = y[k] + x[k];
      x += inner;
    }
    y += inner;
  }
}

/* BatchNormalization (inference): operator/op/batch_normalization_op.cc:11-18; channel = flat index % c. */
ORC_API void orc_batch_norm(const float* x, int64_t size, const float* gamma, const float* beta, const float* mean,
                            const float* var, int64_t c, int nosqrt, float eps, float* y) {
  for (int64_t i = 0; i < size; ++i) {
    int64_t o = i % c;
    float den = nosqrt ? var[o] : sqrtf(var[o] + eps);
    float xn = (x[i] - mean[o]) / den;
    float g = gamma[o] * xn;
    y[i] = g + beta[o];
  }
}
