/*
 * blaze_hip.h -- C ABI of the MI355X (gfx950) kernel layer behind Blaze's sparse
 * CTR inference hot path: Embedding gather/pool, fused FC, batched matmul,
 * standalone activations.
 *
 * Conventions
 *   - every pointer named *_dev / documented "device" is HIP device memory on the
 *     current device; the library never allocates, frees or synchronises;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); all work
 *     is stream ordered;
 *   - return 0 on success, a negative BZ_E* code otherwise; bz_last_error() gives
 *     the message for the calling thread; nothing throws across this boundary.
 *
 * The reference has no C layer at this level: its operators are C++ templates that
 * call cuBLAS / CUDA kernels directly.  Each entry point below names the reference
 * code it stands in for (paths relative to the reference's blaze/ directory).
 */
#ifndef BLAZE_HIP_H_
#define BLAZE_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BZ_API __attribute__((visibility("default")))

typedef void* bz_stream_t;

enum bz_status {
  BZ_OK = 0,
  BZ_EINVAL = -22,  /* bad argument (shape, alignment, enum) */
  BZ_ENOTSUP = -95, /* valid request this build has no kernel for */
  BZ_EHIP = -5      /* a HIP runtime call failed */
};

/* element types; values of the first five follow blaze/proto/blaze.proto:6-19 (DataType) */
enum bz_dtype {
  BZ_F32 = 1,
  BZ_I32 = 2,
  BZ_I8 = 7,
  BZ_I64 = 10,
  BZ_F16 = 12,
  BZ_BF16 = 100 /* not a Blaze DataType; used by the bf16 dense tower */
};

/* pooling kinds, blaze/proto/embedding.proto:20-25 and blaze/store/store.h:21-25 */
enum bz_udf { BZ_SUM = 0, BZ_AVG = 1, BZ_ASSIGN = 2 };
/* blaze/proto/embedding.proto:14-17, blaze/store/sparse_puller.h:35-38 */
enum bz_trunc { BZ_ORDER = 0, BZ_REVERSE = 1 };

/* message of the last failing call on this thread (never NULL); mirrors the
 * thread-local error buffer of blaze/api/c_api/c_api_error.cc:12-28 */
BZ_API const char* bz_last_error(void);

/* library / device probe: fills name (<= cap bytes) with the gcnArchName of the
 * current device, returns BZ_ENOTSUP when it is not gfx950 */
BZ_API int bz_device_check(char* name, size_t cap);

/*
 * One wave that keeps `stream` busy for about `microseconds` (0 .. 10000; 0 = an empty kernel).  No counterpart in the
 * reference: the serving pool uses it to find out which of its streams share a hardware queue (a kernel queued on a
 * stream that shares the busy one's queue cannot finish before it).
 */
BZ_API int bz_spin(int64_t microseconds, bz_stream_t stream);

/* ------------------------------------------------------------------------- */
/* Embedding                                                                  */
/* ------------------------------------------------------------------------- */

/*
 * One (feature group -> block item) unit of work.  An array of these lives in
 * DEVICE memory and is owned by the caller (the Embedding operator), which
 * rewrites it when an input blob moves.  It carries what the reference passes as
 * SparsePullerInput + SparsePullerInput::Param + SparsePullerOutput::OutItem
 * (blaze/store/sparse_puller.h:40-75) plus the resolved table.
 *
 * Table layout (repacked at load time from the QED blob, whose rows start at
 * byte offset 1 and are unaligned, blaze/store/quick_embedding/weight_blob.h:20,42-52):
 * row r starts at table + r*pitch, pitch is a multiple of 16 bytes, the base is
 * 16-byte aligned, bytes between dim*sizeof(elem) and pitch are zero (or hold the
 * row's scale, see row_scale).  The memory system fetches whole 128-byte lines, so
 * a table is best laid out with rows that do not straddle lines: bz_table_pitch
 * gives the pitch this library's own loaders use.
 *
 * ids are row numbers (id outside [0, rows) = not in table) unless hash_buckets is
 * set; then ids are 64-bit keys resolved exactly as HashTable::Lookup does
 * (blaze/store/quick_embedding/hashtable.cc:45-64): bucket = (uint32)key %
 * hash_bucket_size, linear scan of the bucket's (u64 key, u64 row) pairs.
 */
typedef struct bz_embed_slot {
  const void* table;          /* device; NULL = unknown table: the item's columns are zero-filled */
  const float* row_scale;     /* device; BZ_I8 tables only: the scale of row r is the float at byte offset
                                 r * scale_pitch from here (a dense array, or a field inside each table row) */
  const uint64_t* hash_buckets; /* device [hash_bucket_size] records {offset:40 (bytes into pairs), size:24}; or NULL */
  const uint64_t* hash_pairs;   /* device (key,row) pairs */
  const int64_t* ids;         /* device [nnz]   "<fg>.ids"      */
  const float* values;        /* device [nnz]   "<fg>.values"   */
  const int32_t* segments;    /* device [batch] "<fg>.segments": ids per sample (counts, not offsets) */
  int64_t* offsets;           /* device [batch+1] scratch: exclusive scan of segments (written by
                                 bz_segments_to_offsets_slots, read by bz_embed_pool); NULL = fused scan */
  void* out;                  /* device: block base + this item's column offset */
  int64_t rows;
  int64_t out_stride;         /* elements between consecutive samples of the block */
  int64_t nnz;                /* elements of ids / values (SparsePullerInput::key_size).  The kernels never read ids or
                                 values at or beyond nnz: a negative count is taken as 0 and running offsets stop at
                                 nnz, so counts that disagree with the arrays cannot send a read outside them */
  uint32_t hash_bucket_size;
  int32_t pitch;              /* bytes between table rows */
  int32_t dim;
  int32_t table_dtype;        /* BZ_F32 | BZ_F16 | BZ_I8 */
  int32_t out_dtype;          /* BZ_F32 | BZ_F16 */
  int32_t udf;                /* bz_udf */
  int32_t trunc_dir;          /* bz_trunc, BZ_ASSIGN only */
  int32_t trunc_num;          /* BZ_ASSIGN only */
  int32_t batch;
  int32_t wg_begin;           /* filled by bz_embed_plan: first workgroup of this slot */
  int32_t wg_count;           /* filled by bz_embed_plan */
  int32_t scale_pitch;        /* bytes between the scales of consecutive rows; 0 = 4 (a dense float array) */
  int32_t assign_pitch;       /* BZ_ASSIGN only: elements between consecutive positions of a sample; 0 = dim (the
                                 positions of a sample are contiguous, udf_processor.h:103-131).  A larger pitch lets
                                 several items share the rows of one [batch, trunc_num, sum of dims] tensor, each
                                 writing its own columns */
  int32_t reserved_;
} bz_embed_slot;

/*
 * Row pitch in bytes that keeps rows inside 128-byte lines: row_bytes rounded up to 16, then to the next power of two
 * when that is at most 128, or to a multiple of 128 when that costs at most a third more memory.  scale_bytes (0 or 4)
 * is room for a per-row scale stored behind the row's elements (int8 tables), at byte offset
 * round_up(row_bytes, 4) of the row.
 */
BZ_API int32_t bz_table_pitch(int64_t row_bytes, int scale_bytes);

/*
 * Launch geometry of one Embedding invocation, produced on the host by bz_embed_plan
 * and handed back to bz_embed_pool.  No reference counterpart.
 */
typedef struct bz_embed_launch {
  int32_t n_slots;
  int32_t total_wg;     /* workgroups over all slots */
  int32_t wg_per_slot;  /* > 0 when every slot takes the same number of workgroups, else 0 */
  int32_t variant;      /* 0 = generic kernel; else (table_dtype << 8) | lanes_per_row: the specialised
                           ksum/kavg kernel (all slots share dtype, row width class and are sum/avg) */
  int32_t fused_scan;   /* 1: no slot carries offsets; the pooling kernel scans the segments itself */
  int32_t scan_first;   /* advice, set with fused_scan: 1 when so many workgroups per slot would each re-read the counts
                           before their first sample (batch * workgroups * 2 bytes per slot) that scanning once into
                           slot.offsets (bz_segments_to_offsets_slots) and planning again is the cheaper way */
  int32_t max_batch;    /* largest slot.batch of the planned slots */
  int32_t reserved_;
} bz_embed_launch;

/*
 * Host-side planning: validates the slots (host copy), fills wg_begin/wg_count and
 * the launch record.  The caller then copies the slot array to the device.
 * A slot with offsets == NULL asks for the fused scan (the pooling kernel derives
 * each workgroup's offsets from the segments itself; sensible up to a few
 * thousand samples); either all slots carry offsets or none does.
 */
BZ_API int bz_embed_plan(bz_embed_slot* slots_host, int n_slots, bz_embed_launch* launch);

/*
 * segments -> offsets for one array: off[i] = sum(segments[0..i)), off[n] = nnz.
 * Stands in for the pointer walk `key += num; value += num` of
 * QuickEmbeddingDict::Get (blaze/store/quick_embedding/quick_embedding_dict.cc:111-140).
 * n <= 2^24.
 */
BZ_API int bz_segments_to_offsets(const int32_t* segments_dev, int64_t* offsets_dev, int64_t n, bz_stream_t stream);

/* the same scan for every slot of a descriptor array in ONE launch (slot.segments -> slot.offsets) */
BZ_API int bz_segments_to_offsets_slots(const bz_embed_slot* slots_dev, int n_slots, bz_stream_t stream);

/*
 * Gather + pool every slot in ONE launch.  Stands in for SparsePuller::Get as the
 * Embedding operator calls it (blaze/operator/sparse_op/embedding/embedding_op.h:243)
 * = QuickEmbeddingDict::Get (quick_embedding_dict.cc:76-148) over the
 * K{Sum,Avg,Assign}Processors (udf_processor.h:43-133), including the per-item
 * zero fill (InitProcess).  fp32 accumulate, multiply then add (not fused), ids in
 * order: the fp32 output is bit-identical to the reference's loop.
 * Unless launch->fused_scan, slots_dev must already hold offsets
 * (bz_segments_to_offsets_slots on the same stream).
 */
BZ_API int bz_embed_pool(const bz_embed_slot* slots_dev, const bz_embed_launch* launch, bz_stream_t stream);

/*
 * The same launch with the slot records handed over as kernel arguments instead of read from device memory (one trip
 * to memory fewer at the head of every workgroup, and no device copy of the records to keep).  slots_host: the records
 * bz_embed_plan saw, in host memory; they are copied into the launch.  Takes plans with the scan fused in
 * (launch->fused_scan, no slot bringing offsets) and at most BZ_EMBED_ARG_SLOTS slots of one row shape
 * (launch->variant != 0) or at most 16 mixed ones (kassign items, several dims or dtypes); otherwise BZ_ENOTSUP and nothing is launched -- call bz_embed_pool with a
 * device copy then.  Same results bit for bit.
 * Reference: as bz_embed_pool.
 */
#define BZ_EMBED_ARG_SLOTS 26 /* 26 records of 152 bytes + the other arguments fit the 4 KB kernel-argument segment */
BZ_API int bz_embed_pool_args(const bz_embed_slot* slots_host, const bz_embed_launch* launch, bz_stream_t stream);

/*
 * bz_segments_to_offsets_slots + bz_embed_pool for callers that cannot allocate: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  The offsets of every slot (the scan
 * scratch that slot.offsets otherwise brings in; slot.offsets is ignored here) live in a buffer of
 * BZ_EMBED_STATIC_SCRATCH_BYTES inside the library, one per GPU, held until the process ends.  The call makes two
 * launches on `stream` (scan of every slot's segments into that buffer, then the pooling kernel the plan chose reading
 * its offsets from there) and calls no hipMalloc / hipFree or other allocating routine.  Results are those of the
 * two-call form, bit for bit.
 * Limit: n_slots * (launch->max_batch + 1) * 8 bytes must fit the buffer, else BZ_EINVAL (config 5, 200 slots x batch
 * 8192, takes 13.1 MB).  All calls on one GPU share the one buffer: calls whose launches may overlap on the device
 * (different streams, no ordering between them) race on it; calls on one stream, or ordered by events, do not.
 * The first call on a device looks the buffer's address up (hipGetSymbolAddress, which may load the library's code on
 * that device): make one call per device outside any stream capture before relying on it there.
 */
#define BZ_EMBED_STATIC_SCRATCH_BYTES (16u << 20)
BZ_API int bz_embed_pool_static_scratch(const bz_embed_slot* slots_dev, const bz_embed_launch* launch, bz_stream_t stream);

/* name of the pooling kernel as profilers report it (for tooling) */
BZ_API const char* bz_embed_pool_kernel_name(void);

/* ------------------------------------------------------------------------- */
/* Dense                                                                      */
/* ------------------------------------------------------------------------- */

enum bz_act {
  BZ_ACT_NONE = 0,
  BZ_ACT_PRELU = 1,      /* blaze/operator/op/prelu_op.cc:11-30: y = x*((x>0)+(x<0)*w[n % act_size]) */
  BZ_ACT_DICE = 2,       /* blaze/operator/op/dice_op.cc:15-34 */
  BZ_ACT_LEAKY_RELU = 3, /* blaze/operator/op/leaky_relu_op.cc:15-21: x>=0 ? x : act_alpha*x */
  BZ_ACT_SIGMOID = 4,    /* blaze/operator/op/sigmoid_op.cc:15-21: e^x/(1+e^x) */
  BZ_ACT_SOFTMAX = 5     /* blaze/operator/op/softmax_op.cc:21-78 over the N axis; N <= 64 only */
};

/*
 * Y[M,N] = act( alpha * A[M,K] * W + beta * bias )
 * = Gemm op (blaze/operator/op/gemm_op.h:33-107: Y <- broadcast(C); Y = alpha*op(A)op(B) + beta*Y)
 * followed by the separate PRelu / Dice / LeakyRelu / Sigmoid / Softmax op the
 * importer emits after it (blaze/model_importer/ulf_importer.cc:661-782).
 *
 * A is row major with leading dimension lda (elements).  W is the weight in the
 * PACKED layout [N, ldw] = K contiguous per output column (the reference's
 * transB=true form); bz_fc_pack_weight produces it from either form.  A 3-D
 * Gemm with a shared weight (gemm_op.h:52-58,77-91) is the same call with
 * M = batch*M.
 */
struct bz_concat_ew_desc;
/*
 * A second full layer in the launch of an a_pieces layer (bz_fc_desc.next): Z = act(alpha * Y * w^T + beta * bias) with
 * Y the first layer's activated output, rounded to the tensor type as it would have been stored.  With it the
 * descriptor's head_* fields describe a skinny third layer on Z instead of on Y, and both y pointers may be NULL (that
 * tensor is then not stored): the three-layer attention MLP of a DIN model (216 -> 80 -> 40 -> 1 in
 * tools/example_model/din/model/graph_ulf.txt) is one launch that reads q and k and writes the scores.
 */
typedef struct bz_fc_next {
  const void* w;        /* device [n, ldw] packed, K = the first layer's n, dtype in_dtype */
  const float* bias;    /* device [n] or NULL */
  void* y;              /* device [M, ldy], dtype in_dtype, or NULL */
  const float* act_p0;  /* as in bz_fc_desc, for this layer's n columns */
  const float* act_p1;
  const float* act_p2;
  int64_t ldw, ldy;
  int32_t n;            /* 9..64 */
  int32_t act;          /* bz_act but BZ_ACT_SOFTMAX */
  int32_t act_size;
  int32_t dice_nosqrt;
  float alpha, beta, act_alpha;
  int32_t reserved_;
} bz_fc_next;

typedef struct bz_fc_desc {
  const void* a;       /* device [M, lda] */
  const void* w;       /* device [N, ldw] packed */
  const void* bias;    /* device [N] (bias_rows==1) or [M, N] (bias_rows==M) or NULL; same dtype as out_acc_dtype F32 */
  void* y;             /* device [M, ldy] */
  const float* act_p0; /* PRELU: slope [act_size]; DICE: gamma [N] */
  const float* act_p1; /* DICE: mean [N] */
  const float* act_p2; /* DICE: var [N] */
  int64_t lda, ldw, ldy;
  int32_t m, n, k;
  int32_t in_dtype;    /* BZ_F16 | BZ_BF16 | BZ_F32: type of a and w */
  int32_t out_dtype;   /* BZ_F16 | BZ_BF16 | BZ_F32 */
  int32_t bias_rows;   /* 0 none, 1 = [N] broadcast over rows, m = full [M,N] */
  int32_t act;         /* bz_act */
  int32_t act_size;    /* PRELU slope count (1 or N) */
  int32_t dice_nosqrt; /* DICE: divide by var instead of sqrt(var+1e-8) */
  float alpha, beta;
  float act_alpha;     /* LEAKY_RELU slope */
  int32_t reserved_;
  /*
   * Optional second, skinny layer in the same launch (head_n > 0): Z[M, head_n] = head_act(Y * head_w^T + head_bias),
   * computed from the rounded tile of Y while it is still on chip -- the Gemm -> activation -> Gemm(N <= 8) ->
   * Softmax | Sigmoid tail of a CTR tower without the second launch.  Needs 8 < n <= 256 (a workgroup owns whole rows
   * of Y), out_dtype == in_dtype, 16-byte aligned operand rows.  y may be NULL then (Y is not stored).
   */
  const void* head_w;     /* device [head_n, head_ldw], K (= n) contiguous, dtype in_dtype */
  const float* head_bias; /* device [head_n] or NULL */
  void* head_y;           /* device [M, head_ldy] */
  int64_t head_ldw, head_ldy;
  int32_t head_n;         /* 0 = no head, else 1..8 */
  int32_t head_act;       /* BZ_ACT_NONE | BZ_ACT_SIGMOID | BZ_ACT_SOFTMAX */
  int32_t head_out_dtype; /* BZ_F32 | BZ_F16 | BZ_BF16 */
  /*
   * P sibling layers that share A in one launch (FusedParallelGemm, blaze/operator/fused_op/fused_parallel_gemm_op.h:
   * 115-129: GemmStridedBatched with stride_a = 0): W holds the P weights one after the other ([P * n_split, ldw]), n =
   * P * n_split, bias / activation parameters are [n] (slice after slice), and slice p's output is the matrix
   * [M, n_split] with row pitch ldy at y + p * y_split_stride (elements).  A full bias (bias_rows == m) is [P, M, n_split].
   * n_split == 0: a single layer.  No head and no softmax with split outputs.
   */
  int32_t n_split;
  int64_t y_split_stride;
  /* A given as pieces computed on the fly instead of as a stored matrix: when non-NULL, `a` and `lda` are ignored and
   * row r of A is the concatenation bz_concat_ew would write for that row (m = r0 * r1 rows, k = the sum of the widths;
   * dst / dst_pitch of the descriptor are not used).  The layer then reads the pieces' operands and the tensor is never
   * stored: DIN's attention input [q, k, q-k, q*k] (tools/example_model/din/model/graph_ulf.txt) costs its 22 MB of
   * traffic each way otherwise.  Same values as the two-step form: every element of A is rounded to the tensor type
   * exactly as the concat would store it.  Limits: 2-byte types, pieces of one width that do not divide,
   * k <= 224, n <= 96, no head (but see next), no split outputs, per-column bias only; BZ_ENOTSUP (nothing launched)
   * otherwise. */
  const struct bz_concat_ew_desc* a_pieces;
  /* with a_pieces only: a second layer (and, through head_*, a skinny third) in the same launch; out_dtype == in_dtype */
  const bz_fc_next* next;
} bz_fc_desc;

BZ_API int bz_fc_fused(const bz_fc_desc* desc, bz_stream_t stream);

/*
 * Repack a Blaze weight blob for bz_fc_fused: src is [K,N] (trans_b=0) or [N,K]
 * (trans_b=1) row major in src_dtype (F32 or F16); dst is [N, ldw] in dst_dtype
 * with zero fill between K and ldw.  fp32 -> fp16 narrows with round-to-nearest-
 * even like the reference's ConstantFill (blaze/common/proto_helper.cc:174,
 * blaze/common/types.h:78-80).  ldw must be a multiple of 8 elements.
 */
BZ_API int bz_fc_pack_weight(const void* src_dev, int src_dtype, int trans_b, int k, int n, void* dst_dev, int dst_dtype,
                             int64_t ldw, bz_stream_t stream);


/*
 * Strided-batched C[i] = alpha*op(A[i])*op(B[i]) + beta*C[i], row major, element
 * strides (0 = operand shared by the whole batch).  Stands in for
 * GemmStridedBatched (blaze/math/gemm.cc:82-139 / gemm.cu:251-336) as reached from
 * MatMul (blaze/operator/op/matmul_op.h:77-89 via BroadcastGemm_NxN,
 * blaze/math/broadcast.h:157-222), FusedParallelGemm
 * (blaze/operator/fused_op/fused_parallel_gemm_op.h:96-129) and
 * FusedParallelMatMul (fused_parallel_matmul_op.h:36-93).  The DIN attention
 * weighted sum is the case M=1, K=T, N=D.
 */
typedef struct bz_bgemm_desc {
  const void* a;
  const void* b;
  void* c;
  int64_t stride_a, stride_b, stride_c;
  int32_t trans_a, trans_b;
  int32_t m, n, k;
  int32_t batch;
  int32_t dtype;     /* BZ_F32 | BZ_F16 for a, b, c alike (fp32 accumulate) */
  float alpha, beta;
} bz_bgemm_desc;

BZ_API int bz_gemm_strided_batched(const bz_bgemm_desc* desc, bz_stream_t stream);

/*
 * The tail of a DIN attention block in one launch:
 *   att[b, c] = sum_t (w[b, t] * mask[b, t]) * x[b, t, c]        sum[b, c] = sum_t x[b, t, c]
 * i.e. Mul (blaze/operator/op/elementwise_op.h:154-163), MatMul with transA on [B, T, 1] x [B, T, C]
 * (matmul_op.h:77-89) and ReduceSum over axis 1 (reduce_sum_op.h:18-66) as the reference
 * runs them one after the other; the product w * mask is rounded to the tensor type
 * before it is used, as the Mul operator's output would be, and both sums add in
 * ascending t, so the outputs equal the three operators' bit for bit.
 * mask null: w is used as it is.  att null or sum null: that output is not computed.
 * Extension for the Concat that usually follows (DIN joins [target, sum, att] for its main MLP, concat_op.cu:33): att
 * and sum may be rows of a wider matrix (ld_att / ld_sum elements between rows; 0 = c), and one more piece of copy_c
 * elements per item is copied alongside, copy_dst[b, 0..copy_c) = copy_src[b, 0..copy_c), so that the three column
 * ranges of the Concat's output are written by this launch and the Concat has nothing left to do.
 */
typedef struct bz_weighted_pool_desc {
  const void* w;     /* [batch, t] */
  const void* mask;  /* [batch, t] or null */
  const void* x;     /* [batch, t, c] */
  void* att;         /* [batch, c] or null */
  void* sum;         /* [batch, c] or null */
  int64_t batch;
  int32_t t, c;
  int32_t dtype;     /* BZ_F32 | BZ_F16 for all of them */
  int32_t copy_c;    /* elements per item of the copied piece; 0 = none */
  int64_t ld_att, ld_sum;           /* elements between the rows of att / sum; 0 = c */
  const void* copy_src;             /* [batch, copy_c] at ld_copy_src, or null */
  void* copy_dst;                   /* [batch, copy_c] at ld_copy_dst */
  int64_t ld_copy_src, ld_copy_dst; /* elements between rows; 0 = copy_c */
} bz_weighted_pool_desc;

BZ_API int bz_weighted_pool(const bz_weighted_pool_desc* desc, bz_stream_t stream);

/*
 * Standalone activation ops over a [rows, cols] fp32 or fp16 tensor (in place
 * allowed), for graphs where the producer is not a Gemm.  Same formulas and
 * reference citations as bz_act above.
 */
typedef struct bz_act_desc {
  const void* x;
  void* y;
  const float* p0;
  const float* p1;
  const float* p2;
  int64_t rows, cols;
  int32_t dtype;
  int32_t act;
  int32_t act_size;
  int32_t dice_nosqrt;
  float act_alpha;
  int32_t reserved_;
} bz_act_desc;

BZ_API int bz_activation(const bz_act_desc* desc, bz_stream_t stream);

/*
 * Concatenate up to BZ_CONCAT_MAX row-major 2-D pieces side by side in ONE launch:
 * dst[r, col_k .. col_k + width_k) = src_k[r, 0 .. width_k), widths in bytes.  Stands in for Concat along the
 * last axis (blaze/operator/op/concat_op.cu:33), the op that joins the dense features with the embedding block
 * in CTR graphs.
 */
#define BZ_CONCAT_MAX 16
typedef struct bz_concat_desc {
  const void* src[BZ_CONCAT_MAX];
  int64_t width[BZ_CONCAT_MAX];     /* bytes per row of each piece */
  int64_t src_pitch[BZ_CONCAT_MAX]; /* bytes between rows of each piece; 0 repeats its one row for every output row
                                       (Fuse, blaze/operator/op/fuse_op.cc:11-33) */
  void* dst;
  int64_t dst_pitch;            /* bytes per output row */
  int64_t rows;
  int32_t n;
  int32_t reserved_;
} bz_concat_desc;

BZ_API int bz_concat_cols(const bz_concat_desc* desc, bz_stream_t stream);

/*
 * Elementwise ops with multidirectional broadcasting, the shape rule of blaze/math/broadcast.h:39-67:
 * Add / Sub / Mul / Div (blaze/operator/op/elementwise_op.cc:28-165, elementwise_op.cu:55-140),
 * BroadcastTo (elementwise_op.h:193-226) and Where (elementwise_op.h:228-283; condition int32 | int64, nonzero
 * picks x).  Operands are described by element strides over the OUTPUT's dims (0 on a broadcast dim), so any
 * operand layout that is a strided view works.  One fp32 operation per element; fp16 / bf16 tensors are widened,
 * computed in fp32 and rounded once.
 */
#define BZ_MAX_RANK 6
typedef enum bz_ew_op { BZ_EW_ADD = 0, BZ_EW_SUB = 1, BZ_EW_MUL = 2, BZ_EW_DIV = 3, BZ_EW_ASSIGN = 4, BZ_EW_WHERE = 5 } bz_ew_op;
typedef struct bz_bcast_desc {
  const void* a;    /* first operand; the condition for BZ_EW_WHERE */
  const void* b;    /* second operand (unused by BZ_EW_ASSIGN); x for BZ_EW_WHERE */
  const void* c;    /* y for BZ_EW_WHERE, else unused */
  void* out;        /* contiguous, row major over dims[] */
  int64_t dims[BZ_MAX_RANK];
  int64_t a_stride[BZ_MAX_RANK];
  int64_t b_stride[BZ_MAX_RANK];
  int64_t c_stride[BZ_MAX_RANK];
  int32_t rank;
  int32_t op;       /* bz_ew_op */
  int32_t dtype;    /* BZ_F32 | BZ_F16 | BZ_BF16: type of the value operands and of out */
  int32_t cond_dtype; /* BZ_I32 | BZ_I64 (BZ_EW_WHERE) */
} bz_bcast_desc;

BZ_API int bz_broadcast_op(const bz_bcast_desc* desc, bz_stream_t stream);

/*
 * Concat along the last axis whose pieces are computed on the fly: piece p is x[p] (BZ_EW_ASSIGN, a copy or a
 * row-broadcast), or x[p] (op) y[p] for Add / Sub / Mul / Div.  One launch stands in for the reference's sequence
 * BroadcastTo / Sub / Mul / ... followed by Concat (blaze/operator/op/elementwise_op.cu:55-140, concat_op.cu:33), the
 * way a DIN attention unit assembles [q, k, q-k, q*k] (tools/example_model/din/model/graph_ulf.txt), without writing
 * the intermediate tensors.  Each element is computed exactly as the separate operators do (fp32 operation on the
 * widened operands, rounded once to dtype).
 * Rows are indexed by two coordinates, row = i0 * r1 + i1; an operand's element (row, c) is at
 * base[i0 * stride[0] + i1 * stride[1] + c] (stride 0 = broadcast over that coordinate), c < width[p].
 */
#define BZ_CEW_MAX 8
typedef struct bz_concat_ew_desc {
  const void* x[BZ_CEW_MAX];
  const void* y[BZ_CEW_MAX];          /* NULL for BZ_EW_ASSIGN */
  int64_t x_stride[BZ_CEW_MAX][2];    /* in elements */
  int64_t y_stride[BZ_CEW_MAX][2];
  int32_t op[BZ_CEW_MAX];             /* BZ_EW_ADD | SUB | MUL | DIV | ASSIGN */
  int32_t width[BZ_CEW_MAX];          /* columns of the piece */
  void* dst;                          /* [r0 * r1, dst_pitch] */
  int64_t dst_pitch;                  /* elements per output row, >= sum of the widths */
  int64_t r0, r1;
  int32_t n;                          /* pieces, 1..BZ_CEW_MAX */
  int32_t dtype;                      /* BZ_F32 | BZ_F16 | BZ_BF16 */
} bz_concat_ew_desc;

BZ_API int bz_concat_ew(const bz_concat_ew_desc* desc, bz_stream_t stream);

/*
 * ReduceSum over the middle axis of a contiguous [outer, dim, inner] tensor -> [outer, inner], added in ascending
 * order of the axis like blaze/math/reduce.cc:13-29 (fp32 accumulate; bit-exact for fp32 tensors).
 */
BZ_API int bz_reduce_sum(const void* x, void* y, int64_t outer, int64_t dim, int64_t inner, int dtype, bz_stream_t stream);

/*
 * BatchNormalization, inference form (blaze/operator/op/batch_normalization_op.cc:11-18):
 * y = gamma[c] * (x - mean[c]) / (nosqrt ? var[c] : sqrtf(var[c] + eps)) + beta[c], c = flat index % channels.
 * Parameters are fp32 vectors of `channels` elements.
 */
typedef struct bz_bn_desc {
  const void* x;
  void* y;
  const float* gamma;
  const float* beta;
  const float* mean;
  const float* var;
  int64_t size;
  int64_t channels;
  int32_t dtype;  /* BZ_F32 | BZ_F16 | BZ_BF16 */
  int32_t nosqrt;
  float eps;
  int32_t reserved_;
} bz_bn_desc;

BZ_API int bz_batch_norm(const bz_bn_desc* desc, bz_stream_t stream);

/*
 * Softmax over the middle axis of a contiguous [outer, c, inner] tensor (blaze/operator/op/softmax_op.cc:21-78:
 * max-subtracted, exp, sum in ascending order of the axis, divide).  inner == 1 is the row softmax of bz_activation.
 */
BZ_API int bz_softmax_axis(const void* x, void* y, int64_t outer, int64_t c, int64_t inner, int dtype, bz_stream_t stream);

/*
 * Gather along one axis of a contiguous [outer, axis_size, inner] tensor: y[o, j, :] = data[o, indices[j], :] for j <
 * n_indices, rows of inner_bytes bytes (blaze/operator/op/gather_op.h:25-87, gather_op.cc:9-21: one memcpy per index).
 * indices are BZ_I32 or BZ_I64 (ID_TYPE_SWITCH there).  An index outside [0, axis_size), which the reference's memcpy
 * would read out of bounds, gives a row of zeros.
 */
BZ_API int bz_gather_rows(const void* data, const void* indices, int index_dtype, void* y, int64_t outer, int64_t axis_size,
                          int64_t inner_bytes, int64_t n_indices, bz_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* BLAZE_HIP_H_ */
