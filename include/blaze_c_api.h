/*
 * blaze_c_api.h -- the public C ABI of the predictor, entry point for entry point the one the reference
 * exports from blaze/api/c_api/c_api_predictor.h:16-105 and c_api_error.h (what its ctypes binding
 * blaze/binding/python/pyblaze loads).  Conventions kept: opaque void* handles; every call returns 0 on
 * success and -1 on failure; the message of the last failure is thread local (Blaze_GetLastErrorString,
 * c_api_error.cc:12-28); name / shape arrays returned by the List*Names, ParamName, *Shape calls point into
 * thread-local or predictor-owned storage and stay valid until the next such call on that thread / predictor;
 * Blaze_PredictorOutput copies into caller memory; Blaze_PredictorFeed copies `len` bytes in and requires
 * len == element count * sizeof(dtype).  A Predictor is not thread safe: one per serving thread.
 *
 * device_type for Blaze_PredictorCreate: 1 = the accelerator (MI355X), the value existing callers pass for
 * the GPU; -1 = probe; 0 (CPU) fails at operator creation: this build has no CPU execution path.
 *
 * Not provided by this build (they return -1 with a message): the model importers
 * (Blaze_PredictorManagerLoadDeepNetModel, Blaze_ConvertBlaze).  Blaze_OptimizeBlaze runs the two optimizer passes that
 * concern this path's FC layers, the in-order Gemm -> Gemm folding
 * (blaze/graph/pattern/in_order/gemm_gemm_fusion_pattern_impl.cc) and the parallel-Gemm fusion
 * (blaze/graph/pattern/in_parallel/parallel_gemm_fusion_pattern_impl.cc), and writes the model back; the reference's
 * other passes are not part of this build.  The text-to-QED table builders of
 * c_api_qed.h (Blaze_QuickEmbeddingBuildFp32/Fp16) are provided.
 */
#ifndef BLAZE_C_API_H_
#define BLAZE_C_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BLAZE_API __attribute__((visibility("default")))

typedef void* PredictorManagerHandle;
typedef void* PredictorHandle;

/* c_api_error.h */
BLAZE_API void Blaze_GetLastErrorString(const char** msg);
BLAZE_API void Blaze_SetLastErrorString(const char* format, ...);

/* c_api_predictor.h:19-24 -- accepted and ignored: request batching is outside this build */
BLAZE_API int Blaze_InitScheduler(int enable_batching, int max_batch_size, int batch_timeout_micros, int num_threads_for_cpu,
                                  int num_threads_for_cuda, int num_threads_for_pipe);

/* c_api_predictor.h:27-42 */
BLAZE_API int Blaze_PredictorManagerCreate(PredictorManagerHandle* handle);
BLAZE_API int Blaze_PredictorManagerDelete(PredictorManagerHandle handle);
BLAZE_API int Blaze_PredictorManagerSetDataType(PredictorManagerHandle handle, int data_type);
BLAZE_API int Blaze_PredictorManagerSetRunMode(PredictorManagerHandle handle, const char* run_mode);
BLAZE_API int Blaze_LoadSparseModelWeight(PredictorManagerHandle handle, const char* sparse_model_weight_file);
/* (sic) the reference spells it Predcitor; both spellings are exported */
BLAZE_API int Blaze_PredcitorManagerLoadModel(PredictorManagerHandle handle, const char* blaze_model_file, int optimization_pass);
BLAZE_API int Blaze_PredictorManagerLoadModel(PredictorManagerHandle handle, const char* blaze_model_file, int optimization_pass);
BLAZE_API int Blaze_PredictorManagerLoadDeepNetModel(PredictorManagerHandle handle, const char* deepnet_conf_file,
                                                     const char* deepnet_param_file, int optimization_pass);

/* c_api_predictor.h:45-49 */
BLAZE_API int Blaze_PredictorCreate(PredictorManagerHandle predictor_mgr, int device_type, int device_id, PredictorHandle* handle);
BLAZE_API int Blaze_PredictorDelete(PredictorHandle handle);

/* c_api_predictor.h:53-61 */
BLAZE_API int Blaze_PredictorReshapeInput(PredictorHandle handle, const char* name, const int* data, int num);
BLAZE_API int Blaze_PredictorFeed(PredictorHandle handle, const char* name, void* data, int len);
BLAZE_API int Blaze_PredictorForward(PredictorHandle handle);

/* c_api_predictor.h:64-74 */
BLAZE_API int Blaze_PredictorOutputShape(PredictorHandle handle, const char* name, size_t* ndim, size_t** shape);
BLAZE_API int Blaze_PredictorOutputDataType(PredictorHandle handle, const char* name, int* data_type);
BLAZE_API int Blaze_PredictorOutput(PredictorHandle handle, const char* name, void* data, size_t len);

/* c_api_predictor.h:77-90 */
BLAZE_API int Blaze_PredictorParamName(PredictorHandle handle, size_t* ndim, const char*** name);
BLAZE_API int Blaze_PredictorParamShape(PredictorHandle handle, const char* name, size_t* ndim, size_t** shape);
BLAZE_API int Blaze_PredictorParamDataType(PredictorHandle handle, const char* name, int* data_type);
BLAZE_API int Blaze_PredictorParam(PredictorHandle handle, const char* name, void* data, size_t len);

/* c_api_predictor.h:93-98 */
BLAZE_API int Blaze_PredictorListInputNames(PredictorHandle handle, size_t* ndim, const char*** names);
BLAZE_API int Blaze_PredictorListOutputNames(PredictorHandle handle, size_t* ndim, const char*** names);

/* c_api_predictor.h:101-107 -- observer "profile": per-operator host wall time as chrome-trace JSON */
BLAZE_API int Blaze_PredictorRegisterObservers(PredictorHandle handle, size_t ndim, const char** names);
BLAZE_API int Blaze_PredictorDumpObservers(PredictorHandle handle, size_t* ndim, const char*** key, const char*** value);

/* c_api_blaze_converter.h:11-20 / c_api_blaze_optimizer.h: importers and optimizer passes are not part of this
 * build; both return -1 with a message */
BLAZE_API int Blaze_ConvertBlaze(const char* model_conf_file, const char* model_data_file, int model_type, int weight_type,
                                 int io_type, int x_type_num, const char** x_type_key, const int* x_type_value,
                                 const char* blaze_model_file, int binary);
/* c_api_blaze_optimizer.h:12-14: model file (binary or text NetDef) -> optimized model file (binary != 0: wire format) */
BLAZE_API int Blaze_OptimizeBlaze(const char* raw_model_file, const char* optimized_model_file, int binary);
/* c_api_qed.h:13-21: text tables (meta file + per-table files under `path`) -> one QED file, fp32 or fp16 rows */
BLAZE_API int Blaze_QuickEmbeddingBuildFp32(const char* path, const char* meta, const char* output_file, int thread_num);
BLAZE_API int Blaze_QuickEmbeddingBuildFp16(const char* path, const char* meta, const char* output_file, int thread_num);

/* ---- extensions (no reference counterpart) ------------------------------------------------------------ */

/*
 * Register an in-memory table with the manager's device store (created on demand as "qed_hip_sparse_puller")
 * instead of loading a QED file: synthetic benchmarks, tables generated on the device, int8 tables with a
 * per-row fp32 scale (a storage format the reference's QED reader rejects, blaze/store/defines.h:29-50).
 * value_type: 1 fp32, 12 fp16, 7 int8.  rows_ptr: [rows, dim] row major, device memory when on_device else
 * host memory.  keys: host int64[rows] or NULL (ids are row numbers).  scale: [rows] fp32, same place as rows_ptr.
 */
BLAZE_API int Blaze_HipStoreAddTable(PredictorManagerHandle handle, const char* table_name, int value_type, int64_t rows, int dim,
                                     const void* rows_ptr, int on_device, const int64_t* keys, const float* scale);

/*
 * One feature group looked up through the store's host-memory SparsePuller::Get, the form the reference's interface
 * declares (blaze/store/sparse_puller.h:77-83) and its host Embedding operator calls (embedding_op.cc:87): keys [sum of
 * key_num] int64, key_num [batch] int32, values [sum of key_num] fp32 and every out[k] are HOST memory.  Item k pools
 * with udf_type[k] (0 sum, 1 avg, 2 assign) / trunc_direction[k] / trunc_num[k] and writes dim (assign: trunc_num * dim)
 * elements of out_type (1 fp32, 12 fp16) per sample at out[k] + sample * stride[k]; other columns of the block, and
 * every column when the table name is unknown, keep what the caller put there.  The tables live on the device: the
 * call copies the inputs over, runs the pooling kernel, copies the columns back and waits.
 */
BLAZE_API int Blaze_HipStoreGet(PredictorManagerHandle handle, const char* table_name, const int64_t* keys, const int32_t* key_num,
                                size_t batch, const float* values, int dim, int n_items, const int* udf_type,
                                const int* trunc_direction, const int* trunc_num, void* const* out, const size_t* stride,
                                int out_type);

/* load a model from memory: a NetDef in protobuf text format (is_text) or proto2 wire format */
BLAZE_API int Blaze_PredictorManagerLoadModelFromString(PredictorManagerHandle handle, const char* data, size_t len, int is_text);

/*
 * NetDef text format <-> proto2 wire format, for tools without a protobuf toolchain.  Writes at most cap bytes
 * to out (may be NULL to query the size) and the full size to *out_len.
 */
BLAZE_API int Blaze_ConvertNetDef(const char* in, size_t len, int in_is_text, int out_is_text, char* out, size_t cap, size_t* out_len);

/* device address of an input / output blob after ReshapeInput / Forward, for callers that keep inputs on the device */
BLAZE_API int Blaze_PredictorInputDevicePtr(PredictorHandle handle, const char* name, void** ptr);
BLAZE_API int Blaze_PredictorOutputDevicePtr(PredictorHandle handle, const char* name, void** ptr);

/* Blaze_PredictorFeed for `count` inputs in one call (a sparse model has three inputs per feature group).  The shapes
 * must have been set (ReshapeInput).  Inputs that are plain device tensors are staged side by side and travel in one
 * transfer; the predictor's input tensors then view slices of that one device buffer. */
BLAZE_API int Blaze_PredictorFeedMany(PredictorHandle handle, int count, const char* const* names, const void* const* data,
                                      const size_t* lens);

/* number of device and pinned-host allocations the library has made for blobs, feed arenas and Embedding scratch in
 * this process so far (no counterpart in the reference): unchanged across a stretch of requests = that stretch
 * allocated nothing */
BLAZE_API int Blaze_AllocationCount(int64_t* count);

/* run Forward `count` times on the calling thread (benchmark loops without per-call host overhead) */
BLAZE_API int Blaze_PredictorForwardN(PredictorHandle handle, int count);

/*
 * Forward in two halves (no counterpart in the reference, whose Forward is synchronous): ForwardLaunch queues the whole
 * pass on the calling thread's stream and returns, ForwardWait (same thread) returns once that pass has finished on
 * the device.  A thread that owns several predictors can so keep more than one pass queued.  Between the two calls the
 * predictor must not be fed, read or launched again.
 */
BLAZE_API int Blaze_PredictorForwardLaunch(PredictorHandle handle);
BLAZE_API int Blaze_PredictorForwardWait(PredictorHandle handle);

/*
 * A pool of serving threads (no counterpart in the reference's C API; its C++ example runs one loop per thread,
 * blaze/example/cpp/predictor_example.cc).  Blaze_ServePoolRun runs `steps` forward passes: pass i runs predictor
 * i % n_predictors on thread i % n_threads, and returns when all of them have finished on the device.  n_predictors
 * must be a multiple of the pool's thread count so that a predictor only ever runs on one thread.  A thread keeps up
 * to `depth` passes (default 2; 1 = plain synchronous Forward calls) of different predictors queued on its stream,
 * launching the next before it waits for the oldest; it needs that many predictors per thread to do so.
 */
typedef void* ServePoolHandle;
BLAZE_API int Blaze_ServePoolCreate(int n_threads, ServePoolHandle* handle);
BLAZE_API int Blaze_ServePoolRun(ServePoolHandle handle, PredictorHandle* predictors, int n_predictors, int64_t steps);
BLAZE_API int Blaze_ServePoolSetDepth(ServePoolHandle handle, int depth);
/*
 * What every pass of the last Blaze_ServePoolRun took on its thread, from the start of its launch to the return of its
 * wait, in milliseconds: the latency of a request under that job's load (the reference's example times each Forward
 * inside its serving loop, blaze/example/cpp/predictor_example.cc:129-140).  Writes at most `capacity` values, thread
 * after thread, and the number there are to *count.
 */
BLAZE_API int Blaze_ServePoolLatencies(ServePoolHandle handle, float* out_ms, int64_t capacity, int64_t* count);
/*
 * The pool creates its threads' streams itself, at its first job, and spreads them evenly over the device's hardware
 * queues (the runtime serves few of them, 4 by default, and would otherwise hand a new stream the queue that the fewest
 * streams of the whole process use, idle ones included: eight threads can end up 3-3-1-1 and run at the pace of the
 * threads that share).  Which streams share a queue is measured: a kernel queued behind a busy stream of the same queue
 * cannot finish before it.  This call reports the result: queue_of_thread[t] = the queue (numbered in order of
 * discovery) of thread t's stream; *count = the number of threads, 0 before the first job.
 */
BLAZE_API int Blaze_ServePoolStreamQueues(ServePoolHandle handle, int* queue_of_thread, int capacity, int* count);
BLAZE_API int Blaze_ServePoolDelete(ServePoolHandle handle);

#ifdef __cplusplus
}
#endif
#endif /* BLAZE_C_API_H_ */
