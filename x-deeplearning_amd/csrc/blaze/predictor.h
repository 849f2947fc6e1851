// predictor.h -- the public C++ API: PredictorManager (one model) and Predictor (one serving thread).
//
// Same surface and conventions as the reference's blaze/api/cpp_api/predictor.h:19-286: methods return bool,
// exceptions are caught at this boundary (predictor_impl.cc:172-183), a Predictor is NOT thread safe -- use one
// per thread (predictor.h:90-92) -- while PredictorManager::CreatePredictor is (predictor_manager_impl.cc:121).
// Model formats handled here: the Blaze NetDef (binary or text).  The importers for ULF / ONNX / MXNet /
// TensorFlow / XDL and the offline optimizer are outside this build; asking for them fails with a message.
#pragma once

#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "blaze/graph.h"

namespace blaze {

enum PredictDeviceType { kPDT_Unkown = -1, kPDT_CPU = 0, kPDT_CUDA = 1, kPDT_HIP = 1 };
enum PredictDataType { kPDT_Invalid = -1, kPDT_Float = 1, kPDT_Float16 = 12 };
enum ModelType { kBlaze = 0, kUlf, kOnnx, kMxnet, kTensorFlow, kXDL, kXDLUlf };

using PredictorCallback = std::function<void()>;

// what of the last failure on this thread (the C API appends it to its own message)
std::string& last_error_for_thread();

class Predictor {
 public:
  explicit Predictor(std::shared_ptr<Net> net);
  ~Predictor();
  Predictor(const Predictor&) = delete;
  Predictor& operator=(const Predictor&) = delete;
  bool ReshapeInput(const char* name, const std::vector<size_t>& shape);
  bool ReshapeInput(size_t idx, const std::vector<size_t>& shape);
  // copies len bytes in; len must equal size * sizeof(dtype) (predictor_impl.cc:110-138)
  bool Feed(const char* name, const void* data, size_t len);
  bool Feed(size_t idx, const void* data, size_t len);
  // extension: feed `count` inputs at once.  Inputs that are plain device tensors travel in ONE transfer: they are
  // staged side by side in a pinned arena, copied to a device arena of the same layout, and the input blobs become
  // views of their slices (a model with 26 feature groups has 79 inputs; one queued copy instead of 79).  Other
  // inputs (host tensors, inputs living inside a Concat's output) are fed one by one.
  bool FeedMany(int count, const char* const* names, const void* const* data, const size_t* lens);
  size_t InputSize() const { return external_input_blob_.size(); }
  int InputDataType(const char* name) const;
  const std::vector<std::string>& ListInputName() const { return net_->external_input(); }

  bool Forward(const PredictorCallback&& cb = nullptr);
  // extension: Forward in two halves, so that one thread can keep several of its predictors in flight.
  // ForwardLaunch queues the net on the calling thread's stream and returns; ForwardWait (same thread) returns once
  // that pass has finished on the device.  Feed / Output / another launch on this predictor only after the wait.
  bool ForwardLaunch();
  bool ForwardWait();

  // pointer to a host copy owned by the predictor, valid until the next Output call on it (:194-224)
  bool Output(const char* name, void** data, size_t* len);
  bool Output(size_t idx, void** data, size_t* len);
  const std::vector<size_t>& OutputShape(size_t idx) const;
  const std::vector<size_t>& OutputShape(const char* name) const;
  int OutputDataType(const char* name) const;
  size_t OutputSize() const { return external_output_blob_.size(); }
  const std::vector<std::string>& ListOutputName() const { return net_->external_output(); }

  // model parameters (the ConstantFill blobs)
  std::vector<std::string> ListInternalName() const;
  bool InternalParam(const char* name, void** data, size_t* len);
  const std::vector<size_t>& InternalShape(const char* name) const;
  int InternalDataType(const char* name) const;

  void RegisterObservers(const std::vector<std::string>& observer_names);
  void DumpObservers(std::unordered_map<std::string, std::string>* dump_map);

  // extension: the device this predictor's blobs live on (-1: none of them is on a device)
  int device_id() const;
  // extension: device address of an input / output blob, for callers that fill inputs on the device
  void* InputDevicePtr(const char* name);
  void* OutputDevicePtr(const char* name);

 private:
  int InputName2Idx(const char* name) const;
  int OutputName2Idx(const char* name) const;
  std::shared_ptr<Net> net_;
  std::vector<Blob*> external_input_blob_, external_output_blob_;
  std::unordered_map<std::string, int> input_index_, output_index_;
  std::vector<std::shared_ptr<Blob>> output_cpu_;
  // pinned staging of fed inputs: Feed copies the caller's bytes here and queues the transfer on the thread's
  // stream; Forward runs behind it on the same stream.  feed_pending_[i]: input i's staging is still being read.
  std::vector<std::shared_ptr<Blob>> input_cpu_;
  std::vector<bool> feed_pending_;
  bool any_feed_pending_ = false;
  hipEvent_t feed_done_ = nullptr;  // recorded behind the last queued transfer; Forward's stream waits for it
                                    // (Feed and Forward may be called from different threads = different streams)
  char* arena_host_ = nullptr;         // FeedMany's pinned staging arena and its device twin
  char* arena_dev_ = nullptr;
  size_t arena_cap_ = 0;
  std::vector<void*> retired_arenas_;  // device arenas outgrown while blobs may still view them: freed with the predictor
  hipEvent_t forward_done_ = nullptr;  // recorded behind the last operator of a ForwardLaunch
  void* launched_on_ = nullptr;
  bool forward_in_flight_ = false;
  std::unordered_map<std::string, std::shared_ptr<Blob>> param_cpu_;
};

class PredictorManager {
 public:
  PredictorManager() {}
  void SetDataType(PredictDataType data_type) { data_type_ = data_type; }
  void SetRunMode(const char* run_mode) { run_mode_ = run_mode ? run_mode : ""; }
  bool LoadSparseModelWeight(const char* uri, const char* type = "qed_sparse_puller");
  bool LoadModel(const char* filename, bool optimization_pass = true);
  bool LoadDeepNetModel(const char* model_conf, const char* model_data, bool optimization_pass = true);
  bool LoadModel(const char* conf_file, const char* data_file, ModelType model_type, bool optimization_pass = true);
  // extension: hand over an in-memory NetDef (tests, programmatically built models)
  bool LoadNetDef(const NetDef& net_def);
  Predictor* CreatePredictor(PredictDeviceType predict_device_type = kPDT_Unkown, int device_id = 0);
  // the store shared by all predictors; created by LoadSparseModelWeight or on first use by the extension API
  std::shared_ptr<store::SparsePuller>& sparse_puller() { return sparse_puller_; }
  std::shared_ptr<store::SparsePuller>& EnsureSparsePuller(const char* type);

 private:
  PredictDataType data_type_ = kPDT_Float;
  std::string run_mode_;
  NetDef net_def_;
  bool has_net_ = false;
  std::shared_ptr<store::SparsePuller> sparse_puller_;
  std::unordered_map<int, std::unordered_map<int, std::shared_ptr<Workspace>>> workspace_;
  std::mutex mutex_;
};

// the request-batching schedulers are outside this build; kept so callers that configure them still link
bool InitScheduler(bool enable_batching, int max_batch_size, int batch_timeout_micros, int num_threads_for_cpu,
                   int num_threads_for_cuda, int num_threads_for_pipe);

}  // namespace blaze
