// operator.h -- the operator plugin boundary: OpSchema, OperatorBase, Operator<Context>, the per-device
// registries and the REGISTER_*_OPERATOR / OPERATOR_SCHEMA macros.
//
// This is the drop-in boundary of the build.  It re-creates, with the same names, argument meaning and error
// behaviour, what the reference declares in blaze/operator/operator.h:28-294, operator.cc:9-122 and
// operator_schema.h:28-316: an op is a class `T : Operator<Context>` with ctor T(const OperatorDef&, Workspace*)
// and `bool RunOnDevice()`, registered per device under its type string; every op needs an OPERATOR_SCHEMA (the
// registration macro references PLEASE_ADD_OPERATOR_SCHEMA_FOR_<Name>, so a missing schema is a link error).
// The accelerator registry is keyed by device_type 1, the value existing NetDefs use for the GPU.
#pragma once

#include <climits>
#include <functional>
#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "blaze/common.h"
#include "blaze/proto.h"
#include "blaze/registry.h"
#include "blaze/runtime.h"

namespace blaze {

class Workspace;

// ------------------------------------------------------------------------------------------ schema
class OpSchema {
 public:
  OpSchema() {}
  OpSchema(const std::string& file, int line) : file_(file), line_(line) {}

  bool Verify(const OperatorDef& def) const;  // arity + in-place rules (operator_schema.cc)
  OpSchema& NumInputs(int n) { return NumInputs(n, n); }
  OpSchema& NumInputs(int min, int max) {
    min_input_ = min;
    max_input_ = max;
    return *this;
  }
  OpSchema& NumOutputs(int n) { return NumOutputs(n, n); }
  OpSchema& NumOutputs(int min, int max) {
    min_output_ = min;
    max_output_ = max;
    return *this;
  }
  OpSchema& AllowInplace(std::set<std::pair<int, int>> inplace) {
    inplace_ = inplace;
    return *this;
  }
  bool allow_inplace(int in_idx, int out_idx) const { return inplace_.count({in_idx, out_idx}) != 0; }

  typedef std::function<std::vector<DataType>(const OperatorDef&, const std::vector<DataType>&)> TypeInferenceFunctionType;
  OpSchema& TypeInferenceFunction(TypeInferenceFunctionType f) {
    type_inference_ = f;
    return *this;
  }
  OpSchema& IdenticalTypeOfInput(int idx) {
    return TypeInferenceFunction([idx](const OperatorDef& def, const std::vector<DataType>& in) {
      return std::vector<DataType>(def.output_size(), in.at(idx));
    });
  }
  OpSchema& ScalarType(DataType dt) {
    return TypeInferenceFunction(
        [dt](const OperatorDef& def, const std::vector<DataType>&) { return std::vector<DataType>(def.output_size(), dt); });
  }
  std::vector<DataType> InferType(const OperatorDef& def, const std::vector<DataType>& in) const {
    if (type_inference_) return type_inference_(def, in);
    // default: outputs take the type of the first input (kFloat for source ops)
    return std::vector<DataType>(def.output_size(), in.empty() ? kFloat : in[0]);
  }

  // algorithmic cost of one run, summed by the cost observer (operator_schema.h:109-128)
  struct Cost {
    uint64_t flops = 0, bytes_read = 0, bytes_written = 0, params_bytes = 0;
  };
  OpSchema& SetDoc(const std::string& doc) {
    doc_ = doc;
    return *this;
  }
  OpSchema& Input(int, const char*, const char*) { return *this; }
  OpSchema& Output(int, const char*, const char*) { return *this; }
  int min_input() const { return min_input_; }
  int max_input() const { return max_input_; }
  int min_output() const { return min_output_; }
  int max_output() const { return max_output_; }
  const std::string& doc() const { return doc_; }

 private:
  std::string file_ = "unknown", doc_;
  int line_ = 0;
  int min_input_ = 0, max_input_ = INT_MAX, min_output_ = 0, max_output_ = INT_MAX;
  std::set<std::pair<int, int>> inplace_;
  TypeInferenceFunctionType type_inference_;
};

class OpSchemaRegistry {
 public:
  static OpSchema& NewSchema(const std::string& key, const std::string& file, int line);
  static OpSchema* Schema(const std::string& key);  // nullptr when unknown

 private:
  static std::map<std::string, OpSchema>& map();
};

#define OPERATOR_SCHEMA(name)                                                      \
  void PLEASE_ADD_OPERATOR_SCHEMA_FOR_##name() {}                                  \
  static ::blaze::OpSchema* ANONYMOUS_VARIABLE(name) __attribute__((unused)) =     \
      &::blaze::OpSchemaRegistry::NewSchema(#name, __FILE__, __LINE__)

// ------------------------------------------------------------------------------------------ operators
class OperatorBase {
 public:
  OperatorBase(const OperatorDef& def, Workspace* workspace, bool alloc_input_output_blob = true);
  virtual ~OperatorBase() noexcept {}

  bool HasArgument(const std::string& name) const { return ArgumentHelper::Find(def_.arg(), name) != nullptr; }
  template <typename T>
  T GetSingleArgument(const std::string& name, const T& default_value) const {
    return ArgumentHelper::GetSingle<T>(def_.arg(), name, default_value);
  }
  template <typename T>
  std::vector<T> GetRepeatedArgument(const std::string& name, const std::vector<T>& default_value = {}) const {
    return ArgumentHelper::GetRepeated<T>(def_.arg(), name, default_value);
  }

  virtual bool Run(int stream_id = 0) = 0;
  virtual void WaitStream(int stream_id = -1) {}
  // the device stream the operator's work is queued on (of the calling thread), null for host operators
  virtual void* DeviceStream() { return nullptr; }
  // columns of 2-D output `idx` when they are fixed by the operator's arguments (else 0)
  virtual TIndex StaticOutputCols(int idx) const { return 0; }
  // compute-kernel launches of the operator's last run, when it keeps count (else -1); the profile observer reports it
  virtual int LaunchesOfLastRun() const { return -1; }

  const DeviceOption& device_option() const { return device_option_; }
  void set_net_position(int p) { net_position_ = p; }
  int net_position() const { return net_position_; }
  const OperatorDef& operator_def() const { return def_; }
  const std::string& type() const { return type_; }
  const std::string& name() const { return name_; }
  int InputSize() const { return (int)inputs_.size(); }
  int OutputSize() const { return (int)outputs_.size(); }
  std::vector<Blob*>& Inputs() { return inputs_; }
  std::vector<Blob*>& Outputs() { return outputs_; }
  Blob* Input(int idx) {
    BLAZE_CONDITION_THROW(idx >= 0 && idx < (int)inputs_.size(), "input idx=", idx, " size=", inputs_.size(), " ", def_.DebugString());
    return inputs_[idx];
  }
  Blob* Output(int idx) {
    BLAZE_CONDITION_THROW(idx >= 0 && idx < (int)outputs_.size(), "output idx=", idx, " size=", outputs_.size(), " ", def_.DebugString());
    return outputs_[idx];
  }
  // wall time of the last Run on the host, filled when profiling is on (the "profile" observer)
  double last_run_us() const { return last_run_us_; }
  void set_last_run_us(double us) { last_run_us_ = us; }

 protected:
  void AllocInputOutputBlob(const OperatorDef& def);
  void CheckSchema(OpSchema* schema);

  OperatorDef def_;
  Workspace* workspace_;
  DeviceOption device_option_;
  std::string type_, name_;
  std::vector<Blob*> inputs_, outputs_;
  int net_position_ = 0;
  double last_run_us_ = 0;
};

template <class Context>
class Operator : public OperatorBase {
 public:
  Operator(const OperatorDef& def, Workspace* workspace, bool alloc_blob = true)
      : OperatorBase(def, workspace, alloc_blob), context_(def.device_option()) {
    context_.SwitchToDevice(0);
  }
  ~Operator() noexcept override {}

  bool Run(int stream_id = 0) final {
    context_.SwitchToDevice(stream_id);
    return RunOnDevice();
  }
  virtual bool RunOnDevice() = 0;
  const Context& context() const { return context_; }
  void WaitStream(int stream_id = -1) override {
    const int old = context_.stream_id();
    context_.SwitchToDevice(stream_id < 0 ? old : stream_id);
    context_.FinishDeviceComputation();
    context_.SwitchToDevice(old);
  }
  void* DeviceStream() override { return context_.device_stream(); }

 protected:
  Context context_;
};

#define USE_OPERATOR_BASE_FUNCTIONS          \
  using OperatorBase::HasArgument;           \
  using OperatorBase::GetSingleArgument;     \
  using OperatorBase::GetRepeatedArgument;   \
  using OperatorBase::InputSize;             \
  using OperatorBase::OutputSize
#define USE_OPERATOR_FUNCTIONS(context)      \
  USE_OPERATOR_BASE_FUNCTIONS;               \
  using Operator<context>::context_;         \
  using Operator<context>::Input;            \
  using Operator<context>::Inputs;           \
  using Operator<context>::Output;           \
  using Operator<context>::Outputs

typedef Registry<std::unique_ptr<OperatorBase>, const OperatorDef&, Workspace*> OperatorRegistry;
typedef Registerer<std::unique_ptr<OperatorBase>, const OperatorDef&, Workspace*> OperatorRegisterer;
std::map<int, OperatorRegistry*>* GetDeviceTypeRegistry();
OperatorRegistry* CPUOperatorRegistry();
OperatorRegistry* HIPOperatorRegistry();

#define BLAZE_REGISTER_OPERATOR(registry, tag, name, ...)                                                   \
  extern void PLEASE_ADD_OPERATOR_SCHEMA_FOR_##name();                                                      \
  static void __attribute__((unused)) ANONYMOUS_VARIABLE(tag##name)() { PLEASE_ADD_OPERATOR_SCHEMA_FOR_##name(); } \
  namespace {                                                                                               \
  static ::blaze::OperatorRegisterer ANONYMOUS_VARIABLE(g_##tag##name)(                                     \
      #name, ::blaze::registry(), ::blaze::OperatorRegisterer::DefaultCreator<__VA_ARGS__>);                \
  }
#define REGISTER_CPU_OPERATOR(name, ...) BLAZE_REGISTER_OPERATOR(CPUOperatorRegistry, CPU, name, __VA_ARGS__)
#define REGISTER_HIP_OPERATOR(name, ...) BLAZE_REGISTER_OPERATOR(HIPOperatorRegistry, HIP, name, __VA_ARGS__)
// source compatibility for operators written against the reference's macro: the accelerator registry is the same
#define REGISTER_CUDA_OPERATOR(name, ...) REGISTER_HIP_OPERATOR(name, __VA_ARGS__)

// Create an operator with the given definition (operator.cc:100-122): schema must exist and verify, the
// device type must have a registry, the op type must be registered for it.
std::unique_ptr<OperatorBase> CreateOperator(const OperatorDef& def, Workspace* ws, int net_position);

// suffixes of the three tensors of a sparse feature group (blaze/operator/common_helper.h:96-98)
static const char* const kIdSuffix = ".ids";
static const char* const kValueSuffix = ".values";
static const char* const kIdNumSuffix = ".segments";
static const float kDiceEpsilon = 1e-8f;  // common_helper.h:90

}  // namespace blaze
