// proto.h -- the wire/config messages of the path as plain structs, with readers for both encodings.
//
// The reference generates these classes with protoc from blaze/proto/blaze.proto:6-115 and
// blaze/proto/embedding.proto:6-47 and parses text configs through TextFormat
// (blaze/common/proto_configure.cc:68-80).  This build has no protobuf toolchain: the structs below
// carry the same fields (same names, numbers and defaults) and are read by a small text-format
// parser and a proto2 wire-format codec written for exactly these messages.
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "blaze/common.h"

namespace blaze {

struct Argument {             // blaze.proto:25-33
  std::string name;           // 1
  float f = 0;                // 2
  int64_t i = 0;              // 3
  std::string s;              // 4 (bytes)
  std::vector<float> floats;  // 5 [packed]
  std::vector<int64_t> ints;  // 6 [packed]
  std::vector<std::string> strings;  // 7
  bool has_f = false, has_i = false, has_s = false;
};

struct DeviceOption {  // blaze.proto:41-46
  int32_t device_type_ = 0;
  int32_t device_id_ = 0;
  bool is_pipe_ = false;
  int device_type() const { return device_type_; }
  int device_id() const { return device_id_; }
  bool is_pipe() const { return is_pipe_; }
  void set_device_type(int t) { device_type_ = t; }
  void set_device_id(int i) { device_id_ = i; }
};

struct TensorShape {
  std::vector<int64_t> dims;
};

struct OperatorDef {  // blaze.proto:48-65 (the fused-graph field 8 is skipped on read)
  std::string type_, name_;
  std::vector<std::string> input_, output_;
  std::vector<Argument> arg_;
  DeviceOption device_option_;
  bool has_device_option_ = false;
  std::string doc_string_;

  const std::string& type() const { return type_; }
  const std::string& name() const { return name_; }
  int input_size() const { return (int)input_.size(); }
  int output_size() const { return (int)output_.size(); }
  const std::string& input(int i) const { return input_[i]; }
  const std::string& output(int i) const { return output_[i]; }
  const std::vector<std::string>& input() const { return input_; }
  const std::vector<std::string>& output() const { return output_; }
  const std::vector<Argument>& arg() const { return arg_; }
  bool has_device_option() const { return has_device_option_; }
  const DeviceOption& device_option() const { return device_option_; }
  DeviceOption* mutable_device_option() {
    has_device_option_ = true;
    return &device_option_;
  }
  std::string DebugString() const;
};

enum InputType { kInputDense = 0, kInputSparseIds = 1, kInputSparseValues = 2, kInputSparseSegments = 3, kInputIndicator = 4 };

struct ValueInfo {  // blaze.proto:75-90
  std::string name_;
  int32_t dtype_ = kFloat;
  std::string doc_string_;
  int32_t level_ = 0;
  int32_t input_type_ = kInputDense;
  std::string feature_name_;
  TensorShape tensor_shape_;
  const std::string& name() const { return name_; }
  DataType dtype() const { return (DataType)dtype_; }
  int level() const { return level_; }
  int input_type() const { return input_type_; }
  const std::string& feature_name() const { return feature_name_; }
};

struct NetDef {  // blaze.proto:92-115
  std::string name_;
  std::vector<OperatorDef> op_;
  std::string run_mode_ = "simple";
  std::vector<Argument> arg_;
  DeviceOption device_option_;
  bool has_device_option_ = false;
  std::vector<ValueInfo> external_input_, external_output_;
  std::string model_str_;
  int32_t version_ = 1000;

  const std::string& name() const { return name_; }
  int op_size() const { return (int)op_.size(); }
  const OperatorDef& op(int i) const { return op_[i]; }
  const std::vector<OperatorDef>& op() const { return op_; }
  const std::string& run_mode() const { return run_mode_; }
  bool has_device_option() const { return has_device_option_; }
  const DeviceOption& device_option() const { return device_option_; }
  DeviceOption* mutable_device_option() {
    has_device_option_ = true;
    return &device_option_;
  }
  int external_input_size() const { return (int)external_input_.size(); }
  int external_output_size() const { return (int)external_output_.size(); }
  const ValueInfo& external_input(int i) const { return external_input_[i]; }
  const ValueInfo& external_output(int i) const { return external_output_[i]; }
};

// ---- embedding.proto ---------------------------------------------------------------------------
enum TruncDirection { kInorder = 0, kReverse = 1 };  // embedding.proto:14-17
enum UDFType { kSum = 0, kAvg = 1, kAssign = 2 };    // embedding.proto:20-25

struct EmbeddingFeatureGroupConfig {  // embedding.proto:6-10
  std::string feature_group, table_name;
  int32_t dim = 18;
};
struct EmbeddingBlockConfigItem {  // embedding.proto:29-38
  std::string feature_group;
  int32_t udf_type = 0;
  int32_t trunc_direction = kReverse;
  int32_t trunc_num = 0;
  uint64_t offset = 0;
};
struct EmbeddingBlockConfig {  // embedding.proto:40-44
  uint64_t stride = 0;
  std::vector<EmbeddingBlockConfigItem> embedding_block_config_item;
};
struct EmbeddingConfig {  // embedding.proto:46-49
  std::vector<EmbeddingFeatureGroupConfig> feature_group_config;
  std::vector<EmbeddingBlockConfig> block_config;
};

// ---- readers -----------------------------------------------------------------------------------
// protobuf text format (what TextFormat::ParseFromString accepts for these messages); throws on
// malformed input, ignores unknown fields (e.g. the `name` of a block_config in the reference's
// embedding_config_v1.conf, which the schema does not define)
void ParseNetDefText(const std::string& text, NetDef* out);
void ParseEmbeddingConfigText(const std::string& text, EmbeddingConfig* out);
// proto2 wire format (what NetDefHelper::LoadNetDefFromBinaryFile reads); returns false on malformed input
bool ParseNetDefBinary(const void* data, size_t len, NetDef* out);
void SerializeNetDefBinary(const NetDef& net, std::string* out);
void SerializeNetDefText(const NetDef& net, std::string* out);
// model file: binary first, then text (the reference loads text NetDefs only in tests, workspace.cc:33-42)
bool LoadNetDefFromFile(const char* path, NetDef* out, std::string* err);

// ---- argument access (blaze/common/proto_helper.h: ArgumentHelper) ------------------------------
struct ArgumentHelper {
  static const Argument* Find(const std::vector<Argument>& args, const std::string& name) {
    for (const auto& a : args)
      if (a.name == name) return &a;
    return nullptr;
  }
  template <typename T>
  static T GetSingle(const std::vector<Argument>& args, const std::string& name, const T& def);
  template <typename T>
  static std::vector<T> GetRepeated(const std::vector<Argument>& args, const std::string& name,
                                    const std::vector<T>& def = {});
};

}  // namespace blaze
