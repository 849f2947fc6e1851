#include "blaze/operator.h"

#include "blaze/graph.h"

namespace blaze {

bool OpSchema::Verify(const OperatorDef& def) const {
  if (def.input_size() < min_input_ || def.input_size() > max_input_) {
    LOG_ERROR("%s: input size %d not in [%d, %d] (schema at %s:%d)", def.type().c_str(), def.input_size(), min_input_,
              max_input_, file_.c_str(), line_);
    return false;
  }
  if (def.output_size() < min_output_ || def.output_size() > max_output_) {
    LOG_ERROR("%s: output size %d not in [%d, %d] (schema at %s:%d)", def.type().c_str(), def.output_size(), min_output_,
              max_output_, file_.c_str(), line_);
    return false;
  }
  // an output may alias an input only where the schema allows in-place
  for (int i = 0; i < def.input_size(); ++i)
    for (int o = 0; o < def.output_size(); ++o)
      if (def.input(i) == def.output(o) && !allow_inplace(i, o)) {
        LOG_ERROR("%s: input %d and output %d alias (%s) but in-place is not allowed", def.type().c_str(), i, o,
                  def.input(i).c_str());
        return false;
      }
  return true;
}

std::map<std::string, OpSchema>& OpSchemaRegistry::map() {
  static std::map<std::string, OpSchema> m;
  return m;
}
OpSchema& OpSchemaRegistry::NewSchema(const std::string& key, const std::string& file, int line) {
  auto& m = map();
  if (m.count(key)) BLAZE_THROW("Trying to register schema with name ", key, " from file ", file, " line ", line, ", but it is already registered");
  m.emplace(key, OpSchema(file, line));
  return m[key];
}
OpSchema* OpSchemaRegistry::Schema(const std::string& key) {
  auto& m = map();
  auto it = m.find(key);
  return it == m.end() ? nullptr : &it->second;
}

OperatorBase::OperatorBase(const OperatorDef& def, Workspace* workspace, bool alloc_input_output_blob)
    : def_(def), workspace_(workspace), device_option_(def.has_device_option() ? def.device_option() : DeviceOption()) {
  type_ = def_.type();
  name_ = def_.name();
  OpSchema* schema = OpSchemaRegistry::Schema(type_);
  BLAZE_CONDITION_THROW(schema != nullptr, "Schema for op_type ", type_, " is not registered.");
  CheckSchema(schema);
  if (alloc_input_output_blob) AllocInputOutputBlob(def);
}

void OperatorBase::AllocInputOutputBlob(const OperatorDef& def) {
  OpSchema* schema = OpSchemaRegistry::Schema(type_);
  bool newblob = false;
  for (const std::string& input_str : def.input()) {
    Blob* blob = workspace_->CreateBlob(input_str, device_option_, &newblob);
    inputs_.push_back(blob);
    if (newblob) blob->set_data_type(workspace_->input_data_type(input_str));  // a net input: typed by external_input
  }
  std::vector<DataType> input_types;
  for (auto* b : inputs_) input_types.push_back((DataType)b->data_type());
  std::vector<DataType> output_types = schema->InferType(def_, input_types);
  for (int k = 0; k < def.output_size(); ++k) {
    Blob* blob = workspace_->CreateBlob(def.output(k), device_option_, &newblob);
    outputs_.push_back(blob);
    if (newblob) {
      BLAZE_CONDITION_THROW(k < (int)output_types.size(), "k=", k, " output_types.size()=", output_types.size(), " ", def.name());
      blob->set_data_type(output_types[k]);
    }
  }
}

void OperatorBase::CheckSchema(OpSchema* schema) {
  BLAZE_CONDITION_THROW(schema->min_input() <= def_.input_size() && schema->max_input() >= def_.input_size(),
                        "min_input=", schema->min_input(), " max_input=", schema->max_input(),
                        " def_.input_size()=", def_.input_size());
  BLAZE_CONDITION_THROW(schema->min_output() <= def_.output_size() && schema->max_output() >= def_.output_size(),
                        "min_output=", schema->min_output(), " max_output=", schema->max_output(),
                        " def_.output_size()=", def_.output_size());
}

std::map<int, OperatorRegistry*>* GetDeviceTypeRegistry() {
  static std::map<int, OperatorRegistry*> m = {{kCPU, CPUOperatorRegistry()}, {kHIP, HIPOperatorRegistry()}};
  return &m;
}
OperatorRegistry* CPUOperatorRegistry() {
  static OperatorRegistry* r = new OperatorRegistry();
  return r;
}
OperatorRegistry* HIPOperatorRegistry() {
  static OperatorRegistry* r = new OperatorRegistry();
  return r;
}

std::unique_ptr<OperatorBase> CreateOperator(const OperatorDef& def, Workspace* ws, int net_position) {
  const auto& op_type = def.type();
  const int device_type = def.device_option().device_type();
  auto* schema = OpSchemaRegistry::Schema(op_type);
  BLAZE_CONDITION_THROW(schema != nullptr, "Schema for op_type ", op_type, " is not registered.");
  BLAZE_CONDITION_THROW(schema->Verify(def), "Verify schema failed. ", def.DebugString());
  BLAZE_CONDITION_THROW(GetDeviceTypeRegistry()->count(device_type), "Device type ", device_type, " not registered.");
  OperatorRegistry* registry = GetDeviceTypeRegistry()->at(device_type);
  BLAZE_CONDITION_THROW(registry->Has(op_type), "op_type=", op_type, " is not registered for device type ", device_type,
                        device_type == kCPU ? " (this build implements the path on the accelerator only; there is no CPU fallback)" : "");
  auto op = registry->Create(op_type, def, ws);
  BLAZE_CONDITION_THROW(op, "op_type=", op_type);
  op->set_net_position(net_position);
  return op;
}

}  // namespace blaze
