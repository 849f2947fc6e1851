#include "blaze/predictor.h"

#include <algorithm>

#include "blaze/qed_store.h"

namespace blaze {

Predictor::Predictor(std::shared_ptr<Net> net) : net_(net) {
  for (const auto& name : net_->external_output()) {
    Blob* b = net_->external_output_blob(name);
    BLAZE_CONDITION_THROW(b != nullptr, "external_output: ", name, " is not in external_output_blob");
    output_index_[name] = (int)external_output_blob_.size();
    external_output_blob_.push_back(b);
    DeviceOption cpu;
    cpu.set_device_type(kCPU);
    output_cpu_.push_back(std::make_shared<Blob>(cpu));
    output_cpu_.back()->set_data_type((DataType)b->data_type());
  }
  for (const auto& name : net_->external_input()) {
    Blob* b = net_->external_input_blob(name);
    BLAZE_CONDITION_THROW(b != nullptr, "external_input: ", name, " is not in external_input_blob");
    input_index_[name] = (int)external_input_blob_.size();
    external_input_blob_.push_back(b);
    DeviceOption cpu;
    cpu.set_device_type(kCPU);
    input_cpu_.push_back(std::make_shared<Blob>(cpu));
    feed_pending_.push_back(false);
  }
}

Predictor::~Predictor() {
  // Wait only for work that is still queued: an event that was already waited for may belong to a stream that died with
  // its serving thread.  Nothing here may leave an error behind for the caller's next runtime call.
  if (feed_done_ && any_feed_pending_) (void)hipEventSynchronize(feed_done_);
  if (forward_done_ && forward_in_flight_) (void)hipEventSynchronize(forward_done_);
  if (arena_host_) (void)hipHostFree(arena_host_);
  if (arena_dev_) (void)hipFree(arena_dev_);
  for (void* a : retired_arenas_) (void)hipFree(a);
  if (forward_done_) (void)hipEventDestroy(forward_done_);
  if (feed_done_) (void)hipEventDestroy(feed_done_);
  (void)hipGetLastError();
}

int Predictor::InputName2Idx(const char* name) const {
  auto it = input_index_.find(name);
  return it == input_index_.end() ? -1 : it->second;
}
int Predictor::OutputName2Idx(const char* name) const {
  auto it = output_index_.find(name);
  return it == output_index_.end() ? -1 : it->second;
}

bool Predictor::ReshapeInput(const char* name, const std::vector<size_t>& shape) {
  const int idx = InputName2Idx(name);
  if (idx < 0) {
    LOG_ERROR("The name: %s is not The input of net", name);
    return false;
  }
  return ReshapeInput((size_t)idx, shape);
}
bool Predictor::ReshapeInput(size_t idx, const std::vector<size_t>& shape) {
  if (idx >= external_input_blob_.size()) {
    LOG_ERROR("The idx=%zu exceed size=%zu", idx, external_input_blob_.size());
    return false;
  }
  try {
    external_input_blob_[idx]->Reshape(shape);
  } catch (std::exception& e) {
    LOG_ERROR("reshape failed: %s", e.what());
    return false;
  }
  return true;
}

bool Predictor::Feed(const char* name, const void* data, size_t len) {
  const int idx = InputName2Idx(name);
  if (idx < 0) {
    LOG_ERROR("The name: %s is not The input of net", name);
    return false;
  }
  return Feed((size_t)idx, data, len);
}
bool Predictor::Feed(size_t idx, const void* data, size_t len) {
  if (idx >= external_input_blob_.size()) {
    LOG_ERROR("The idx=%zu exceed size=%zu", idx, external_input_blob_.size());
    return false;
  }
  Blob* blob = external_input_blob_[idx];
  const size_t need = blob->size() * DataTypeSize(blob->data_type());
  if (len != need) {
    LOG_ERROR("The len=%zu need size=%zu blob->size()=%zu", len, need, (size_t)blob->size());
    return false;
  }
  try {
    if (blob->device_type() == kCPU) {
      memcpy(blob->data(), data, need);
    } else {
      HIPContext ctx(blob->device_option());
      ctx.Activate();
      hipStream_t st = ctx.hip_stream();
      if (blob->unplaced()) {  // outgrew its slice of the FeedMany arena: back to memory of its own
        const std::vector<TIndex> shape = blob->shape();
        blob->DropArenaView();
        blob->Reshape(shape);
      }
      // stage in pinned memory and queue the transfer; a second Feed of the same input first waits for the first
      if (feed_done_ == nullptr) HIP_CHECK(hipEventCreateWithFlags(&feed_done_, hipEventDisableTiming));
      if (feed_pending_[idx]) {
        HIP_CHECK(hipEventSynchronize(feed_done_));
        std::fill(feed_pending_.begin(), feed_pending_.end(), false);
        any_feed_pending_ = false;
      }
      Blob* stage = input_cpu_[idx].get();
      stage->set_data_type((DataType)blob->data_type());
      stage->Reshape(blob->shape());
      memcpy(stage->data(), data, need);
      if (blob->pitch() != 0) {  // the input lives inside a Concat's output: rows are `pitch` elements apart
        const size_t es = DataTypeSize(blob->data_type()), w = blob->shape()[1] * es;
        HIP_CHECK(hipMemcpy2DAsync(blob->data(), blob->pitch() * es, stage->data(), w, w, blob->shape()[0], hipMemcpyHostToDevice, st));
      } else if (need > 0) {
        HIP_CHECK(hipMemcpyAsync(blob->data(), stage->data(), need, hipMemcpyHostToDevice, st));
      }
      HIP_CHECK(hipEventRecord(feed_done_, st));
      feed_pending_[idx] = true;
      any_feed_pending_ = true;
    }
  } catch (std::exception& e) {
    LOG_ERROR("feed failed: %s", e.what());
    return false;
  }
  return true;
}

bool Predictor::FeedMany(int count, const char* const* names, const void* const* data, const size_t* lens) {
  try {
    struct Item {
      int idx;
      int arg;
      size_t offset;
    };
    std::vector<Item> in_arena;
    size_t total = 0;
    const DeviceOption* dev = nullptr;
    for (int i = 0; i < count; ++i) {
      const int idx = InputName2Idx(names[i]);
      if (idx < 0) {
        LOG_ERROR("The name: %s is not The input of net", names[i]);
        return false;
      }
      Blob* blob = external_input_blob_[idx];
      const size_t need = blob->size() * DataTypeSize(blob->data_type());
      if (lens[i] != need) {
        LOG_ERROR("The len=%zu need size=%zu blob->size()=%zu", lens[i], need, (size_t)blob->size());
        return false;
      }
      if (blob->device_type() != kHIP || blob->pitch() != 0) {
        if (!Feed((size_t)idx, data[i], lens[i])) return false;
        continue;
      }
      dev = &blob->device_option();
      in_arena.push_back({idx, i, total});
      total += (need + 255) / 256 * 256;  // every slice 256-byte aligned
    }
    if (in_arena.empty()) return true;
    HIPContext ctx(*dev);
    ctx.Activate();
    hipStream_t st = ctx.hip_stream();
    if (feed_done_ == nullptr) HIP_CHECK(hipEventCreateWithFlags(&feed_done_, hipEventDisableTiming));
    if (any_feed_pending_) {  // the staging arena may still be read by the previous transfer
      HIP_CHECK(hipEventSynchronize(feed_done_));
      std::fill(feed_pending_.begin(), feed_pending_.end(), false);
      any_feed_pending_ = false;
    }
    if (total > arena_cap_) {
      if (arena_host_) HIP_CHECK(hipHostFree(arena_host_));
      if (arena_dev_) retired_arenas_.push_back(arena_dev_);
      arena_host_ = arena_dev_ = nullptr;
      arena_cap_ = 0;
      const size_t cap = total + total / 4;
      AllocationCount() += 2;
      HIP_CHECK(hipHostMalloc((void**)&arena_host_, cap, hipHostMallocDefault));
      HIP_CHECK(hipMalloc((void**)&arena_dev_, cap));
      arena_cap_ = cap;
    }
    for (const Item& it : in_arena) memcpy(arena_host_ + it.offset, data[it.arg], lens[it.arg]);
    HIP_CHECK(hipMemcpyAsync(arena_dev_, arena_host_, total, hipMemcpyHostToDevice, st));
    HIP_CHECK(hipEventRecord(feed_done_, st));
    for (const Item& it : in_arena) {
      Blob* blob = external_input_blob_[it.idx];
      // (also when the slice did not move: this records the slice's new size and clears "unplaced")
      const std::vector<TIndex> shape = blob->shape();
      blob->RefReshape(shape, arena_dev_ + it.offset, /*arena_view=*/true);
      feed_pending_[it.idx] = true;
    }
    any_feed_pending_ = true;
  } catch (std::exception& e) {
    LOG_ERROR("feed failed: %s", e.what());
    last_error_for_thread() = e.what();
    return false;
  }
  return true;
}

int Predictor::InputDataType(const char* name) const {
  const int idx = InputName2Idx(name);
  return idx < 0 ? (int)kPDT_Invalid : external_input_blob_[idx]->data_type();
}

int Predictor::device_id() const {
  for (const auto* list : {&external_output_blob_, &external_input_blob_})
    for (Blob* b : *list)
      if (b->device_type() == kHIP) return b->device_option().device_id();
  return -1;
}

bool Predictor::ForwardLaunch() {
  try {
    for (size_t i = 0; i < external_input_blob_.size(); ++i)
      if (external_input_blob_[i]->unplaced()) {
        last_error_for_thread() = "input " + net_->external_input()[i] + " was reshaped beyond its fed size and has not been fed since";
        LOG_ERROR("%s", last_error_for_thread().c_str());
        return false;
      }
    if (any_feed_pending_) {
      // the transfers were queued on the feeding thread's stream: make this thread's stream wait for them
      for (Blob* b : external_input_blob_) {
        if (b->device_type() != kHIP) continue;
        HIPContext ctx(b->device_option());
        ctx.Activate();
        HIP_CHECK(hipStreamWaitEvent(ctx.hip_stream(), feed_done_, 0));
        break;
      }
    }
    if (!net_->Launch()) return false;
    launched_on_ = net_->StreamOfLastLaunch();
    if (launched_on_ != nullptr) {
      if (forward_done_ == nullptr) HIP_CHECK(hipEventCreateWithFlags(&forward_done_, hipEventDisableTiming));
      HIP_CHECK(hipEventRecord(forward_done_, (hipStream_t)launched_on_));
    }
    forward_in_flight_ = true;
    return true;
  } catch (std::exception& e) {
    LOG_ERROR("failed: %s", e.what());
    last_error_for_thread() = e.what();
    return false;
  }
}

bool Predictor::ForwardWait() {
  try {
    if (!forward_in_flight_) {
      last_error_for_thread() = "ForwardWait without a ForwardLaunch before it";
      return false;
    }
    forward_in_flight_ = false;
    // the event sits behind the net's last operator, which sits behind the queued input transfers
    if (launched_on_ != nullptr) HIP_CHECK(hipEventSynchronize(forward_done_));
    if (any_feed_pending_) {
      std::fill(feed_pending_.begin(), feed_pending_.end(), false);
      any_feed_pending_ = false;
    }
    return true;
  } catch (std::exception& e) {
    LOG_ERROR("failed: %s", e.what());
    last_error_for_thread() = e.what();
    return false;
  }
}

bool Predictor::Forward(const PredictorCallback&& cb) {
  try {
    if (forward_in_flight_ && !ForwardWait()) return false;  // a launch the caller never waited for
    for (size_t i = 0; i < external_input_blob_.size(); ++i)
      if (external_input_blob_[i]->unplaced()) {
        last_error_for_thread() = "input " + net_->external_input()[i] + " was reshaped beyond its fed size and has not been fed since";
        LOG_ERROR("%s", last_error_for_thread().c_str());
        return false;
      }
    if (any_feed_pending_) {
      // the transfers were queued on the feeding thread's stream: make this thread's stream wait for them
      for (Blob* b : external_input_blob_) {
        if (b->device_type() != kHIP) continue;
        HIPContext ctx(b->device_option());
        ctx.Activate();
        HIP_CHECK(hipStreamWaitEvent(ctx.hip_stream(), feed_done_, 0));
        break;
      }
    }
    if (!net_->Run()) return false;
    if (any_feed_pending_) {  // Run waited for the stream, which had waited for the transfers
      std::fill(feed_pending_.begin(), feed_pending_.end(), false);
      any_feed_pending_ = false;
    }
    if (cb) cb();
    return true;
  } catch (std::exception& e) {
    LOG_ERROR("failed: %s", e.what());
    last_error_for_thread() = e.what();
    return false;
  }
}

bool Predictor::Output(const char* name, void** data, size_t* len) {
  const int idx = OutputName2Idx(name);
  if (idx < 0) {
    LOG_ERROR("The name: %s is not The output of net", name);
    return false;
  }
  return Output((size_t)idx, data, len);
}
bool Predictor::Output(size_t idx, void** data, size_t* len) {
  if (idx >= external_output_blob_.size()) {
    LOG_ERROR("The idx=%zu exceed size=%zu", idx, external_output_blob_.size());
    return false;
  }
  Blob* blob = external_output_blob_[idx];
  const size_t bytes = blob->size() * DataTypeSize(blob->data_type());
  try {
    if (blob->device_type() == kCPU) {
      *data = blob->data();
    } else {
      std::shared_ptr<Blob>& cpu = output_cpu_[idx];
      cpu->set_data_type((DataType)blob->data_type());
      cpu->Reshape(blob->shape());
      HIPContext ctx(blob->device_option());
      ctx.Activate();
      CopyBytes(cpu->data(), kCPU, blob->data(), kHIP, bytes, ctx.hip_stream());
      *data = cpu->data();
    }
  } catch (std::exception& e) {
    LOG_ERROR("output failed: %s", e.what());
    return false;
  }
  if (len) *len = bytes;
  return true;
}

const std::vector<size_t>& Predictor::OutputShape(size_t idx) const {
  BLAZE_CONDITION_THROW(idx < external_output_blob_.size(), "The idx=", idx, " blob is null");
  return external_output_blob_[idx]->shape();
}
const std::vector<size_t>& Predictor::OutputShape(const char* name) const {
  const int idx = OutputName2Idx(name);
  BLAZE_CONDITION_THROW(idx >= 0, "The name ", name, " is not Output of net");
  return OutputShape((size_t)idx);
}
int Predictor::OutputDataType(const char* name) const {
  const int idx = OutputName2Idx(name);
  return idx < 0 ? (int)kPDT_Invalid : external_output_blob_[idx]->data_type();
}

std::vector<std::string> Predictor::ListInternalName() const {
  std::vector<std::string> names;
  for (const auto& it : net_->workspace()->constant_blobs()) names.push_back(it.first);
  return names;
}
bool Predictor::InternalParam(const char* name, void** data, size_t* len) {
  const auto& m = net_->workspace()->constant_blobs();
  auto it = m.find(name);
  if (it == m.end()) return false;
  Blob* blob = it->second;
  const size_t bytes = blob->size() * DataTypeSize(blob->data_type());
  try {
    if (blob->device_type() == kCPU) {
      *data = blob->data();
    } else {
      DeviceOption cpu_opt;
      cpu_opt.set_device_type(kCPU);
      auto& cpu = param_cpu_[name];
      if (!cpu) cpu = std::make_shared<Blob>(cpu_opt);
      cpu->set_data_type((DataType)blob->data_type());
      cpu->Reshape(blob->shape());
      HIPContext ctx(blob->device_option());
      ctx.Activate();
      CopyBytes(cpu->data(), kCPU, blob->data(), kHIP, bytes, ctx.hip_stream());
      *data = cpu->data();
    }
  } catch (std::exception& e) {
    LOG_ERROR("param copy failed: %s", e.what());
    return false;
  }
  if (len) *len = bytes;
  return true;
}
const std::vector<size_t>& Predictor::InternalShape(const char* name) const {
  const auto& m = net_->workspace()->constant_blobs();
  auto it = m.find(name);
  BLAZE_CONDITION_THROW(it != m.end(), "The name ", name, " is not a parameter of net");
  return it->second->shape();
}
int Predictor::InternalDataType(const char* name) const {
  const auto& m = net_->workspace()->constant_blobs();
  auto it = m.find(name);
  return it == m.end() ? (int)kPDT_Invalid : it->second->data_type();
}

void Predictor::RegisterObservers(const std::vector<std::string>& names) {
  for (const auto& n : names)
    if (n == "profile") net_->set_profile(true);
}
void Predictor::DumpObservers(std::unordered_map<std::string, std::string>* dump_map) {
  (*dump_map)["profile"] = net_->DumpProfile();
}

void* Predictor::InputDevicePtr(const char* name) {
  const int idx = InputName2Idx(name);
  if (idx >= 0 && external_input_blob_[idx]->unplaced()) {  // outgrew its feed-arena slice: memory of its own
    Blob* blob = external_input_blob_[idx];
    const std::vector<TIndex> shape = blob->shape();
    blob->DropArenaView();
    blob->Reshape(shape);
  }
  // (a strided input -- one that lives inside a Concat's output -- has no plain buffer to hand out)
  return idx < 0 || external_input_blob_[idx]->pitch() != 0 ? nullptr : external_input_blob_[idx]->data();
}
void* Predictor::OutputDevicePtr(const char* name) {
  const int idx = OutputName2Idx(name);
  return idx < 0 ? nullptr : external_output_blob_[idx]->data();
}

std::string& last_error_for_thread() {
  static thread_local std::string s;
  return s;
}

// ------------------------------------------------------------------------------------------ manager
std::shared_ptr<store::SparsePuller>& PredictorManager::EnsureSparsePuller(const char* type) {
  if (!sparse_puller_) sparse_puller_.reset(store::SparsePullerCreationRegisterer::Get()->CreateSparsePuller(type));
  return sparse_puller_;
}

bool PredictorManager::LoadSparseModelWeight(const char* uri, const char* type) {
  try {
    sparse_puller_.reset(store::SparsePullerCreationRegisterer::Get()->CreateSparsePuller(type));
    if (store::kOK != sparse_puller_->Load(uri)) {
      LOG_ERROR("load sparse model %s failed", uri);
      return false;
    }
  } catch (std::exception& e) {
    LOG_ERROR("load sparse model %s failed: %s", uri, e.what());
    last_error_for_thread() = e.what();
    return false;
  }
  return true;
}

bool PredictorManager::LoadModel(const char* filename, bool optimization_pass) {
  return LoadModel(filename, "", kBlaze, optimization_pass);
}
bool PredictorManager::LoadDeepNetModel(const char* model_conf, const char* model_data, bool optimization_pass) {
  return LoadModel(model_conf, model_data, kUlf, optimization_pass);
}
bool PredictorManager::LoadModel(const char* conf_file, const char*, ModelType model_type, bool) {
  if (model_type != kBlaze) {
    LOG_ERROR("model type %d needs an importer that is not part of this build; convert the model to a Blaze NetDef first", model_type);
    last_error_for_thread() = "unsupported model type";
    return false;
  }
  std::string err;
  NetDef def;
  if (!LoadNetDefFromFile(conf_file, &def, &err)) {
    LOG_ERROR("Load model %s failed: %s", conf_file, err.c_str());
    last_error_for_thread() = err;
    return false;
  }
  return LoadNetDef(def);
}
bool PredictorManager::LoadNetDef(const NetDef& net_def) {
  std::lock_guard<std::mutex> lock(mutex_);
  net_def_ = net_def;
  if (!run_mode_.empty()) net_def_.run_mode_ = run_mode_;
  has_net_ = true;
  workspace_.clear();
  return true;
}

Predictor* PredictorManager::CreatePredictor(PredictDeviceType predict_device, int device_id) {
  std::lock_guard<std::mutex> lock(mutex_);
  try {
    BLAZE_CONDITION_THROW(has_net_, "no model loaded");
    if (device_id < 0) device_id = 0;
    DeviceOption device_option;
    switch (predict_device) {
      case kPDT_CPU:
        device_option.set_device_type(kCPU);
        device_option.set_device_id(0);
        break;
      case kPDT_HIP:
        device_option.set_device_type(kHIP);
        device_option.set_device_id(device_id);
        break;
      default: {  // ProbeDevice (predictor_manager_impl.cc:162-177): round robin over the visible accelerators
        static int next = 0;
        int count = 0;
        HIP_CHECK(hipGetDeviceCount(&count));
        BLAZE_CONDITION_THROW(count > 0, "no accelerator visible and this build has no CPU path");
        device_option.set_device_type(kHIP);
        device_option.set_device_id(next++ % count);
      }
    }
    const int dt = device_option.device_type(), di = device_option.device_id();
    auto& ws = workspace_[dt][di];
    if (!ws) {
      ws.reset(new Workspace());
      ws->Init(net_def_);
      auto* opt = ws->net_def()->mutable_device_option();
      opt->set_device_type(dt);
      opt->set_device_id(di);
      // the device of the predictor overrides what individual operators were exported with
      for (auto& op : ws->net_def()->op_) {
        if (op.has_device_option()) {
          op.device_option_.set_device_type(dt);
          op.device_option_.set_device_id(di);
        }
      }
      ws->SetSparsePuller(sparse_puller_);
    }
    std::shared_ptr<Net> net = ws->CreateNet();
    BLAZE_CONDITION_THROW(net != nullptr, "net creation failed");
    return new Predictor(net);
  } catch (std::exception& e) {
    LOG_ERROR("Create Model Predictor failed, msg=%s", e.what());
    last_error_for_thread() = e.what();
    return nullptr;
  }
}

bool InitScheduler(bool, int, int, int, int, int) { return true; }

}  // namespace blaze
