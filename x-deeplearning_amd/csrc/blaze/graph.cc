#include "blaze/graph.h"
#include "blaze_hip.h"

#include <stdlib.h>

#include <chrono>
#include <fstream>

namespace blaze {

// ------------------------------------------------------------------------------------------ workspace
Workspace::~Workspace() {
  std::set<Blob*> removed;
  for (auto& it : blob_map_) removed.insert(it.second);
  for (auto* b : blob_recycle_bins_) removed.insert(b);
  for (auto* b : removed) delete b;
  for (auto& it : constant_fill_blob_map_) delete it.second;
}

Blob* Workspace::CreateConstantBlob(const std::string& name, const DeviceOption& device_option, bool* newblob) {
  auto it = constant_fill_blob_map_.find(name);
  if (it == constant_fill_blob_map_.end()) {
    it = constant_fill_blob_map_.emplace(name, new Blob(device_option)).first;
    if (newblob) *newblob = true;
  } else if (newblob) {
    *newblob = false;
  }
  return it->second;
}

Blob* Workspace::CreateBlob(const std::string& name, const DeviceOption& device_option, bool* newblob) {
  auto c = constant_fill_blob_map_.find(name);
  if (c != constant_fill_blob_map_.end()) {
    if (newblob) *newblob = false;
    return c->second;
  }
  auto it = blob_map_.find(name);
  if (it == blob_map_.end()) {
    it = blob_map_.emplace(name, new Blob(device_option)).first;
    if (newblob) *newblob = true;
  } else if (newblob) {
    *newblob = false;
  }
  return it->second;
}

void Workspace::Init(const NetDef& net_def) {
  std::unique_lock<std::mutex> lock(mutex_);
  net_def_.reset(new NetDef(net_def));
  input_data_type_map_.clear();
  input_info_map_.clear();
  for (const auto& in : net_def_->external_input_) {
    input_data_type_map_[in.name()] = in.dtype();
    input_info_map_[in.name()] = in;
  }
}

void Workspace::RecycleBlobMap() {
  for (auto& it : blob_map_) blob_recycle_bins_.insert(it.second);
  blob_map_.clear();
}

std::shared_ptr<Net> Workspace::CreateNet() {
  std::unique_lock<std::mutex> lock(mutex_);
  BLAZE_CONDITION_THROW(net_def_ != nullptr, "Workspace::Init was not called");
  RecycleBlobMap();  // every net (= predictor) gets its own activation blobs; constants stay shared
  std::string run_mode = net_def_->run_mode();
  if (!NetRegistry()->Has(run_mode)) {
    LOG_INFO("run_mode %s is not available in this build, using the simple executor", run_mode.c_str());
    run_mode = "simple";
  }
  return NetRegistry()->Create(run_mode, net_def_, this);
}

std::shared_ptr<Net> Workspace::CreateNet(const char* net_file) {
  NetDef def;
  std::string err;
  if (!LoadNetDefFromFile(net_file, &def, &err)) BLAZE_THROW("Open net_file: ", net_file, " failed: ", err);
  Init(def);
  return CreateNet();
}

DataType Workspace::input_data_type(const std::string& input_name) const {
  auto it = input_data_type_map_.find(input_name);
  BLAZE_CONDITION_THROW(it != input_data_type_map_.end(), "input_name: ", input_name, " data_type not defined");
  return it->second;
}

const ValueInfo& Workspace::input_info(const std::string& input_name) const {
  auto it = input_info_map_.find(input_name);
  BLAZE_CONDITION_THROW(it != input_info_map_.end(), "input_name=", input_name, " is not input name");
  return it->second;
}

// ------------------------------------------------------------------------------------------ net
NetRegistryType* NetRegistry() {
  static NetRegistryType* r = new NetRegistryType();
  return r;
}

Net::Net(const std::shared_ptr<const NetDef>& def, Workspace* ws) : name_(def->name()), net_def_(def), workspace_(ws) {
  BLAZE_CONDITION_THROW(net_def_->has_device_option(), "net has no device option");
  // external inputs: tensors consumed before any operator produced them, in order of first use; external
  // outputs: the declared ones, else tensors nobody consumes
  std::set<std::string> produced, consumed;
  for (const auto& op : def->op()) {
    for (const auto& in : op.input()) {
      if (!produced.count(in) && !consumed.count(in)) external_input_.push_back(in);
      consumed.insert(in);
    }
    for (const auto& out : op.output()) produced.insert(out);
  }
  if (def->external_output_size() > 0) {
    for (const auto& v : def->external_output_) external_output_.push_back(v.name());
  } else {
    for (const auto& op : def->op())
      for (const auto& out : op.output())
        if (!consumed.count(out)) external_output_.push_back(out);
  }
  if (def->external_input_size() > 0) {
    for (const auto& in : external_input_) {
      bool declared = false;
      for (const auto& v : def->external_input_) declared |= v.name() == in;
      BLAZE_CONDITION_THROW(declared, "Source for input ", in, " is unkown for net ", def->name());
    }
  }
}

Blob* Net::external_input_blob(const std::string& name) const {
  auto it = external_input_blob_.find(name);
  return it == external_input_blob_.end() ? nullptr : it->second;
}
Blob* Net::external_output_blob(const std::string& name) const {
  auto it = external_output_blob_.find(name);
  return it == external_output_blob_.end() ? nullptr : it->second;
}

bool Net::Launch() {
  if (!RunImpl()) {
    LOG_ERROR("Failed to run impl");
    return false;
  }
  return true;
}

void* Net::StreamOfLastLaunch() {
  for (auto it = operators_.rbegin(); it != operators_.rend(); ++it)
    if (void* st = (*it)->DeviceStream()) return st;
  return nullptr;
}

bool Net::Run() {
  if (!Launch()) return false;
  // all operators run on stream 0 of this thread: waiting for that stream waits for the net (simple_net.cc:27-32)
  if (!operators_.empty()) operators_.back()->WaitStream();
  return true;
}

std::string Net::DumpProfile() const {
  std::stringstream ss;
  ss << "{\"traceEvents\":[";
  double t = 0;
  bool first = true;
  for (const auto& op : operators_) {
    if (!first) ss << ",";
    first = false;
    ss << "{\"name\":\"" << op->type() << ":" << op->name() << "\",\"ph\":\"X\",\"pid\":0,\"tid\":0,\"ts\":" << t
       << ",\"dur\":" << op->last_run_us();
    if (op->LaunchesOfLastRun() >= 0) ss << ",\"args\":{\"launches\":" << op->LaunchesOfLastRun() << "}";
    ss << "}";
    t += op->last_run_us();
  }
  ss << "]}";
  return ss.str();
}

SimpleNet::SimpleNet(const std::shared_ptr<const NetDef>& net_def, Workspace* ws) : Net(net_def, ws) {
  const bool net_has_device_option = net_def->has_device_option();
  for (int idx = 0; idx < net_def->op_size(); ++idx) {
    OperatorDef def(net_def->op(idx));
    if (!def.has_device_option() && net_has_device_option) *def.mutable_device_option() = net_def->device_option();
    std::unique_ptr<OperatorBase> op = CreateOperator(def, ws, idx);
    for (int i = 0; i < def.input_size(); ++i)
      for (const auto& ei : external_input_)
        if (ei == def.input(i)) external_input_blob_[ei] = op->Input(i);
    for (int i = 0; i < def.output_size(); ++i)
      for (const auto& eo : external_output_)
        if (eo == def.output(i)) external_output_blob_[eo] = op->Output(i);
    operators_.emplace_back(std::move(op));
  }
  skipped_.assign(operators_.size(), false);
  // Gemm -> activation folding: the consumer must be the only reader of the producer's output
  const Argument* fuse_arg = ArgumentHelper::Find(net_def->arg_, "fuse_gemm_activation");
  const char* env = getenv("BLAZE_NO_FUSION");
  const bool fuse = !(env && atoi(env) != 0) && !(fuse_arg && fuse_arg->has_i && fuse_arg->i == 0);
  if (fuse) {
    for (size_t i = 0; i + 1 < operators_.size(); ++i) {
      auto* producer = dynamic_cast<FusableProducer*>(operators_[i].get());
      if (!producer || skipped_[i]) continue;
      const OperatorDef& pd = operators_[i]->operator_def();
      const OperatorDef& cd = operators_[i + 1]->operator_def();
      if (pd.output_size() != 1 || cd.input_size() < 1 || cd.input(0) != pd.output(0)) continue;
      const std::string& mid = pd.output(0);
      bool other_reader = false;
      for (size_t j = 0; j < operators_.size(); ++j) {
        if (j == i + 1) continue;
        for (const auto& in : operators_[j]->operator_def().input()) other_reader |= (j != i && in == mid);
      }
      bool is_output = false;
      for (const auto& eo : external_output_) is_output |= (eo == mid && cd.output(0) != mid);
      if (other_reader || is_output) continue;
      if (producer->TryFuse(operators_[i + 1].get())) skipped_[i + 1] = true;
    }
    FuseFcHeads();
    PackSiblingFcs();
    AliasConcatInputs();
    InterleaveAssignBlocks();
    FuseConcatPieces();
    FuseWeightedPools();
    FuseConcatsIntoFcs();
    ChainNarrowFcs();
    FuseConcatsIntoWeightedPools();
    MergeSiblingEmbeddings();
  }
}

// Readers of a tensor name among all operators -- skipped ones too: an operator that another one has taken over still
// runs, through its host, and reads what its definition names -- except `folded`, the activation a layer has folded
// into its own epilogue (written in place it names the layer's output as its input).
int SimpleNet::ReadersOf(const std::string& name, const OperatorBase* folded) const {
  int readers = 0;
  for (const auto& op : operators_) {
    if (op.get() == folded) continue;
    for (const auto& in : op->operator_def().input()) readers += (in == name);
  }
  return readers;
}

// FC layer (with its folded activation) -> FC layer of at most 8 outputs (with its folded Softmax / Sigmoid), the
// first one's result read by nothing else: one launch (graph.h, StackableFc::CanHostHead).  Switch: fuse_fc_head: 0.
void SimpleNet::FuseFcHeads() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "fuse_fc_head");
  if (arg && arg->has_i && arg->i == 0) return;
  for (size_t i = 0; i < operators_.size(); ++i) {
    auto* first = skipped_[i] ? nullptr : dynamic_cast<StackableFc*>(operators_[i].get());
    int n1 = 0;
    if (!first || !first->CanHostHead(&n1)) continue;
    size_t j = i + 1;
    while (j < operators_.size() && skipped_[j]) ++j;  // (the first layer's folded activation)
    if (j >= operators_.size()) break;
    auto* second = dynamic_cast<StackableFc*>(operators_[j].get());
    if (!second || !second->CanBeHead(n1)) continue;
    const std::string& mid = first->StackOutputOp()->operator_def().output(0);
    if (operators_[j]->operator_def().input(0) != mid) continue;
    OperatorBase* out_op = first->StackOutputOp();
    const int readers = ReadersOf(mid, out_op != operators_[i].get() ? out_op : nullptr);
    bool is_output = false;
    for (const auto& eo : external_output_) is_output |= (eo == mid);
    if (readers != 1 || is_output) continue;
    first->AbsorbHead(second);
    skipped_[j] = true;
  }
}

// Mul -> MatMul(transA) [+ ReduceSum of the MatMul's second input over axis 1] -> the MatMul alone (graph.h,
// WeightedPoolHost).  The Mul is taken over when its output is read only by the MatMul and is no output of the net; the
// ReduceSum when it comes after the MatMul and nothing in between writes the tensor both read.  Switch:
// fuse_weighted_pool: 0.
void SimpleNet::FuseWeightedPools() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "fuse_weighted_pool");
  if (arg && arg->has_i && arg->i == 0) return;
  auto readers_of = [&](const std::string& name) {
    int readers = 0;
    for (size_t j = 0; j < operators_.size(); ++j)
      for (const auto& in : operators_[j]->operator_def().input()) readers += (in == name);
    for (const auto& eo : external_output_) readers += (eo == name);
    return readers;
  };
  for (size_t m = 0; m < operators_.size(); ++m) {
    auto* host = skipped_[m] ? nullptr : dynamic_cast<WeightedPoolHost*>(operators_[m].get());
    if (!host || !host->WeightedPoolEligible()) continue;
    const OperatorDef& md = operators_[m]->operator_def();
    if (md.input_size() != 2) continue;
    // the Mul: last writer of Input(0) before the MatMul
    int mul = -1;
    for (int j = (int)m - 1; j >= 0 && mul < 0; --j)
      for (const auto& out : operators_[j]->operator_def().output())
        if (out == md.input(0)) mul = j;
    if (mul >= 0) {
      const OperatorDef& pd = operators_[mul]->operator_def();
      bool ok = !skipped_[mul] && operators_[mul]->type() == "Mul" && pd.input_size() == 2 && pd.output_size() == 1 &&
                readers_of(md.input(0)) == 1 && pd.output(0) != pd.input(0) && pd.output(0) != pd.input(1);
      // nothing between the Mul and the MatMul may overwrite what the Mul reads
      for (size_t k = mul + 1; k < m && ok; ++k)
        for (const auto& out : operators_[k]->operator_def().output()) ok &= (out != pd.input(0) && out != pd.input(1));
      if (!ok) mul = -1;
    }
    int red = -1;
    for (size_t j = m + 1; j < operators_.size() && red < 0; ++j) {
      const OperatorDef& rd = operators_[j]->operator_def();
      bool writes = false;
      for (const auto& out : rd.output()) writes |= (out == md.input(1));
      if (writes) break;  // the history changes here: a later ReduceSum sums something else
      if (skipped_[j] || operators_[j]->type() != "ReduceSum" || rd.input_size() != 1 || rd.input(0) != md.input(1)) continue;
      if (ArgumentHelper::GetSingle<int>(rd.arg(), "axis", 0) != 1 || ArgumentHelper::GetSingle<int>(rd.arg(), "keepdims", 1) != 0) continue;
      // moved up to the MatMul's position: its output must not be something an operator in between still reads or writes
      bool ok = rd.output_size() == 1;
      for (size_t k = m; k < j && ok; ++k) {
        for (const auto& in : operators_[k]->operator_def().input()) ok &= (in != rd.output(0));
        for (const auto& out : operators_[k]->operator_def().output()) ok &= (out != rd.output(0));
      }
      if (ok) red = (int)j;
    }
    if (mul < 0 && red < 0) continue;
    host->AdoptWeightedPool(mul >= 0 ? operators_[mul].get() : nullptr, red >= 0 ? operators_[red].get() : nullptr);
    if (mul >= 0) skipped_[mul] = true;
    if (red >= 0) skipped_[red] = true;
  }
}

// MatMul that runs as a weighted pool -> Reshape of its [B, 1, C] result to [B, C] -> Concat (axis 1) of that with the
// adopted ReduceSum's result and at most one more tensor: the MatMul's launch writes the Concat's output (graph.h,
// WeightedPoolHost::AdoptTailConcat).  The Reshape's and the ReduceSum's results must be read by the Concat alone, the
// other tensor must be final before the MatMul, and nothing between the MatMul and the Concat may touch the Concat's
// output.  Switch: fuse_concat_into_weighted_pool: 0.
void SimpleNet::FuseConcatsIntoWeightedPools() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "fuse_concat_into_weighted_pool");
  if (arg && arg->has_i && arg->i == 0) return;
  auto readers_of = [&](const std::string& name) {
    int readers = 0;
    for (size_t j = 0; j < operators_.size(); ++j)
      for (const auto& in : operators_[j]->operator_def().input()) readers += (in == name);
    for (const auto& eo : external_output_) readers += (eo == name);
    return readers;
  };
  for (size_t m = 0; m < operators_.size(); ++m) {
    auto* host = skipped_[m] ? nullptr : dynamic_cast<WeightedPoolHost*>(operators_[m].get());
    if (!host || !host->WeightedPoolEligible()) continue;
    const OperatorDef& md = operators_[m]->operator_def();
    if (md.output_size() != 1 || readers_of(md.output(0)) != 1) continue;
    int r = -1;
    for (size_t j = m + 1; j < operators_.size() && r < 0; ++j)
      if (!skipped_[j] && operators_[j]->type() == "Reshape" && operators_[j]->operator_def().input_size() == 2 &&
          operators_[j]->operator_def().input(0) == md.output(0) && operators_[j]->operator_def().output_size() == 1)
        r = (int)j;
    if (r < 0) continue;
    const std::string& att = operators_[r]->operator_def().output(0);
    if (att == md.output(0) || readers_of(att) != 1) continue;
    int c = -1;
    for (size_t j = r + 1; j < operators_.size() && c < 0; ++j)
      for (const auto& in : operators_[j]->operator_def().input())
        if (in == att) c = (int)j;
    if (c < 0 || skipped_[c] || operators_[c]->type() != "Concat") continue;
    const OperatorDef& cd = operators_[c]->operator_def();
    if (ArgumentHelper::GetSingle<int>(cd.arg(), "axis", 1) != 1 || cd.output_size() != 1) continue;
    OperatorBase* red = host->AdoptedReduceSum();
    int att_pos = -1, sum_pos = -1, copy_pos = -1;
    bool ok = true;
    for (int i = 0; i < cd.input_size() && ok; ++i) {
      const std::string& name = cd.input(i);
      if (name == att) {
        ok = att_pos < 0;
        att_pos = i;
      } else if (red && name == red->operator_def().output(0)) {
        ok = sum_pos < 0 && readers_of(name) == 1;
        sum_pos = i;
      } else {
        ok = copy_pos < 0 && name != cd.output(0);
        copy_pos = i;
      }
    }
    if (!ok || att_pos < 0) continue;
    // the copied tensor is final when the MatMul runs; the Concat's output is untouched between the two
    for (size_t k = m; k < (size_t)c && ok; ++k) {
      const OperatorDef& kd = operators_[k]->operator_def();
      for (const auto& out : kd.output()) ok &= (out != cd.output(0)) && (copy_pos < 0 || out != cd.input(copy_pos));
      for (const auto& in : kd.input()) ok &= (in != cd.output(0));
    }
    if (!ok) continue;
    host->AdoptTailConcat(operators_[c].get(), operators_[r].get(), att_pos, sum_pos, copy_pos);
    skipped_[r] = skipped_[c] = true;
  }
}

// Concat (last axis) -> Gemm, the Concat's output read by nothing else: the Gemm takes the Concat over (graph.h,
// ConcatForFc) and computes its rows while it loads them.  Nothing between the two may overwrite what the Concat, or an
// elementwise producer the Concat has taken over, reads.  Switch: fuse_concat_into_fc: 0.
void SimpleNet::FuseConcatsIntoFcs() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "fuse_concat_into_fc");
  if (arg && arg->has_i && arg->i == 0) return;
  for (size_t g = 0; g < operators_.size(); ++g) {
    auto* fc = skipped_[g] ? nullptr : dynamic_cast<ConcatAdopter*>(operators_[g].get());
    if (!fc || !fc->CanAdoptConcat()) continue;
    const std::string& in = operators_[g]->operator_def().input(0);
    int c = -1;
    for (int j = (int)g - 1; j >= 0 && c < 0; --j)
      for (const auto& out : operators_[j]->operator_def().output())
        if (out == in) c = j;
    if (c < 0 || skipped_[c] || dynamic_cast<ConcatForFc*>(operators_[c].get()) == nullptr) continue;
    int readers = 0;
    for (size_t j = 0; j < operators_.size(); ++j)
      for (const auto& name : operators_[j]->operator_def().input()) readers += (name == in);
    for (const auto& eo : external_output_) readers += (eo == in);
    if (readers != 1 || workspace_->HasConstantBlob(in)) continue;
    // what the Concat reads, directly or through a producer it runs itself
    std::set<std::string> sources(operators_[c]->operator_def().input().begin(), operators_[c]->operator_def().input().end());
    // (to a fixed point: a taken-over producer may itself read another one's result, BroadcastTo -> Sub -> Concat)
    for (size_t before = 0; before != sources.size();) {
      before = sources.size();
      for (int j = c - 1; j >= 0; --j) {
        if (!skipped_[j]) continue;
        bool feeds = false;
        for (const auto& out : operators_[j]->operator_def().output()) feeds |= sources.count(out) != 0;
        if (feeds) sources.insert(operators_[j]->operator_def().input().begin(), operators_[j]->operator_def().input().end());
      }
    }
    bool clean = true;
    for (size_t k = c + 1; k < g && clean; ++k)
      for (const auto& out : operators_[k]->operator_def().output()) clean &= sources.count(out) == 0;
    if (!clean) continue;
    fc->AdoptConcat(operators_[c].get());
    skipped_[c] = true;
  }
}

// A Gemm that computes its Concat input itself -> the narrow Gemm that reads only its result: the second (and the skinny
// layer it may host) runs in the first one's launch (graph.h, ConcatAdopter::CanChainNext).  Switch: chain_narrow_fcs: 0.
void SimpleNet::ChainNarrowFcs() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "chain_narrow_fcs");
  if (arg && arg->has_i && arg->i == 0) return;
  for (size_t i = 0; i < operators_.size(); ++i) {
    auto* first = skipped_[i] ? nullptr : dynamic_cast<ConcatAdopter*>(operators_[i].get());
    auto* first_fc = first ? dynamic_cast<StackableFc*>(operators_[i].get()) : nullptr;
    if (!first || !first_fc || !first->HasAdoptedConcat()) continue;
    size_t j = i + 1;
    while (j < operators_.size() && skipped_[j]) ++j;  // (the first layer's folded activation)
    if (j >= operators_.size()) break;
    if (!first->CanChainNext(operators_[j].get())) continue;
    const std::string& mid = first_fc->StackOutputOp()->operator_def().output(0);
    if (operators_[j]->operator_def().input(0) != mid) continue;
    OperatorBase* out_op = first_fc->StackOutputOp();
    const int readers = ReadersOf(mid, out_op != operators_[i].get() ? out_op : nullptr);
    bool is_output = false;
    for (const auto& eo : external_output_) is_output |= (eo == mid);
    if (readers != 1 || is_output) continue;
    first->AdoptNext(operators_[j].get());
    skipped_[j] = true;
  }
}

// Sibling Gemm operators (same input, same attributes, constant weights of one shape) -> one launch over the stacked
// weights (graph.h, SiblingFc).  Switch: pack_sibling_gemms: 0.
void SimpleNet::PackSiblingFcs() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "pack_sibling_gemms");
  if (arg && arg->has_i && arg->i == 0) return;
  std::map<std::string, std::vector<size_t>> groups;
  for (size_t i = 0; i < operators_.size(); ++i) {
    auto* fc = skipped_[i] ? nullptr : dynamic_cast<SiblingFc*>(operators_[i].get());
    if (!fc) continue;
    const std::string key = fc->SiblingKey();
    if (!key.empty()) groups[key].push_back(i);
  }
  for (auto& kv : groups) {
    std::vector<size_t>& idx = kv.second;
    if (idx.size() < 2) continue;
    // the shared input must not be rewritten between the first and the last sibling (an in-place operator in between)
    const std::string& in = operators_[idx[0]]->operator_def().input(0);
    bool clean = true;
    for (size_t k = idx.front() + 1; k < idx.back() && clean; ++k)
      for (const auto& out : operators_[k]->operator_def().output()) clean &= (out != in);
    // a later sibling's result appears where the first sibling runs: nothing from there up to the sibling's own place may
    // read or write that name (or the name of the tensor between the sibling and its folded activation)
    for (size_t m = 1; m < idx.size() && clean; ++m) {
      std::set<std::string> names(operators_[idx[m]]->operator_def().output().begin(), operators_[idx[m]]->operator_def().output().end());
      if (auto* st = dynamic_cast<StackableFc*>(operators_[idx[m]].get()))
        names.insert(st->StackOutputOp()->operator_def().output().begin(), st->StackOutputOp()->operator_def().output().end());
      for (size_t k = idx.front(); k < idx[m] && clean; ++k) {
        for (const auto& in : operators_[k]->operator_def().input()) clean &= names.count(in) == 0;
        for (const auto& out : operators_[k]->operator_def().output()) clean &= names.count(out) == 0;
      }
    }
    if (!clean) continue;
    std::vector<SiblingFc*> others;
    for (size_t m = 1; m < idx.size(); ++m) {
      others.push_back(dynamic_cast<SiblingFc*>(operators_[idx[m]].get()));
      skipped_[idx[m]] = true;
    }
    dynamic_cast<SiblingFc*>(operators_[idx[0]].get())->AbsorbSiblings(others);
  }
}

// Concat inputs that are outputs of elementwise operators -> pieces computed by the Concat itself (graph.h,
// ConcatPieceSource).  A producer is taken over when its output is read only by the Concat -- or, as a shape
// reference (second input of BroadcastTo), by another producer the same Concat takes over -- is neither an output of the
// net nor written in place, and nothing between the producer and the Concat overwrites the producer's inputs.
void SimpleNet::FuseConcatPieces() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "fuse_concat_pieces");
  if (arg && arg->has_i && arg->i == 0) return;
  auto is_external_output = [&](const std::string& name) {
    for (const auto& eo : external_output_)
      if (eo == name) return true;
    return false;
  };
  for (size_t c = 0; c < operators_.size(); ++c) {
    auto* host = skipped_[c] ? nullptr : dynamic_cast<ConcatPieceHost*>(operators_[c].get());
    if (!host) continue;
    const OperatorDef& cd = operators_[c]->operator_def();
    // candidate producer of every input: the last operator before the Concat that writes the name
    std::vector<int> producer(cd.input_size(), -1);
    for (int i = 0; i < cd.input_size(); ++i) {
      int readers_in_concat = 0;
      for (const auto& in : cd.input()) readers_in_concat += (in == cd.input(i));
      if (readers_in_concat != 1 || is_external_output(cd.input(i)) || workspace_->HasConstantBlob(cd.input(i))) continue;
      for (size_t j = 0; j < c; ++j) {
        if (skipped_[j]) continue;
        const OperatorDef& pd = operators_[j]->operator_def();
        for (const auto& out : pd.output())
          if (out == cd.input(i)) producer[i] = (int)j;
      }
      if (producer[i] < 0) continue;
      const OperatorDef& pd = operators_[producer[i]]->operator_def();
      bool ok = dynamic_cast<ConcatPieceSource*>(operators_[producer[i]].get()) != nullptr && pd.output_size() == 1;
      for (const auto& in : pd.input()) ok &= (in != pd.output(0));  // in place: the "intermediate" is somebody's input
      // nothing between the producer and the Concat may overwrite what the producer reads
      for (size_t k = producer[i] + 1; k < c && ok; ++k)
        for (const auto& out : operators_[k]->operator_def().output())
          for (const auto& in : pd.input()) ok &= (out != in);
      if (!ok) producer[i] = -1;
    }
    // drop candidates whose output has a reader other than the Concat or a shape-only read by another candidate
    for (bool changed = true; changed;) {
      changed = false;
      for (int i = 0; i < cd.input_size(); ++i) {
        if (producer[i] < 0) continue;
        bool ok = true;
        for (size_t j = 0; j < operators_.size() && ok; ++j) {
          if (j == c) continue;
          const OperatorDef& rd = operators_[j]->operator_def();
          for (int k = 0; k < rd.input_size() && ok; ++k) {
            if (rd.input(k) != cd.input(i)) continue;
            bool shape_only_by_candidate = rd.type() == "BroadcastTo" && k == 1;
            bool is_candidate = false;
            for (int q = 0; q < cd.input_size(); ++q) is_candidate |= (producer[q] == (int)j);
            ok = shape_only_by_candidate && is_candidate && !skipped_[j];
          }
        }
        if (!ok) {
          producer[i] = -1;
          changed = true;
        }
      }
    }
    int taken = 0;
    for (int i = 0; i < cd.input_size(); ++i) taken += producer[i] >= 0;
    if (taken == 0 || cd.input_size() > BZ_CEW_MAX) continue;
    for (int i = 0; i < cd.input_size(); ++i) {
      if (producer[i] < 0) continue;
      host->AdoptProducer(i, operators_[producer[i]].get(), producer[i]);
      skipped_[producer[i]] = true;
    }
  }
}

// Embedding kAssign blocks -> Reshape [batch, T, D] -> Concat(axis 2): the Embedding writes into the Concat's output
// (graph.h, AssignInterleaver).  Every tensor on the way is read by nothing else and is no output of the net; each
// Reshape's target is a constant [-1 | 0, T, D_i] with the block's own T and D_i.  Switch: interleave_assign_blocks: 0.
void SimpleNet::InterleaveAssignBlocks() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "interleave_assign_blocks");
  if (arg && arg->has_i && arg->i == 0) return;
  auto readers_of = [&](const std::string& name) {
    int readers = 0;
    for (size_t j = 0; j < operators_.size(); ++j)
      for (const auto& in : operators_[j]->operator_def().input()) readers += (in == name);
    for (const auto& eo : external_output_) readers += (eo == name);
    return readers;
  };
  auto producer_of = [&](const std::string& name, size_t before, int* out_idx) {
    for (size_t j = before; j-- > 0;) {
      const OperatorDef& pd = operators_[j]->operator_def();
      for (int o = 0; o < pd.output_size(); ++o)
        if (pd.output(o) == name) {
          *out_idx = o;
          return (int)j;
        }
    }
    return -1;
  };
  for (size_t c = 0; c < operators_.size(); ++c) {
    if (skipped_[c] || operators_[c]->type() != "Concat") continue;
    const OperatorDef& cd = operators_[c]->operator_def();
    if (ArgumentHelper::GetSingle<int>(cd.arg(), "axis", 1) != 2 || cd.input_size() < 2 || cd.output_size() != 1) continue;
    int emb = -1, T = 0;
    std::vector<int> blocks, reshapes;
    bool ok = true;
    for (int i = 0; i < cd.input_size() && ok; ++i) {
      int o = 0, eo = 0, fo = 0;
      const int r = readers_of(cd.input(i)) == 1 ? producer_of(cd.input(i), c, &o) : -1;
      if (r < 0 || skipped_[r] || operators_[r]->type() != "Reshape") {
        ok = false;
        break;
      }
      const OperatorDef& rd = operators_[r]->operator_def();
      const int e = rd.input_size() == 2 && readers_of(rd.input(0)) == 1 && rd.output(0) != rd.input(0) ? producer_of(rd.input(0), r, &eo) : -1;
      const int f = rd.input_size() == 2 ? producer_of(rd.input(1), operators_.size(), &fo) : -1;
      auto* host = e >= 0 && !skipped_[e] ? dynamic_cast<AssignInterleaver*>(operators_[e].get()) : nullptr;
      int t = 0, d = 0;
      std::vector<int> target;
      if (f >= 0 && operators_[f]->type() == "ConstantFill" && workspace_->HasConstantBlob(rd.input(1)))
        target = ArgumentHelper::GetRepeated<int>(operators_[f]->operator_def().arg(), "value");
      if (!host || (emb >= 0 && e != emb) || !host->AssignBlock(eo, &t, &d) || (T != 0 && t != T) || target.size() != 3 ||
          target[0] > 0 || target[1] != t || target[2] != d || std::find(blocks.begin(), blocks.end(), eo) != blocks.end()) {
        ok = false;
        break;
      }
      emb = e;
      T = t;
      blocks.push_back(eo);
      reshapes.push_back(r);
    }
    if (!ok) continue;
    // the Concat's output appears earlier than before: nothing up to the Concat may touch that name
    const std::string& out = cd.output(0);
    for (size_t j = 0; j < c && ok; ++j) {
      for (const auto& in : operators_[j]->operator_def().input()) ok &= (in != out);
      for (const auto& o2 : operators_[j]->operator_def().output()) ok &= (o2 != out);
    }
    for (const auto& ei : external_input_) ok &= (ei != out);
    if (!ok) continue;
    dynamic_cast<AssignInterleaver*>(operators_[emb].get())->InterleaveInto(blocks, operators_[c]->Output(0));
    for (int r : reshapes) skipped_[r] = true;
    skipped_[c] = true;
  }
}

// Embedding operators whose inputs no operator of the net produces: the later ones are run by the first (graph.h,
// EmbeddingSibling), which may then look everything up in one launch.  Moved up to the first one's position, a later
// operator's outputs must not be named by anything in between.  Switch: merge_sibling_embeddings: 0.
void SimpleNet::MergeSiblingEmbeddings() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "merge_sibling_embeddings");
  if (arg && arg->has_i && arg->i == 0) return;
  auto produced = [&](const std::string& name) {
    for (const auto& op : operators_)
      for (const auto& out : op->operator_def().output())
        if (out == name) return true;
    return false;
  };
  auto from_outside = [&](size_t i) {
    for (const auto& in : operators_[i]->operator_def().input())
      if (produced(in)) return false;
    return true;
  };
  int host = -1;
  for (size_t i = 0; i < operators_.size(); ++i) {
    if (skipped_[i] || dynamic_cast<EmbeddingSibling*>(operators_[i].get()) == nullptr || !from_outside(i)) continue;
    if (host < 0) {
      host = (int)i;
      continue;
    }
    bool ok = true;
    for (size_t k = host; k < i && ok; ++k) {
      const OperatorDef& kd = operators_[k]->operator_def();
      for (const auto& out : operators_[i]->operator_def().output()) {
        for (const auto& name : kd.input()) ok &= (name != out);
        for (const auto& name : kd.output()) ok &= (name != out);
      }
    }
    if (!ok) continue;
    dynamic_cast<EmbeddingSibling*>(operators_[host].get())->AdoptSibling(operators_[i].get());
    skipped_[i] = true;
  }
}

// Concat along the last axis of 2-D tensors whose inputs are all either blocks of an Embedding operator or
// external inputs, each read by nothing else: the inputs become column slices of the Concat's output (their
// producers write in place) and the Concat has nothing left to copy.
void SimpleNet::AliasConcatInputs() {
  const Argument* arg = ArgumentHelper::Find(net_def_->arg_, "alias_concat_inputs");
  if (arg && arg->has_i && arg->i == 0) return;
  for (size_t c = 0; c < operators_.size(); ++c) {
    if (skipped_[c] || operators_[c]->type() != "Concat") continue;
    const OperatorDef& cd = operators_[c]->operator_def();
    if (ArgumentHelper::GetSingle<int>(cd.arg(), "axis", 1) != 1 || cd.input_size() < 1) continue;
    std::vector<Blob*> children;
    std::vector<TIndex> widths;
    bool ok = true;
    for (int i = 0; i < cd.input_size() && ok; ++i) {
      const std::string& name = cd.input(i);
      int readers = 0;
      for (size_t j = 0; j < operators_.size(); ++j)
        for (const auto& in : operators_[j]->operator_def().input()) readers += (in == name);
      for (const auto& eo : external_output_) readers += (eo == name);
      if (readers != 1 || workspace_->HasConstantBlob(name)) {
        ok = false;
        break;
      }
      TIndex w = 0;
      bool produced = false;
      for (size_t j = 0; j < c && !produced; ++j) {
        const OperatorDef& pd = operators_[j]->operator_def();
        for (int o = 0; o < pd.output_size(); ++o) {
          if (pd.output(o) != name) continue;
          produced = true;
          w = operators_[j]->StaticOutputCols(o);
          if (operators_[j]->type() != "Embedding" || w == 0) ok = false;
        }
      }
      bool external = false;
      for (const auto& ei : external_input_) external |= (ei == name);
      if (!produced && !external) ok = false;
      children.push_back(operators_[c]->Input(i));
      widths.push_back(w);
    }
    if (ok) Blob::LinkColumnSlices(operators_[c]->Output(0), children, widths);
  }
}

bool SimpleNet::RunImpl() {
  for (size_t i = 0; i < operators_.size(); ++i) {
    if (skipped_[i]) continue;
    auto& op = operators_[i];
    bool res;
    if (profile_) {
      auto t0 = std::chrono::steady_clock::now();
      res = op->Run();
      op->WaitStream();
      op->set_last_run_us(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
    } else {
      res = op->Run();
    }
    if (!res) {
      LOG_ERROR("Operator failed, name=%s type=%s", op->name().c_str(), op->type().c_str());
      return false;
    }
  }
  return true;
}

REGISTER_NET(simple, SimpleNet);

}  // namespace blaze
