// embedding_op.cc -- the Embedding operator on the accelerator.
//
// Same operator as the reference's CPU-only one (blaze/operator/sparse_op/embedding/embedding_op.{h,cc}): it
// parses the text `embedding_config` argument (blaze/proto/embedding.proto), lays every block out as a
// [batch, stride] tensor whose items sit at their running offsets (embedding_op.h:65-108), maps the input
// triples <fg>.ids / <fg>.values / <fg>.segments to feature groups by stripping the suffixes
// (embedding_op.cc:31-59), validates them (embedding_op.h:110-139) and hands one SparsePullerInput /
// SparsePullerOutput per feature group to the store (embedding_op.h:188-247).  Here the blobs are device
// memory and the store launches one pooling kernel for all groups on the operator's stream.
#include "blaze/graph.h"
#include "blaze/operator.h"

namespace blaze {

using store::SparsePuller;

template <class Context>
class EmbeddingOp final : public Operator<Context>, public AssignInterleaver, public EmbeddingSibling {
 public:
  USE_OPERATOR_FUNCTIONS(Context);

  void AdoptSibling(OperatorBase* other) override {
    auto* e = dynamic_cast<EmbeddingOp*>(other);
    BLAZE_CONDITION_THROW(e != nullptr && e != this, "AdoptSibling: not another Embedding operator of this device");
    siblings_.push_back(e);
  }
  int LaunchesOfLastRun() const override { return launches_; }

  bool AssignBlock(int idx, int* trunc_num, int* dim) const override {
    if (idx < 0 || (size_t)idx >= config_.block_config.size()) return false;
    const auto& items = config_.block_config[idx].embedding_block_config_item;
    if (items.size() != 1 || items[0].udf_type != kAssign || items[0].trunc_num <= 0) return false;
    auto it = fg_config_idx_.find(items[0].feature_group);
    if (it == fg_config_idx_.end()) return false;
    *trunc_num = items[0].trunc_num;
    *dim = config_.feature_group_config[it->second].dim;
    return *dim > 0;
  }
  void InterleaveInto(const std::vector<int>& blocks, Blob* target) override {
    Interleaved g;
    g.target = target;
    g.blocks = blocks;
    int t = 0, d = 0;
    for (int b : blocks) {
      BLAZE_CONDITION_THROW(AssignBlock(b, &t, &d) && (g.trunc_num == 0 || g.trunc_num == t), "block ", b, " is no kAssign item of ", g.trunc_num, " positions");
      g.trunc_num = t;
      g.col.push_back(g.total);
      g.total += d;
    }
    interleaved_.push_back(g);
  }

  EmbeddingOp(const OperatorDef& def, Workspace* workspace) : Operator<Context>(def, workspace) {
    sparse_puller_ = workspace->GetSparsePuller();
    const std::string config_str = OperatorBase::GetSingleArgument<std::string>("embedding_config", "");
    try {
      ParseEmbeddingConfigText(config_str, &config_);
    } catch (std::exception& e) {
      BLAZE_THROW("Parse embedding config failed:", config_str, " (", e.what(), ")");
    }
    InitLayout();
    BLAZE_CONDITION_THROW(def.input_size() % 3 == 0, "input size is not multiply of 3");
    BLAZE_CONDITION_THROW((size_t)def.output_size() == config_.block_config.size(), "embedding op has ", def.output_size(),
                          " outputs but the config has ", config_.block_config.size(), " blocks");
    for (int i = 0, p = 0; i < def.input_size(); i += 3, ++p) {
      const std::string& id_name = def.input(i);
      const std::string& value_name = def.input(i + 1);
      const std::string& num_name = def.input(i + 2);
      const std::string fg = id_name.substr(0, id_name.rfind(kIdSuffix));
      const std::string value_fg = value_name.substr(0, value_name.rfind(kValueSuffix));
      const std::string num_fg = num_name.substr(0, num_name.rfind(kIdNumSuffix));
      BLAZE_CONDITION_THROW(!fg.empty(), "invalid input name=", id_name);
      BLAZE_CONDITION_THROW(!value_fg.empty(), "invalid input name=", value_name);
      BLAZE_CONDITION_THROW(!num_fg.empty(), "invalid input name=", num_name);
      BLAZE_CONDITION_THROW(fg == value_fg && fg == num_fg, "id input name=", id_name, " value_input_name=", value_name,
                            " num_input_name=", num_name);
      input_fg_idx_[fg] = p;
    }
    // extension: the element type of the blocks (default: that of the values, as the schema infers)
    out_dtype_ = OperatorBase::GetSingleArgument<int>("out_dtype", 0);
    if (out_dtype_ != 0) {
      BLAZE_CONDITION_THROW(out_dtype_ == kFloat || out_dtype_ == kFloat16, "out_dtype=", out_dtype_);
      for (auto* out : this->outputs_) out->set_data_type((DataType)out_dtype_);
    }
  }

  bool RunOnDevice() override {
    hipStream_t st = context_.hip_stream();
    Prepare(st);
    launches_ = 1;
    if (siblings_.empty()) {
      Pull(puller_in_, puller_out_, st, &cache_);
      return true;
    }
    // the operators this one runs (graph.h, EmbeddingSibling): everything in one launch when none of them loses by it
    bool together = RidesFree();
    for (EmbeddingOp* e : siblings_) {
      e->Prepare(st);
      together &= e->RidesFree() && e->sparse_puller_ == sparse_puller_;
    }
    if (!together) {
      Pull(puller_in_, puller_out_, st, &cache_);
      for (EmbeddingOp* e : siblings_) e->Pull(e->puller_in_, e->puller_out_, st, &e->cache_);
      launches_ += (int)siblings_.size();
      return true;
    }
    size_t n = puller_in_.size();
    for (EmbeddingOp* e : siblings_) n += e->puller_in_.size();
    merged_in_.resize(n);  // (element-wise assignment below: the strings and item lists keep their storage run to run)
    merged_out_.resize(n);
    size_t at = 0;
    auto append = [&](const EmbeddingOp* e) {
      for (size_t i = 0; i < e->puller_in_.size(); ++i, ++at) {
        merged_in_[at] = e->puller_in_[i];
        merged_out_[at] = e->puller_out_[i];
      }
    };
    append(this);
    for (EmbeddingOp* e : siblings_) append(e);
    Pull(merged_in_, merged_out_, st, &merged_cache_);
    return true;
  }

 protected:
  struct BlockInfo {
    int block_idx, item_idx;
  };

  // InitFeatureGroupConfigMeta + InitEmbeddingBlockConfigMeta (embedding_op.h:53-94)
  void InitLayout() {
    for (size_t i = 0; i < config_.feature_group_config.size(); ++i) fg_config_idx_[config_.feature_group_config[i].feature_group] = i;
    fg_blocks_.resize(config_.feature_group_config.size());
    for (size_t i = 0; i < config_.block_config.size(); ++i) {
      auto& block = config_.block_config[i];
      size_t offset = 0;
      for (size_t j = 0; j < block.embedding_block_config_item.size(); ++j) {
        auto& item = block.embedding_block_config_item[j];
        auto it = fg_config_idx_.find(item.feature_group);
        BLAZE_CONDITION_THROW(it != fg_config_idx_.end(), "feature group config not exist, fg: ", item.feature_group);
        fg_blocks_[it->second].push_back({(int)i, (int)j});
        item.offset = offset;
        offset += ItemStride(item, config_.feature_group_config[it->second].dim);
      }
      block.stride = offset;
    }
  }

  // GetEmbeddingBlockItemStride (embedding_op.h:97-108)
  static int ItemStride(const EmbeddingBlockConfigItem& item, int dim) {
    switch (item.udf_type) {
      case kSum:
      case kAvg:
        return dim;
      case kAssign:
        return dim * item.trunc_num;
      default:
        BLAZE_THROW("Unsupported udf type: ", item.udf_type);
    }
  }

  void CheckValid() {
    BLAZE_CONDITION_THROW(this->InputSize() % 3 == 0, "embedding op input size=", this->InputSize());
    for (int i = 0; i < this->InputSize(); ++i) {
      Blob* x = this->Input(i % 3);
      Blob* y = this->Input(i);
      BLAZE_CONDITION_THROW(x->data_type() == y->data_type(), "x->data_type()=", x->data_type(), " y->data_type()=", y->data_type());
    }
    for (int i = 0; i < this->InputSize() / 3; ++i) {
      Blob* id_blob = this->Input(i * 3);
      Blob* value_blob = this->Input(i * 3 + 1);
      BLAZE_CONDITION_THROW(id_blob->size() == value_blob->size(), "id_blob->size()=", id_blob->size(),
                            " value_blob->size()=", value_blob->size(), " ", this->def_.DebugString());
    }
  }

  // output blocks: [batch, stride]; all groups of a block must agree on the batch (embedding_op.h:155-184)
  void Setup() {
    needs_zero_.assign(config_.block_config.size(), false);
    for (auto& g : interleaved_) g.shaped = false;
    for (size_t i = 0; i < config_.block_config.size(); ++i) {
      size_t batch = 0;
      bool first = true;
      for (const auto& item : config_.block_config[i].embedding_block_config_item) {
        auto it = input_fg_idx_.find(item.feature_group);
        BLAZE_CONDITION_THROW(it != input_fg_idx_.end(), "feature group of block item is not in input list, fg: ", item.feature_group);
        const size_t n = this->Input((int)it->second * 3 + 2)->size();
        if (!first && n != batch) BLAZE_THROW("batch size of each feature group in block must be equal");
        batch = n;
        first = false;
      }
      Blob* out = this->Output((int)i);
      int slot = 0;
      if (Interleaved* g = GroupOf((int)i, &slot)) {
        // lives in the group's tensor: the block keeps its shape for whoever asks, and no memory
        out->SetShapeOnly({(TIndex)batch, (TIndex)config_.block_config[i].stride});
        BLAZE_CONDITION_THROW(!g->shaped || (TIndex)batch == g->batch, "blocks of one history tensor with ", batch, " and ", g->batch,
                              " samples");
        if (!g->shaped) {
          g->shaped = true;
          g->batch = (TIndex)batch;
          g->target->set_data_type((DataType)out->data_type());
          g->target->Reshape({(TIndex)batch, (TIndex)g->trunc_num, (TIndex)g->total});
        }
        continue;
      }
      out->Reshape({(TIndex)batch, (TIndex)config_.block_config[i].stride});
    }
  }
  struct Interleaved {
    Blob* target = nullptr;
    std::vector<int> blocks;   // in column order
    std::vector<TIndex> col;   // first column of each
    TIndex total = 0;          // columns of a position
    int trunc_num = 0;
    TIndex batch = 0;          // samples of the run being set up, once `shaped`
    bool shaped = false;
  };
  Interleaved* GroupOf(int block, int* slot) {
    for (auto& g : interleaved_)
      for (size_t k = 0; k < g.blocks.size(); ++k)
        if (g.blocks[k] == block) {
          *slot = (int)k;
          return &g;
        }
    return nullptr;
  }

  TIndex StaticOutputCols(int idx) const override {
    return idx >= 0 && (size_t)idx < config_.block_config.size() ? (TIndex)config_.block_config[idx].stride : 0;
  }

  // everything of a run but the lookup itself: checks, output shapes, the puller structs, zero fills (on `st`)
  void Prepare(hipStream_t st) {
    CheckValid();
    Blob* id = this->Input(0);
    Blob* value = this->Input(1);
    Blob* id_num = this->Input(2);
    // ID_TYPE_SWITCH / TYPE_SWITCH of embedding_op.cc:70-82; the QED store then insists on int64 / float / int32
    BLAZE_CONDITION_THROW(id->data_type() == kInt64 || id->data_type() == kInt32, "Unsupported type:", id->data_type());
    BLAZE_CONDITION_THROW(value->data_type() == kFloat, "Unsupported type:", value->data_type());
    BLAZE_CONDITION_THROW(id_num->data_type() == kInt64 || id_num->data_type() == kInt32, "Unsupported type:", id_num->data_type());
    BLAZE_CONDITION_THROW(sparse_puller_ != nullptr, "no sparse puller: call LoadSparseModelWeight before creating predictors");
    BLAZE_CONDITION_THROW(sparse_puller_->on_device(), "the Embedding operator of this build needs a device sparse puller "
                          "(qed_hip_sparse_puller); there is no host fallback");
    Setup();
    RunEmbedding(id->data_type(), value->data_type(), id_num->data_type(), st);
  }
  void Pull(const std::vector<store::SparsePullerInput>& in, std::vector<store::SparsePullerOutput>& out, hipStream_t st,
            std::unique_ptr<SparsePuller::DeviceCache>* cache) {
    auto status = sparse_puller_->GetOnStream(in, out, st, cache);
    BLAZE_CONDITION_THROW(status == store::kOK, "pull data failed, status=", status);
  }
  // whether a launch shared with other operators costs this one's lookups nothing: every fed feature group either has
  // only kAssign items (the generic kernel's work in any launch) or at most two ids a sample on average
  bool RidesFree() const {
    for (size_t i = 0; i < puller_in_.size(); ++i) {
      const auto& in = puller_in_[i];
      if (fg_input_[i] < 0 || in.in_item.empty()) continue;
      bool all_assign = true;
      for (const auto& item : in.in_item) all_assign &= item.udf_type == store::kAssign;
      if (!all_assign && in.key_size > 2 * in.key_num_size) return false;
    }
    return true;
  }

  void RunEmbedding(int key_type, int value_type, int num_type, hipStream_t st) {
    const size_t n_fg = config_.feature_group_config.size();
    // the puller structs live in the operator: their names, item lists and input positions are the same every run,
    // only pointers and sizes change (a request-sized forward pass should not pay 2 allocations per feature group)
    std::vector<store::SparsePullerInput>& inputs = puller_in_;
    std::vector<store::SparsePullerOutput>& outputs = puller_out_;
    if (inputs.size() != n_fg) {
      inputs.assign(n_fg, store::SparsePullerInput());
      outputs.assign(n_fg, store::SparsePullerOutput());
      fg_input_.assign(n_fg, -1);
      for (size_t i = 0; i < n_fg; ++i) {
        inputs[i].name = config_.feature_group_config[i].table_name;
        auto it = input_fg_idx_.find(config_.feature_group_config[i].feature_group);
        if (it != input_fg_idx_.end()) fg_input_[i] = (int)it->second;
      }
    }
    for (size_t i = 0; i < n_fg; ++i) {
      const auto& fgc = config_.feature_group_config[i];
      auto& in = inputs[i];
      auto& out = outputs[i];
      if (fg_input_[i] < 0) {
        // a configured group that is not fed: its items' columns stay zero (embedding_op.h:204-208)
        for (const auto& bi : fg_blocks_[i]) needs_zero_[bi.block_idx] = true;
        continue;
      }
      const int idx = fg_input_[i];
      Blob* ids = this->Input(idx * 3);
      Blob* values = this->Input(idx * 3 + 1);
      Blob* nums = this->Input(idx * 3 + 2);
      in.key = ids->data();
      in.key_size = ids->size();
      in.key_num = nums->data();
      in.key_num_size = nums->size();
      in.value = values->data();
      in.key_type = key_type;
      in.value_type = value_type;
      in.num_type = num_type;
      in.dim = fgc.dim;
      in.in_item.resize(fg_blocks_[i].size());
      out.out_item.resize(fg_blocks_[i].size());
      for (size_t j = 0; j < fg_blocks_[i].size(); ++j) {
        const auto& bi = fg_blocks_[i][j];
        const auto& item = config_.block_config[bi.block_idx].embedding_block_config_item[bi.item_idx];
        in.in_item[j].udf_type = (store::UDFType)item.udf_type;
        in.in_item[j].trunc_direction = (store::TruncDirection)item.trunc_direction;
        in.in_item[j].trunc_num = item.trunc_num;
        Blob* block = this->Output(bi.block_idx);
        out.out_type = block->data_type();
        int slot = 0;
        if (Interleaved* g = GroupOf(bi.block_idx, &slot)) {
          // position p of sample b at row b * T + p of the group's tensor, columns col .. col + dim
          out.out_item[j].out = (char*)g->target->data() + g->col[slot] * DataTypeSize(block->data_type());
          out.out_item[j].stride = (size_t)(g->trunc_num * g->total);
          out.out_item[j].assign_pitch = (size_t)g->total;
          continue;
        }
        out.out_item[j].out = (char*)block->data() + item.offset * DataTypeSize(block->data_type());
        // a block that lives inside a Concat's output has that tensor's row pitch
        out.out_item[j].stride = block->pitch() ? (int)block->pitch() : config_.block_config[bi.block_idx].stride;
        out.out_item[j].assign_pitch = 0;
      }
    }
    for (size_t b = 0; b < needs_zero_.size(); ++b)
      if (needs_zero_[b]) {
        Blob* block = this->Output((int)b);
        const size_t es = DataTypeSize(block->data_type());
        int slot = 0;
        if (Interleaved* g = GroupOf((int)b, &slot)) {
          int t = 0, d = 0;
          AssignBlock((int)b, &t, &d);
          HIP_CHECK(hipMemset2DAsync((char*)g->target->data() + g->col[slot] * es, g->total * es, 0, d * es,
                                     (size_t)(g->batch * g->trunc_num), st));
        } else if (block->pitch())
          HIP_CHECK(hipMemset2DAsync(block->data(), block->pitch() * es, 0, block->shape()[1] * es, block->shape()[0], st));
        else
          HIP_CHECK(hipMemsetAsync(block->data(), 0, block->size() * es, st));
      }
  }

  std::shared_ptr<SparsePuller> sparse_puller_;
  EmbeddingConfig config_;
  std::vector<std::vector<BlockInfo>> fg_blocks_;            // feature group -> the block items it feeds
  std::unordered_map<std::string, size_t> input_fg_idx_;    // feature group -> input triple index
  std::unordered_map<std::string, size_t> fg_config_idx_;   // feature group -> config index
  std::vector<bool> needs_zero_;
  std::vector<Interleaved> interleaved_;
  std::vector<store::SparsePullerInput> puller_in_;    // reused every run (RunEmbedding)
  std::vector<store::SparsePullerOutput> puller_out_;
  std::vector<int> fg_input_;  // feature group -> position of its triple among the inputs, -1 = not fed
  std::unique_ptr<SparsePuller::DeviceCache> cache_;
  // the Embedding operators this one runs, the joined structs of a shared launch and that launch's own slot cache
  std::vector<EmbeddingOp*> siblings_;
  std::vector<store::SparsePullerInput> merged_in_;
  std::vector<store::SparsePullerOutput> merged_out_;
  std::unique_ptr<SparsePuller::DeviceCache> merged_cache_;
  int launches_ = 1;
  int out_dtype_ = 0;
};

REGISTER_HIP_OPERATOR(Embedding, EmbeddingOp<HIPContext>);

// Input: (ids, values, segments) per feature group.  Output: dense embedding blocks.
OPERATOR_SCHEMA(Embedding)
    .NumInputs(3, INT_MAX)
    .NumOutputs(1, INT_MAX)
    .TypeInferenceFunction([](const OperatorDef& def, const std::vector<DataType>& input_type) {
      return std::vector<DataType>(def.output_size(), input_type[1]);
    })
    .SetDoc("The embedding op.");

}  // namespace blaze
