// graph.h -- Workspace (blob ownership per model / per predictor) and the sequential executor.
//
// Minimal re-creation of the callers of the operator boundary: blaze/graph/workspace.h:24-196 (constants are
// shared by every net of a workspace, activations belong to one net), blaze/graph/net.h:21-178 and
// blaze/graph/simple_net.cc:9-46 (create one operator per OperatorDef, run them in order on stream 0, wait
// for the stream).  The DAG / hybrid executors, observers beyond a wall-clock profile, and the batching
// schedulers are not part of this build; run_mode strings other than "simple" fall back to this executor.
#pragma once

#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

#include "blaze/operator.h"
#include "blaze/sparse_puller.h"

struct bz_concat_ew_desc;

namespace blaze {

class Net;

class Workspace {
 public:
  ~Workspace();
  Blob* CreateConstantBlob(const std::string& name, const DeviceOption& device_option, bool* newblob = nullptr);
  Blob* CreateBlob(const std::string& name, const DeviceOption& device_option, bool* newblob = nullptr);
  bool HasConstantBlob(const std::string& name) const { return constant_fill_blob_map_.count(name) != 0; }
  const std::map<std::string, Blob*>& constant_blobs() const { return constant_fill_blob_map_; }

  void SetSparsePuller(std::shared_ptr<store::SparsePuller> p) { sparse_puller_ = p; }
  std::shared_ptr<store::SparsePuller>& GetSparsePuller() { return sparse_puller_; }

  void Init(const NetDef& net_def);
  std::shared_ptr<Net> CreateNet();
  std::shared_ptr<Net> CreateNet(const char* net_file);  // text or binary NetDef (tests, small models)

  DataType input_data_type(const std::string& input_name) const;
  bool has_input_info(const std::string& input_name) const { return input_info_map_.count(input_name) != 0; }
  const ValueInfo& input_info(const std::string& input_name) const;
  std::shared_ptr<NetDef>& net_def() { return net_def_; }

 private:
  void RecycleBlobMap();
  std::map<std::string, Blob*> constant_fill_blob_map_;  // shared by all predictors of the model
  std::map<std::string, Blob*> blob_map_;                // the blobs of the net being built
  std::set<Blob*> blob_recycle_bins_;                    // blobs of nets built earlier
  std::shared_ptr<NetDef> net_def_;
  std::map<std::string, DataType> input_data_type_map_;
  std::unordered_map<std::string, ValueInfo> input_info_map_;
  std::shared_ptr<store::SparsePuller> sparse_puller_;
  std::mutex mutex_;
};

class Net {
 public:
  Net(const std::shared_ptr<const NetDef>& net_def, Workspace* ws);
  virtual ~Net() noexcept {}
  // reset, run every operator, wait for the device (net.h:33-49); exceptions propagate to the Predictor
  virtual bool Run();
  // Run in two halves: Launch queues every operator on the calling thread's stream and returns; StreamOfLastLaunch is
  // that stream (null when the net has no device operator).  Run = Launch + waiting for the stream.
  bool Launch();
  void* StreamOfLastLaunch();
  const std::vector<std::string>& external_input() const { return external_input_; }
  const std::vector<std::string>& external_output() const { return external_output_; }
  Blob* external_input_blob(const std::string& name) const;
  Blob* external_output_blob(const std::string& name) const;
  const ValueInfo& external_input_info(const std::string& name) const { return workspace_->input_info(name); }
  bool has_external_input_info(const std::string& name) const { return workspace_->has_input_info(name); }
  std::vector<std::unique_ptr<OperatorBase>>& GetOperators() { return operators_; }
  Workspace* workspace() { return workspace_; }
  // "profile" observer: per-operator host wall time of the last Run, as chrome-trace JSON
  void set_profile(bool on) { profile_ = on; }
  std::string DumpProfile() const;
  const std::string& name() const { return name_; }

 protected:
  virtual bool RunImpl() = 0;
  std::string name_;
  std::shared_ptr<const NetDef> net_def_;
  Workspace* workspace_;
  std::vector<std::unique_ptr<OperatorBase>> operators_;
  std::vector<std::string> external_input_, external_output_;
  std::map<std::string, Blob*> external_input_blob_, external_output_blob_;
  bool profile_ = false;
};

class SimpleNet : public Net {
 public:
  SimpleNet(const std::shared_ptr<const NetDef>& net_def, Workspace* ws);

 protected:
  bool RunImpl() override;
  void AliasConcatInputs();
  void FuseConcatPieces();
  void FuseFcHeads();
  void PackSiblingFcs();
  void FuseWeightedPools();
  void FuseConcatsIntoWeightedPools();
  void FuseConcatsIntoFcs();
  void ChainNarrowFcs();
  int ReadersOf(const std::string& name, const OperatorBase* folded) const;
  void InterleaveAssignBlocks();
  void MergeSiblingEmbeddings();
  std::vector<bool> skipped_;  // ops folded into their producer's epilogue, or run by the operator that took them over
};

typedef Registry<std::shared_ptr<Net>, const std::shared_ptr<const NetDef>&, Workspace*> NetRegistryType;
NetRegistryType* NetRegistry();
#define REGISTER_NET(name, ...)                                                                                    \
  namespace {                                                                                                      \
  static ::blaze::Registerer<std::shared_ptr<::blaze::Net>, const std::shared_ptr<const ::blaze::NetDef>&,         \
                             ::blaze::Workspace*>                                                                  \
      ANONYMOUS_VARIABLE(g_net_##name)(#name, ::blaze::NetRegistry(),                                              \
                                       [](const std::shared_ptr<const ::blaze::NetDef>& d, ::blaze::Workspace* w) { \
                                         return std::shared_ptr<::blaze::Net>(new __VA_ARGS__(d, w));              \
                                       });                                                                         \
  }

// An operator whose kernel can apply the following activation operator in its epilogue.  SimpleNet offers each
// (producer, consumer) pair; when TryFuse accepts, the consumer is skipped at run time.  The reference fuses
// sibling GEMMs but never GEMM + activation (blaze/graph/pattern/); numerically the fused result equals the
// composition Activation(Gemm(x, W, b)).
class FusableProducer {
 public:
  virtual ~FusableProducer() {}
  virtual bool TryFuse(OperatorBase* consumer) = 0;
};

// An FC operator (Gemm, with or without a folded activation) that can run a following skinny layer in its own launch.
class StackableFc {
 public:
  virtual ~StackableFc() {}
  // the operator whose Output(0) receives this layer's result (the folded activation, else the operator itself)
  virtual OperatorBase* StackOutputOp() = 0;
  // A layer of at most 256 outputs followed by a layer of at most 8 (the logit / score of a tower): the second is
  // computed in the first one's launch from the output tile still on chip (bz_fc_desc.head_*), and what the first
  // layer would have stored for it is not stored at all.
  virtual bool CanHostHead(int* n_out) = 0;   // static eligibility of the first layer; reports its width
  virtual bool CanBeHead(int k_in) = 0;       // static eligibility of the second layer for a first layer of width k_in
  virtual void AbsorbHead(StackableFc* head) = 0;
};

// Sibling FC operators -- Gemms that read the same input with constant weights of one shape and the same arguments
// (and the same kind of folded activation) -- run as ONE launch over the stacked weights, each writing its own output
// matrix: what the reference's ParallelGemm fusion does by rewriting them into FusedParallelGemm + Split
// (blaze/graph/pattern/in_parallel/parallel_gemm_fusion_pattern_impl.cc:20-98, CanFusion :118-140).  SimpleNet groups
// operators with equal SiblingKey(); the first of a group absorbs the others, which are skipped.  The outputs become
// views of one buffer the first operator owns (no Split launch).  Same sums per output element as the separate
// launches up to the tile shape the wider launch picks: equal within one rounding of the tensor type.
class SiblingFc {
 public:
  virtual ~SiblingFc() {}
  // empty: not eligible.  Otherwise everything that must agree between siblings, the input blob included.
  virtual std::string SiblingKey() = 0;
  virtual void AbsorbSiblings(const std::vector<SiblingFc*>& others) = 0;
};

// A Concat along the last axis whose inputs are elementwise results (Add / Sub / Mul / Div / BroadcastTo of tensors
// that differ only by broadcasting over rows) read by nothing else: the Concat computes those pieces while it
// writes them (bz_concat_ew) and their operators are skipped -- the attention unit's [q, k, q-k, q*k] in one launch
// without the intermediate tensors.  Same bits as the separate operators.
struct ConcatPiece {
  Blob* x = nullptr;
  Blob* y = nullptr;            // null: the piece is x itself, broadcast over rows where its dims are 1
  int op = 0;                   // bz_ew_op; BZ_EW_ASSIGN when y is null
  std::vector<TIndex> shape;    // of the piece
};
class ConcatPieceSource {  // implemented by the elementwise operators
 public:
  virtual ~ConcatPieceSource() {}
  // Describes Output(0) without computing it and gives the output blob its shape (no memory), so that operators that
  // only read that shape still work.  False: this instance cannot be described (in-place output, type mismatch).
  virtual bool DescribePiece(ConcatPiece* piece) = 0;
};
class ConcatPieceHost {  // implemented by Concat
 public:
  virtual ~ConcatPieceHost() {}
  // input `input_idx` is the output of `producer` (net position `position`), which the net will not run any more
  virtual void AdoptProducer(int input_idx, OperatorBase* producer, int position) = 0;
};

// A Concat along the last axis -- with or without elementwise producers it has taken over -- whose only reader is an FC
// operator: the FC computes the Concat's rows itself while it loads them (bz_fc_desc.a_pieces) and the tensor between
// the two is never stored (the attention unit's [q, k, q-k, q*k] in front of its first layer).  Same values as the
// separate operators up to the order of the layer's K sum.
class ConcatForFc {  // implemented by Concat
 public:
  virtual ~ConcatForFc() {}
  // Describes Output(0) as pieces without computing it and gives the output blob its shape (no memory).  False: the
  // inputs do not fit the piece model; nothing has been touched.
  virtual bool DescribeAsPieces(bz_concat_ew_desc* desc) = 0;
};
class ConcatAdopter {  // implemented by Gemm
 public:
  virtual ~ConcatAdopter() {}
  virtual bool CanAdoptConcat() = 0;  // static part: constant 2-byte weight of a shape the kernel takes, no transposed A
  virtual void AdoptConcat(OperatorBase* concat) = 0;
  virtual bool HasAdoptedConcat() const = 0;
  // The narrow layer after such a layer (with the skinny layer it may already host) in the same launch
  // (bz_fc_desc.next): the attention MLP 4E -> 80 -> 40 -> 1 as one kernel.  `next` reads only this layer's result, and
  // nothing else does.
  virtual bool CanChainNext(OperatorBase* next) = 0;  // static part
  virtual void AdoptNext(OperatorBase* next) = 0;
};

// Embedding blocks that are each one kAssign item [batch, T * D_i] -> Reshape [batch, T, D_i] (read by nothing else) ->
// Concat(axis 2) of exactly these, in any block order: the Embedding writes every item at its columns of the Concat's
// output [batch, T, sum D_i] (bz_embed_slot.assign_pitch) and the Reshapes and the Concat are skipped.  Same bits: the
// rows only land somewhere else.  DIN's history of (item, category, shop) embeddings.
class AssignInterleaver {  // implemented by Embedding
 public:
  virtual ~AssignInterleaver() {}
  // whether output block idx is a single kAssign item; its positions a sample and columns a position
  virtual bool AssignBlock(int idx, int* trunc_num, int* dim) const = 0;
  // blocks (in the Concat's input order) go to `target` from now on; the blocks themselves only keep their shape
  virtual void InterleaveInto(const std::vector<int>& blocks, Blob* target) = 0;
};

// MatMul(transA) of a weight column [B, T, 1] with a history [B, T, C] whose weight is the product of two equally
// shaped tensors (score * mask) read by nothing else, optionally next to a ReduceSum of the same history over T:
// the MatMul computes all of it in one launch (bz_weighted_pool) and the Mul and the ReduceSum are skipped.  Same
// bits as the separate operators.
class WeightedPoolHost {  // implemented by MatMul
 public:
  virtual ~WeightedPoolHost() {}
  virtual bool WeightedPoolEligible() const = 0;  // static part: transA, no transB
  // mul: producer of Input(0) (may be null); reduce_sum: a ReduceSum(axis 1, keepdims 0) of Input(1) (may be null)
  virtual void AdoptWeightedPool(OperatorBase* mul, OperatorBase* reduce_sum) = 0;
  virtual OperatorBase* AdoptedReduceSum() const = 0;
  // The Concat (last axis of 2-D tensors) that joins this MatMul's result - flattened from [B, 1, C] to [B, C] by
  // `reshape`, which nothing else reads - with the adopted ReduceSum's result and at most one other tensor that is
  // final before the MatMul runs (DIN: [target, sum, att] in front of the main MLP): the launch writes its outputs
  // into the Concat's output and copies the other tensor there; the Reshape and the Concat do not run.  Positions are
  // indices among the Concat's inputs, -1 = the Concat has no such input.
  virtual void AdoptTailConcat(OperatorBase* concat, OperatorBase* reshape, int att_pos, int sum_pos, int copy_pos) = 0;
};

// Embedding operators of one net that read only tensors from outside the net: the first one (in order) takes the later
// ones over and looks everything up in ONE pooling launch when that costs the taken-over lookups nothing - every
// operator of the group is either all kAssign (the generic kernel's work anyway) or light (at most two ids a sample on
// average in each of its feature groups, where the specialised kernel's deeper walk buys nothing); decided per run,
// otherwise each operator launches as before.  DIN: the target item's lookup rides in the history's launch.
class EmbeddingSibling {  // implemented by Embedding
 public:
  virtual ~EmbeddingSibling() {}
  virtual void AdoptSibling(OperatorBase* other) = 0;
};

}  // namespace blaze
