// dense_ops.cc -- Gemm, MatMul, FusedParallelGemm, FusedParallelMatMul on the accelerator.
//
// Operator-level behaviour (argument names and defaults, shape rules, error messages) follows the reference:
//   Gemm                 blaze/operator/op/gemm_op.h:21-153       (transA, transB, alpha=1, beta=1; 2-D or 3-D A)
//   MatMul               blaze/operator/op/matmul_op.h:21-171     (transA, transB, from_deepnet; numpy broadcast, outer rank <= 1)
//   FusedParallelGemm    blaze/operator/fused_op/fused_parallel_gemm_op.h:32-184
//   FusedParallelMatMul  blaze/operator/fused_op/fused_parallel_matmul_op.h:24-200
// The arithmetic goes to the kernel layer (include/blaze_hip.h): an FC is one bz_fc_fused launch (MFMA, fp32
// accumulate, bias and -- when the following activation operator was folded in -- activation in the epilogue);
// batched products are bz_gemm_strided_batched.
#include "blaze/graph.h"
#include "blaze/operator.h"
#include "blaze_hip.h"

namespace blaze {

namespace {

int BzType(int data_type) {
  switch (data_type) {
    case kFloat: return BZ_F32;
    case kFloat16: return BZ_F16;
    default: BLAZE_THROW("Unsupported type: ", data_type);
  }
}

// A device buffer derived from a blob (packed weight, fp32 copy of a parameter), rebuilt when the blob moves.
struct Derived {
  void* ptr = nullptr;
  size_t bytes = 0;
  const Blob* src = nullptr;
  uint64_t version = ~0ull;
  ~Derived() {
    if (ptr) (void)hipFree(ptr);
  }
  bool Stale(const Blob* b) const { return ptr == nullptr || src != b || version != b->version(); }
  void Resize(size_t n) {
    if (n > bytes) {
      if (ptr) (void)hipFree(ptr);
      HIP_CHECK(hipMalloc(&ptr, n));
      bytes = n;
    }
  }
  void Mark(const Blob* b) {
    src = b;
    version = b->version();
  }
};

// fp32 view of a parameter blob (bias, PRelu slope, Dice gamma/mean/var): fp32 blobs are used in place, fp16
// ones are widened once on the device (exact) and cached.  Constant blobs are immutable after load; for other
// producers the copy is redone every run.
const float* AsFloatParam(Blob* b, Derived* cache, bool constant, hipStream_t st) {
  if (b->data_type() == kFloat) return b->as<float>();
  BLAZE_CONDITION_THROW(b->data_type() == kFloat16, "Unsupported type: ", b->data_type());
  if (!constant || cache->Stale(b)) {
    const int n = (int)b->size();
    const int64_t ld = (n + 7) / 8 * 8;
    cache->Resize(ld * sizeof(float));
    BZ_CHECK(bz_fc_pack_weight(b->data(), BZ_F16, 1, n, 1, cache->ptr, BZ_F32, ld, st));
    cache->Mark(b);
  }
  return (const float*)cache->ptr;
}

// One FC:  y[M,N] = act(alpha * op(A) * op(B) + beta * bias) through bz_fc_fused.
struct FcCall {
  // operands
  const void* a = nullptr;
  const bz_concat_ew_desc* a_pieces = nullptr;  // instead of a: the rows as pieces computed on the fly (bz_fc_desc.a_pieces)
  const bz_fc_next* next = nullptr;             // with a_pieces: a second layer in the same launch
  int a_rows = 0, a_cols = 0;  // as stored
  bool trans_a = false;
  Blob* b_blob = nullptr;
  const void* b = nullptr;     // b_blob->data() + offset
  int b_rows = 0, b_cols = 0;  // as stored
  bool trans_b = false;
  bool b_constant = false;
  int dtype = kFloat;
  const float* bias = nullptr;
  int bias_rows = 0;
  void* y = nullptr;
  int y_dtype = kFloat;
  float alpha = 1.f, beta = 1.f;
  // epilogue
  int act = BZ_ACT_NONE;
  const float *p0 = nullptr, *p1 = nullptr, *p2 = nullptr;
  int act_size = 0;
  bool dice_nosqrt = false;
  float act_alpha = 0.f;
  // P sibling layers on one input in one launch (bz_fc_desc.n_split): B holds P weights stacked on dim 0 -- [P*N, K]
  // under trans_b, else [P*K, N] -- bias / activation parameters are [P*N], slice p's output starts p * y_split_stride
  // elements after y
  int slices = 1;
  int64_t y_split_stride = 0;
  // a second, skinny layer in the same launch (bz_fc_desc.head_*); y may then be null
  const void* head_w = nullptr;
  int64_t head_ldw = 0;
  const float* head_bias = nullptr;
  void* head_y = nullptr;
  int head_n = 0, head_act = BZ_ACT_NONE, head_y_dtype = kFloat;
};

// false only with a_pieces, when the kernel does not take them (nothing has been launched then)
bool RunFc(const FcCall& c, Derived* packed_b, Derived* packed_a, hipStream_t st) {
  const int P = c.slices;
  const int M = c.trans_a ? c.a_cols : c.a_rows;
  const int K = c.trans_a ? c.a_rows : c.a_cols;
  const int Ns = c.trans_b ? c.b_rows / P : c.b_cols;  // columns of one slice
  const int N = Ns * P;
  const int bt = BzType(c.dtype);
  const int es = (int)DataTypeSize(c.dtype);
  const int chunk = 16 / es;
  bz_fc_desc d;
  memset(&d, 0, sizeof(d));
  // A: row major [M,K] is used in place; a transposed A is re-laid out K-contiguous first
  if (c.trans_a) {
    const int64_t lda = (K + 7) / 8 * 8;
    packed_a->Resize((size_t)M * lda * es);
    BZ_CHECK(bz_fc_pack_weight(c.a, bt, 0, K, M, packed_a->ptr, bt, lda, st));
    d.a = packed_a->ptr;
    d.lda = lda;
  } else {
    d.a = c.a;
    d.lda = K;
  }
  // W: [N,K] with aligned rows is used in place (stacked slices under trans_b are exactly that), anything else is
  // packed (once for constants), slice by slice when the slices are stacked [K,N] matrices
  if (c.trans_b && (K % chunk == 0) && ((uintptr_t)c.b % 16 == 0)) {
    d.w = c.b;
    d.ldw = K;
  } else {
    const int64_t ldw = (K + 7) / 8 * 8;
    const bool redo = !c.b_constant || packed_b->Stale(c.b_blob) || packed_b->bytes < (size_t)N * ldw * es;
    if (redo) {
      packed_b->Resize((size_t)N * ldw * es);
      if (c.trans_b) {
        BZ_CHECK(bz_fc_pack_weight(c.b, bt, 1, K, N, packed_b->ptr, bt, ldw, st));
      } else {
        for (int p = 0; p < P; ++p)
          BZ_CHECK(bz_fc_pack_weight((const char*)c.b + (size_t)p * K * Ns * es, bt, 0, K, Ns,
                                     (char*)packed_b->ptr + (size_t)p * Ns * ldw * es, bt, ldw, st));
      }
      packed_b->Mark(c.b_blob);
    }
    d.w = packed_b->ptr;
    d.ldw = ldw;
  }
  if (P > 1) {
    d.n_split = Ns;
    d.y_split_stride = c.y_split_stride;
  }
  d.bias = c.bias;
  d.bias_rows = c.bias_rows;
  d.y = c.y;
  d.ldy = Ns;
  d.m = M;
  d.n = N;
  d.k = K;
  d.in_dtype = bt;
  d.out_dtype = BzType(c.y_dtype);
  d.act = c.act;
  d.act_p0 = c.p0;
  d.act_p1 = c.p1;
  d.act_p2 = c.p2;
  d.act_size = c.act_size;
  d.dice_nosqrt = c.dice_nosqrt ? 1 : 0;
  d.alpha = c.alpha;
  d.beta = c.bias ? c.beta : 0.f;
  d.act_alpha = c.act_alpha;
  if (c.head_n > 0) {
    d.head_w = c.head_w;
    d.head_ldw = c.head_ldw;
    d.head_bias = c.head_bias;
    d.head_y = c.head_y;
    d.head_ldy = c.head_n;
    d.head_n = c.head_n;
    d.head_act = c.head_act;
    d.head_out_dtype = BzType(c.head_y_dtype);
  }
  if (c.a_pieces != nullptr) {
    d.a_pieces = c.a_pieces;
    d.next = c.next;
    d.a = nullptr;
    const int rc = bz_fc_fused(&d, st);
    if (rc == BZ_ENOTSUP) return false;
    BZ_CHECK(rc);
    return true;
  }
  BZ_CHECK(bz_fc_fused(&d, st));
  return true;
}

}  // namespace

// ------------------------------------------------------------------------------------------ Gemm
template <class Context>
class GemmOp : public Operator<Context>, public FusableProducer, public StackableFc, public SiblingFc, public ConcatAdopter {
 public:
  USE_OPERATOR_FUNCTIONS(Context);

  GemmOp(const OperatorDef& def, Workspace* workspace) : Operator<Context>(def, workspace) {
    transa_ = OperatorBase::GetSingleArgument<bool>("transA", false);
    transb_ = OperatorBase::GetSingleArgument<bool>("transB", false);
    alpha_ = OperatorBase::GetSingleArgument<float>("alpha", 1.0);
    beta_ = OperatorBase::GetSingleArgument<float>("beta", 1.0);
    b_constant_ = workspace->HasConstantBlob(def.input(1));
    for (int i = 2; i < def.input_size(); ++i) c_constant_ = workspace->HasConstantBlob(def.input(i));
  }

  // Fold the activation operator that consumes this Gemm's output into the epilogue.  Only shapes the epilogue
  // expresses exactly are accepted: per-column parameters of size N (or a single PRelu slope).
  bool TryFuse(OperatorBase* consumer) override {
    if (!b_constant_ || this->Input(1)->shape().size() != 2) return false;
    const int N = (int)(transb_ ? this->Input(1)->shape()[0] : this->Input(1)->shape()[1]);
    const std::string& t = consumer->type();
    auto param_ok = [&](int idx, bool scalar_ok) {
      Blob* p = consumer->Input(idx);
      if (!this->workspace_->HasConstantBlob(consumer->operator_def().input(idx))) return false;
      return (int)p->size() == N || (scalar_ok && p->size() == 1);
    };
    if (t == "PRelu") {
      if (!param_ok(1, true)) return false;
      fused_act_ = BZ_ACT_PRELU;
    } else if (t == "Dice") {
      if (!param_ok(1, false) || !param_ok(2, false) || !param_ok(3, false)) return false;
      fused_act_ = BZ_ACT_DICE;
      fused_nosqrt_ = ArgumentHelper::GetSingle<bool>(consumer->operator_def().arg(), "nosqrt", false);
    } else if (t == "LeakyRelu") {
      fused_act_ = BZ_ACT_LEAKY_RELU;
      fused_alpha_ = ArgumentHelper::GetSingle<float>(consumer->operator_def().arg(), "alpha", 0.01f);
    } else if (t == "Sigmoid") {
      fused_act_ = BZ_ACT_SIGMOID;
    } else if (t == "Softmax") {
      const size_t axis = ArgumentHelper::GetSingle<size_t>(consumer->operator_def().arg(), "axis", 1);
      if (N > 8 || axis != 1 || this->Input(0)->shape().size() == 3) return false;
      fused_act_ = BZ_ACT_SOFTMAX;
    } else {
      return false;
    }
    fused_ = consumer;
    return true;
  }

  // ---- StackableFc: the operator whose output is this layer's result (its folded activation, or itself)
  OperatorBase* StackOutputOp() override { return fused_ ? fused_ : this; }

  // ---- a following layer of at most 8 outputs in this operator's launch
  bool CanHostHead(int* n_out) override {
    Blob* b = this->Input(1);
    if (!b_constant_ || transa_ || b->shape().size() != 2 || head_ != nullptr) return false;
    const int N = (int)(transb_ ? b->shape()[0] : b->shape()[1]);
    if (N > 256 || N <= 8 || N % 8 != 0) return false;
    if (this->InputSize() > 2 && (!c_constant_ || (int)this->Input(2)->size() != N)) return false;
    if (fused_ && fused_act_ == BZ_ACT_SOFTMAX) return false;
    *n_out = N;
    return true;
  }
  bool CanBeHead(int k_in) override {
    Blob* b = this->Input(1);
    if (!b_constant_ || transa_ || b->shape().size() != 2 || head_ != nullptr) return false;
    const int K = (int)(transb_ ? b->shape()[1] : b->shape()[0]);
    const int N = (int)(transb_ ? b->shape()[0] : b->shape()[1]);
    if (K != k_in || N > 8 || alpha_ != 1.f || beta_ != 1.f) return false;
    if (this->InputSize() > 2 && (!c_constant_ || (int)this->Input(2)->size() != N)) return false;
    if (fused_ && fused_act_ != BZ_ACT_SOFTMAX && fused_act_ != BZ_ACT_SIGMOID) return false;
    return true;
  }
  void AbsorbHead(StackableFc* head) override { head_ = static_cast<GemmOp*>(head); }

  // ---- sibling layers (same input, same shape of constant weight, same arguments) in one launch
  std::string SiblingKey() override {
    Blob* b = this->Input(1);
    if (!b_constant_ || transa_ || b->shape().size() != 2 || head_ != nullptr || !siblings_.empty()) return "";
    const TIndex N = transb_ ? b->shape()[0] : b->shape()[1];
    // (the stacked parameter vectors take N floats from every sibling: a bias of another length is no sibling's)
    if (this->InputSize() > 2 && (!c_constant_ || this->Input(2)->shape().size() != 1 || (TIndex)this->Input(2)->size() != N)) return "";
    if (fused_ && fused_act_ == BZ_ACT_SOFTMAX) return "";
    if (fused_ && fused_act_ == BZ_ACT_PRELU && (TIndex)fused_->Input(1)->size() != N) return "";  // a scalar slope is per layer
    Blob* y = fused_ ? fused_->Output(0) : this->Output(0);
    if (y->pitch() != 0 || y == this->Input(0)) return "";
    std::stringstream ss;
    ss << this->def_.input(0) << "|" << b->shape()[0] << "x" << b->shape()[1] << "|" << b->data_type() << "|" << transb_ << "|"
       << alpha_ << "|" << beta_ << "|" << (this->InputSize() > 2 ? this->Input(2)->data_type() : -1) << "|"
       << (fused_ ? fused_act_ : -1) << "|" << fused_nosqrt_ << "|" << fused_alpha_ << "|" << y->data_type() << "|"
       << this->device_option().device_id();
    return ss.str();
  }
  void AbsorbSiblings(const std::vector<SiblingFc*>& others) override {
    siblings_.clear();
    for (SiblingFc* o : others) siblings_.push_back(static_cast<GemmOp*>(o));
  }

  // ---- the Concat that makes this layer's input, computed while it is loaded
  // (the static part of what bz_fc_desc.a_pieces takes: a 2-byte layer of 9..96 columns and at most 224 inputs)
  bool CanAdoptConcat() override {
    Blob* b = this->Input(1);
    if (!b_constant_ || transa_ || b->shape().size() != 2) return false;
    if (b->data_type() != kFloat16) return false;
    const TIndex K = transb_ ? b->shape()[1] : b->shape()[0], N = transb_ ? b->shape()[0] : b->shape()[1];
    if (this->InputSize() > 2 && (!c_constant_ || (TIndex)this->Input(2)->size() != N)) return false;
    return N > 8 && N <= 96 && K <= 224 && !(fused_ && fused_act_ == BZ_ACT_SOFTMAX);
  }
  void AdoptConcat(OperatorBase* concat) override { concat_ = concat; }
  bool HasAdoptedConcat() const override { return concat_ != nullptr; }
  bool CanChainNext(OperatorBase* next_op) override {
    auto* g = dynamic_cast<GemmOp*>(next_op);
    if (g == nullptr || concat_ == nullptr || head_ != nullptr || !siblings_.empty() || next_ != nullptr) return false;
    Blob* b0 = this->Input(1);
    Blob* b = g->Input(1);
    if (!g->b_constant_ || g->transa_ || b->shape().size() != 2 || b->data_type() != b0->data_type()) return false;
    if (!g->siblings_.empty() || g->concat_ != nullptr) return false;
    const TIndex N1 = transb_ ? b0->shape()[0] : b0->shape()[1];
    const TIndex K2 = g->transb_ ? b->shape()[1] : b->shape()[0], N2 = g->transb_ ? b->shape()[0] : b->shape()[1];
    if (K2 != N1 || N2 <= 8 || N2 > 64) return false;
    if (g->InputSize() > 2 && (!g->c_constant_ || (TIndex)g->Input(2)->size() != N2)) return false;
    if (g->fused_ && g->fused_act_ == BZ_ACT_SOFTMAX) return false;
    if (g->fused_ && g->fused_act_ == BZ_ACT_PRELU && (TIndex)g->fused_->Input(1)->size() != N2 && g->fused_->Input(1)->size() != 1) return false;
    return true;
  }
  void AdoptNext(OperatorBase* next_op) override { next_ = static_cast<GemmOp*>(next_op); }

  int LaunchesOfLastRun() const override { return launches_; }

  bool RunOnDevice() override {
    launches_ = 1;
    if (concat_ != nullptr) {
      if (siblings_.empty() && head_ == nullptr) {
        bz_concat_ew_desc pieces;
        auto* c = dynamic_cast<ConcatForFc*>(concat_);
        if (c != nullptr && c->DescribeAsPieces(&pieces)) {
          if (next_ != nullptr && RunSelf(false, &pieces, true)) return true;  // this layer, the next and its head
          if (RunSelf(false, &pieces)) return RunNextAlone();
        }
      }
      // a shape the one-launch form does not take: the Concat runs after all
      if (!concat_->Run(context_.stream_id())) return false;
      launches_ = 2;
      // (the paths below count their own launches from 1)
    }
    const int before = launches_ - 1;
    const bool ok = RunRest();
    launches_ += before;
    return ok && RunNextAlone();
  }

 protected:
  // the adopted next layer as launches of its own
  bool RunNextAlone() {
    if (next_ == nullptr) return true;
    if (!next_->Run(context_.stream_id())) return false;
    launches_ += next_->LaunchesOfLastRun() > 0 ? next_->LaunchesOfLastRun() : 1;
    return true;
  }
  bool RunRest() {
    launches_ = 1;
    if (!siblings_.empty()) {
      if (RunSiblings()) return true;
      // an input the one-launch form does not take (3-D, few columns): one launch per layer
      launches_ = 1 + (int)siblings_.size();
      if (!RunSelf(false)) return false;
      for (GemmOp* g : siblings_)
        if (!g->RunSelf(false)) return false;
      return true;
    }
    if (head_ != nullptr) {
      if (RunSelf(true)) return true;
      // an input the one-launch form does not take (unaligned rows, mixed types): one launch per layer
      return RunSelf(false) && head_->RunSelf(false);
    }
    return RunSelf(false);
  }

  // this layer and its absorbed siblings as one launch over the stacked weights; every layer's output blob becomes a
  // view of its slice of one buffer.  False (nothing launched) when the input is not a plain 2-D matrix.
  bool RunSiblings() {
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    if (a->shape().size() != 2 || a->pitch() != 0) return false;
    const int P = 1 + (int)siblings_.size();
    const TIndex M = a->shape()[0], K = a->shape()[1];
    const TIndex N = transb_ ? b->shape()[0] : b->shape()[1];
    if ((TIndex)P * N <= 8) return false;
    CheckValid();
    std::vector<GemmOp*> all = {this};
    all.insert(all.end(), siblings_.begin(), siblings_.end());
    hipStream_t st = context_.hip_stream();
    const int es = (int)DataTypeSize(b->data_type());
    const int bt = BzType(b->data_type());
    const int64_t ldw = (K + 7) / 8 * 8;
    // stacked constants, built once: weights [P*N, ldw], bias and activation parameters [P*N] fp32
    bool stale = sib_w_.ptr == nullptr;
    for (GemmOp* g : all) stale |= g->sib_src_ != g->Input(1) || g->sib_version_ != g->Input(1)->version();
    if (stale) {
      sib_w_.Resize((size_t)P * N * ldw * es);
      const bool has_bias = this->InputSize() > 2;
      const int n_params = !fused_ ? 0 : (fused_act_ == BZ_ACT_PRELU ? 1 : (fused_act_ == BZ_ACT_DICE ? 3 : 0));
      sib_f32_.Resize((size_t)(1 + n_params) * P * N * sizeof(float));
      for (int p = 0; p < P; ++p) {
        GemmOp* g = all[p];
        BZ_CHECK(bz_fc_pack_weight(g->Input(1)->data(), bt, transb_ ? 1 : 0, (int)K, (int)N, (char*)sib_w_.ptr + (size_t)p * N * ldw * es,
                                   bt, ldw, st));
        if (has_bias)
          HIP_CHECK(hipMemcpyAsync((float*)sib_f32_.ptr + (size_t)p * N, AsFloatParam(g->Input(2), &g->bias_f32_, true, st),
                                   N * sizeof(float), hipMemcpyDeviceToDevice, st));
        for (int q = 0; q < n_params; ++q)
          HIP_CHECK(hipMemcpyAsync((float*)sib_f32_.ptr + ((size_t)(1 + q) * P + p) * N,
                                   AsFloatParam(g->fused_->Input(1 + q), &g->p_f32_[q], true, st), N * sizeof(float),
                                   hipMemcpyDeviceToDevice, st));
        g->sib_src_ = g->Input(1);
        g->sib_version_ = g->Input(1)->version();
      }
    }
    Blob* y0 = fused_ ? fused_->Output(0) : this->Output(0);
    const size_t ys = DataTypeSize(y0->data_type());
    sib_y_.Resize((size_t)P * M * N * ys);
    for (int p = 0; p < P; ++p) {
      Blob* y = all[p]->fused_ ? all[p]->fused_->Output(0) : all[p]->Output(0);
      y->RefReshape({M, N}, (char*)sib_y_.ptr + (size_t)p * M * N * ys);
    }
    bz_fc_desc d;
    memset(&d, 0, sizeof(d));
    d.a = a->data();
    d.lda = K;
    d.w = sib_w_.ptr;
    d.ldw = ldw;
    d.y = sib_y_.ptr;
    d.ldy = N;
    d.n_split = (int)N;
    d.y_split_stride = (int64_t)M * N;
    d.m = (int)M;
    d.n = (int)(P * N);
    d.k = (int)K;
    d.in_dtype = bt;
    d.out_dtype = BzType(y0->data_type());
    d.alpha = alpha_;
    if (this->InputSize() > 2) {
      d.bias = sib_f32_.ptr;
      d.bias_rows = 1;
      d.beta = beta_;
    }
    if (fused_) {
      d.act = fused_act_;
      d.dice_nosqrt = fused_nosqrt_ ? 1 : 0;
      d.act_alpha = fused_alpha_;
      const float* base = (const float*)sib_f32_.ptr + (size_t)P * N;
      if (fused_act_ == BZ_ACT_PRELU) {
        d.act_p0 = base;
        d.act_size = d.n;
      } else if (fused_act_ == BZ_ACT_DICE) {
        d.act_p0 = base;
        d.act_p1 = base + (size_t)P * N;
        d.act_p2 = base + (size_t)2 * P * N;
        d.act_size = d.n;
      }
    }
    BZ_CHECK(bz_fc_fused(&d, st));
    return true;
  }

  // with_head: also compute head_'s layer in this launch and leave this layer's own output unstored; false when the
  // operands do not allow it (nothing has been launched then)
  // pieces: the input given as pieces computed on the fly (an adopted Concat); false when the kernel does not take them
  // chain: also run next_ (and the skinny layer it hosts) in this launch; this layer's and next_'s own outputs are then
  // not stored
  bool RunSelf(bool with_head, const bz_concat_ew_desc* pieces = nullptr, bool chain = false) {
    CheckValid();
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->InputSize() > 2 ? this->Input(2) : nullptr;
    Blob* y = fused_ ? fused_->Output(0) : this->Output(0);
    if (with_head) {
      const size_t es = DataTypeSize(a->data_type());
      const TIndex k = a->shape().back();
      if (a->data_type() != y->data_type() || a->data_type() != head_->Input(1)->data_type() || (k * es) % 16 != 0 ||
          (uintptr_t)a->data() % 16 != 0 || a->pitch() != 0)
        return false;
    }
    const auto& a_shape = a->shape();
    const auto& b_shape = b->shape();
    TIndex M = a_shape.size() == 3 ? a_shape[1] : a_shape[0];
    TIndex K = a_shape.size() == 3 ? a_shape[2] : a_shape[1];
    if (transa_) std::swap(M, K);
    const TIndex N = transb_ ? b_shape[0] : b_shape[1];
    TIndex rows = M;  // rows of the one 2-D product that realises the op
    Blob* hy = nullptr;
    if (with_head) {
      Blob* hb = head_->Input(1);
      const TIndex n2 = head_->transb_ ? hb->shape()[0] : hb->shape()[1];
      hy = head_->fused_ ? head_->fused_->Output(0) : head_->Output(0);
      if (a_shape.size() == 3)
        hy->Reshape({a_shape[0], M, n2});
      else
        hy->Reshape({M, n2});
    }
    if (a_shape.size() == 3) {
      if (with_head || chain)
        y->SetShapeOnly({a_shape[0], M, N});
      else
        y->Reshape({a_shape[0], M, N});
      // M == 1 collapses to a 2-D Gemm with M = batch (gemm_op.h:54-55); M > 1 with a shared weight is the
      // strided-batched case (stride_b = 0, :77-91), which over contiguous slices is again one 2-D product
      BLAZE_CONDITION_THROW(!transa_ || a_shape[0] == 1, "3-D Gemm with transA is not supported on this device");
      rows = a_shape[0] * M;
    } else if (with_head || chain) {
      y->SetShapeOnly({M, N});
    } else {
      y->Reshape({M, N});
    }
    hipStream_t st = context_.hip_stream();
    FcCall call;
    bz_fc_next nx;
    if (chain) {
      // next_ (with its folded activation) as bz_fc_next, the skinny layer it hosts through the head_* fields
      GemmOp* g = next_;
      Blob* b2 = g->Input(1);
      if (y->data_type() != a->data_type()) return false;
      const int es2 = (int)DataTypeSize(b2->data_type());
      const int n2 = (int)(g->transb_ ? b2->shape()[0] : b2->shape()[1]);
      const int64_t ldw2 = (N + 7) / 8 * 8;
      if (g->packed_b_.Stale(b2) || g->packed_b_.bytes < (size_t)n2 * ldw2 * es2) {
        g->packed_b_.Resize((size_t)n2 * ldw2 * es2);
        BZ_CHECK(bz_fc_pack_weight(b2->data(), BzType(b2->data_type()), g->transb_ ? 1 : 0, (int)N, n2, g->packed_b_.ptr,
                                   BzType(b2->data_type()), ldw2, st));
        g->packed_b_.Mark(b2);
      }
      memset(&nx, 0, sizeof(nx));
      nx.w = g->packed_b_.ptr;
      nx.ldw = ldw2;
      nx.n = n2;
      nx.alpha = g->alpha_;
      nx.beta = g->beta_;
      if (g->InputSize() > 2) nx.bias = AsFloatParam(g->Input(2), &g->bias_f32_, true, st);
      if (g->fused_) {
        nx.act = g->fused_act_;
        nx.dice_nosqrt = g->fused_nosqrt_ ? 1 : 0;
        nx.act_alpha = g->fused_alpha_;
        if (g->fused_act_ == BZ_ACT_PRELU) {
          nx.act_p0 = AsFloatParam(g->fused_->Input(1), &g->p_f32_[0], true, st);
          nx.act_size = (int)g->fused_->Input(1)->size();
        } else if (g->fused_act_ == BZ_ACT_DICE) {
          nx.act_p0 = AsFloatParam(g->fused_->Input(1), &g->p_f32_[0], true, st);
          nx.act_p1 = AsFloatParam(g->fused_->Input(2), &g->p_f32_[1], true, st);
          nx.act_p2 = AsFloatParam(g->fused_->Input(3), &g->p_f32_[2], true, st);
          nx.act_size = n2;
        }
      }
      Blob* y2 = g->fused_ ? g->fused_->Output(0) : g->Output(0);
      if (y2->data_type() != a->data_type()) return false;
      const std::vector<TIndex> shape2 = a_shape.size() == 3 ? std::vector<TIndex>{a_shape[0], M, (TIndex)n2} : std::vector<TIndex>{M, (TIndex)n2};
      if (g->head_ != nullptr) {
        GemmOp* h = g->head_;
        Blob* hb = h->Input(1);
        const int n3 = (int)(h->transb_ ? hb->shape()[0] : hb->shape()[1]);
        const int es3 = (int)DataTypeSize(hb->data_type());
        if (hb->data_type() != a->data_type()) return false;
        const int64_t ldw3 = (n2 + 7) / 8 * 8;
        if (h->packed_b_.Stale(hb) || h->packed_b_.bytes < (size_t)n3 * ldw3 * es3) {
          h->packed_b_.Resize((size_t)n3 * ldw3 * es3);
          BZ_CHECK(bz_fc_pack_weight(hb->data(), BzType(hb->data_type()), h->transb_ ? 1 : 0, n2, n3, h->packed_b_.ptr,
                                     BzType(hb->data_type()), ldw3, st));
          h->packed_b_.Mark(hb);
        }
        y2->SetShapeOnly(shape2);
        Blob* hy3 = h->fused_ ? h->fused_->Output(0) : h->Output(0);
        std::vector<TIndex> shape3 = shape2;
        shape3.back() = n3;
        hy3->Reshape(shape3);
        call.head_w = h->packed_b_.ptr;
        call.head_ldw = ldw3;
        if (h->InputSize() > 2) call.head_bias = AsFloatParam(h->Input(2), &h->bias_f32_, true, st);
        call.head_y = hy3->data();
        call.head_y_dtype = hy3->data_type();
        call.head_n = n3;
        call.head_act = h->fused_ ? h->fused_act_ : BZ_ACT_NONE;
      } else {
        y2->Reshape(shape2);
        nx.y = y2->data();
        nx.ldy = n2;
      }
      call.next = &nx;
    }
    call.a = pieces ? nullptr : a->data();
    call.a_pieces = pieces;
    call.a_rows = transa_ ? (int)K : (int)rows;
    call.a_cols = transa_ ? (int)rows : (int)K;
    call.trans_a = transa_;
    call.b_blob = b;
    call.b = b->data();
    call.b_rows = (int)b_shape[0];
    call.b_cols = (int)b_shape[1];
    call.trans_b = transb_;
    call.b_constant = b_constant_;
    call.dtype = a->data_type();
    call.y = (with_head || chain) ? nullptr : y->data();
    call.y_dtype = y->data_type();
    call.alpha = alpha_;
    call.beta = beta_;
    if (with_head) {
      Blob* hb = head_->Input(1);
      const int n2 = (int)(head_->transb_ ? hb->shape()[0] : hb->shape()[1]);
      const int es = (int)DataTypeSize(hb->data_type());
      const int64_t ldw = (N + 7) / 8 * 8;
      if (head_->packed_b_.Stale(hb) || head_->packed_b_.bytes < (size_t)n2 * ldw * es) {
        head_->packed_b_.Resize((size_t)n2 * ldw * es);
        BZ_CHECK(bz_fc_pack_weight(hb->data(), BzType(hb->data_type()), head_->transb_ ? 1 : 0, (int)N, n2, head_->packed_b_.ptr,
                                   BzType(hb->data_type()), ldw, st));
        head_->packed_b_.Mark(hb);
      }
      call.head_w = head_->packed_b_.ptr;
      call.head_ldw = ldw;
      if (head_->InputSize() > 2) call.head_bias = AsFloatParam(head_->Input(2), &head_->bias_f32_, true, st);
      call.head_y = hy->data();
      call.head_y_dtype = hy->data_type();
      call.head_n = n2;
      call.head_act = head_->fused_ ? head_->fused_act_ : BZ_ACT_NONE;
    }
    if (c != nullptr) {
      call.bias = AsFloatParam(c, &bias_f32_, c_constant_, st);
      if (c->shape().size() == 2 && c->shape()[0] != 1) {
        // a full [M,N] bias; under a 3-D A it repeats for every batch slice (DimEqualBroadcastAssign)
        BLAZE_CONDITION_THROW(a_shape.size() != 3 || a_shape[0] == 1, "3-D Gemm with an [M,N] bias is not supported on this device");
        call.bias_rows = (int)rows;
      } else {
        call.bias_rows = 1;
      }
    }
    if (fused_) {
      call.act = fused_act_;
      call.dice_nosqrt = fused_nosqrt_;
      call.act_alpha = fused_alpha_;
      if (fused_act_ == BZ_ACT_PRELU) {
        call.p0 = AsFloatParam(fused_->Input(1), &p_f32_[0], true, st);
        call.act_size = (int)fused_->Input(1)->size();
      } else if (fused_act_ == BZ_ACT_DICE) {
        for (int i = 0; i < 3; ++i) {
          const float* p = AsFloatParam(fused_->Input(1 + i), &p_f32_[i], true, st);
          (i == 0 ? call.p0 : (i == 1 ? call.p1 : call.p2)) = p;
        }
        call.act_size = (int)N;
      }
    }
    return RunFc(call, &packed_b_, &packed_a_, st);
  }

  void CheckValid() {
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->InputSize() > 2 ? this->Input(2) : nullptr;
    BLAZE_CONDITION_THROW(a->shape().size() == 2 || a->shape().size() == 3, "a->shape.size()=", a->shape().size());
    BLAZE_CONDITION_THROW(b->shape().size() == 2, "b->shape.size()=", b->shape().size(), " ", this->def_.DebugString());
    if (c != nullptr) BLAZE_CONDITION_THROW(c->shape().size() <= 2, "c->shape().size()=", c->shape().size());
    BLAZE_CONDITION_THROW(a->data_type() == b->data_type(), "a->data_type()=", a->data_type(), " b->data_type()=", b->data_type());
    const auto& a_shape = a->shape();
    const auto& b_shape = b->shape();
    TIndex a_m = a_shape.size() == 3 ? a_shape[1] : a_shape[0];
    TIndex a_k = a_shape.size() == 3 ? a_shape[2] : a_shape[1];
    if (transa_) std::swap(a_m, a_k);
    TIndex b_k = b_shape[0], b_n = b_shape[1];
    if (transb_) std::swap(b_k, b_n);
    BLAZE_CONDITION_THROW(a_k == b_k, "a_k=", a_k, " b_k=", b_k, " ", this->def_.DebugString());
    if (c != nullptr) {
      if (c->shape().size() == 2) {
        BLAZE_CONDITION_THROW(a_m == c->shape()[0], "a_m=", a_m, " c->shape()[0]=", c->shape()[0]);
        BLAZE_CONDITION_THROW(b_n == c->shape()[1], "b_n=", b_n, " c->shape()[1]=", c->shape()[1]);
      } else {
        BLAZE_CONDITION_THROW(b_n == c->shape()[0], "b_n=", b_n, " c->shape()[0]=", c->shape()[0]);
      }
    }
  }

  float alpha_, beta_;
  bool transa_, transb_;
  bool b_constant_ = false, c_constant_ = false;
  Derived packed_b_, packed_a_, bias_f32_, p_f32_[3];
  GemmOp* head_ = nullptr;       // the layer of at most 8 outputs computed in this operator's launch
  OperatorBase* concat_ = nullptr;  // the Concat that makes Input(0), computed by this operator's kernel
  GemmOp* next_ = nullptr;          // the narrow layer after this one, computed in this operator's launch
  std::vector<GemmOp*> siblings_;  // layers on the same input computed in this operator's launch
  Derived sib_w_, sib_f32_, sib_y_;  // stacked weights / fp32 parameters / outputs
  const Blob* sib_src_ = nullptr;    // this layer's weight as it was stacked
  uint64_t sib_version_ = 0;
  int launches_ = 1;
  OperatorBase* fused_ = nullptr;
  int fused_act_ = BZ_ACT_NONE;
  bool fused_nosqrt_ = false;
  float fused_alpha_ = 0.f;
};

REGISTER_HIP_OPERATOR(Gemm, GemmOp<HIPContext>);

// Input: A, B, [C]  Output: Y
OPERATOR_SCHEMA(Gemm)
    .NumInputs(2, 3)
    .NumOutputs(1)
    .IdenticalTypeOfInput(0)
    .SetDoc("General Matrix multiplication: Y = alpha * op(A) * op(B) + beta * C, with a 2-D or 3-D A");

// ------------------------------------------------------------------------------------------ batched helpers
namespace {

void StridedBatched(bool ta, bool tb, int M, int N, int K, float alpha, const void* A, int64_t sa, const void* B, int64_t sb,
                    float beta, void* C, int64_t sc, int batch, int data_type, hipStream_t st) {
  bz_bgemm_desc d;
  memset(&d, 0, sizeof(d));
  d.a = A;
  d.b = B;
  d.c = C;
  d.stride_a = sa;
  d.stride_b = sb;
  d.stride_c = sc;
  d.trans_a = ta;
  d.trans_b = tb;
  d.m = M;
  d.n = N;
  d.k = K;
  d.batch = batch;
  d.dtype = BzType(data_type);
  d.alpha = alpha;
  d.beta = beta;
  BZ_CHECK(bz_gemm_strided_batched(&d, st));
}

TIndex Prod(const std::vector<TIndex>& v) {
  TIndex p = 1;
  for (auto d : v) p *= d;
  return p;
}

// ULF batchdot compatibility: 2-D B [b,k] -> [b,1,k], 2-D A [b,k] -> [b,k,1] (matmul_op.h:147-165)
void UlfCompatibleReshape(Blob* a, Blob* b) {
  if (b->shape().size() == 2) b->Reshape({b->shape()[0], 1, b->shape()[1]});
  if (a->shape().size() == 2) a->Reshape({a->shape()[0], a->shape()[1], 1});
}

}  // namespace

// ------------------------------------------------------------------------------------------ MatMul
template <class Context>
class MatMulOp : public Operator<Context>, public WeightedPoolHost {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  bool WeightedPoolEligible() const override { return transa_ && !transb_ && !from_deepnet_; }
  void AdoptWeightedPool(OperatorBase* mul, OperatorBase* reduce_sum) override {
    pool_mul_ = mul;
    pool_sum_ = reduce_sum;
  }
  OperatorBase* AdoptedReduceSum() const override { return pool_sum_; }
  void AdoptTailConcat(OperatorBase* concat, OperatorBase* reshape, int att_pos, int sum_pos, int copy_pos) override {
    concat_ = concat;
    concat_reshape_ = reshape;
    att_pos_ = att_pos;
    sum_pos_ = sum_pos;
    copy_pos_ = copy_pos;
  }
  int LaunchesOfLastRun() const override { return launches_; }

  MatMulOp(const OperatorDef& def, Workspace* workspace) : Operator<Context>(def, workspace) {
    transa_ = OperatorBase::GetSingleArgument<bool>("transA", false);
    transb_ = OperatorBase::GetSingleArgument<bool>("transB", false);
    from_deepnet_ = OperatorBase::GetSingleArgument<bool>("from_deepnet", false);
  }

  bool RunOnDevice() override {
    launches_ = 1;
    if (pool_mul_ || pool_sum_ || concat_) {
      if (RunWeightedPool()) return true;
      // shapes the one-launch form does not take: the adopted operators run after all
      if (pool_mul_ && !pool_mul_->Run(context_.stream_id())) return false;
      if (pool_sum_ && !pool_sum_->Run(context_.stream_id())) return false;
      launches_ += (pool_mul_ != nullptr) + (pool_sum_ != nullptr);
    }
    if (!RunPlain()) return false;
    return RunTailConcat();
  }

 protected:
  // the Reshape and the Concat behind this MatMul, when its own launch has not written the Concat's output
  bool RunTailConcat() {
    if (!concat_) return true;
    ++launches_;
    return concat_reshape_->Run(context_.stream_id()) && concat_->Run(context_.stream_id());
  }
  bool RunPlain() {
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->Output(0);
    Setup();
    std::vector<TIndex> a_outer(a->shape().begin(), a->shape().end() - 2);
    std::vector<TIndex> b_outer(b->shape().begin(), b->shape().end() - 2);
    int M = (int)a->shape()[a->shape().size() - 2], K = (int)a->shape()[a->shape().size() - 1];
    if (transa_) std::swap(M, K);
    const int N = (int)(transb_ ? b->shape()[b->shape().size() - 2] : b->shape()[b->shape().size() - 1]);
    // BroadcastGemm is instantiated for outer rank <= 1 only (math/broadcast.h:236-246)
    BLAZE_CONDITION_THROW(a_outer.size() <= 1 && b_outer.size() <= 1, "Not Implemented BroadcastGemm!");
    const TIndex a_size = Prod(a_outer), b_size = Prod(b_outer);
    if (a_size != 1 && b_size != 1) BLAZE_CONDITION_THROW(a_size == b_size, "a_size=", a_size, " b_size=", b_size);
    // BroadcastGemm_NxN (math/broadcast.h:157-222): a side with one matrix is shared by the whole batch
    StridedBatched(transa_, transb_, M, N, K, 1.0f, a->data(), a_size == 1 ? 0 : (int64_t)M * K, b->data(),
                   b_size == 1 ? 0 : (int64_t)K * N, 0.f, c->data(), (int64_t)M * N, (int)std::max(a_size, b_size),
                   a->data_type(), context_.hip_stream());
    return true;
  }
  void Setup() {
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->Output(0);
    if (from_deepnet_) UlfCompatibleReshape(a, b);
    BLAZE_CONDITION_THROW(a->shape().size() >= 2, "a->shape().size()=", a->shape().size());
    BLAZE_CONDITION_THROW(b->shape().size() >= 2, "b->shape().size()=", b->shape().size());
    BLAZE_CONDITION_THROW(a->data_type() == b->data_type(), "a->data_type()=", a->data_type(), " b->data_type()=", b->data_type());
    Blob *min = a, *max = b;
    if (a->shape().size() > b->shape().size()) std::swap(min, max);
    std::vector<TIndex> shape = max->shape();
    const size_t off = max->shape().size() - min->shape().size();
    for (size_t k = 0; k + 2 < min->shape().size(); ++k) {
      const TIndex dim_min = min->shape()[k], dim_max = max->shape()[off + k];
      BLAZE_CONDITION_THROW(dim_min == dim_max || dim_min == 1 || dim_max == 1, "dim_min=", dim_min, " dim_max=", dim_max,
                            " op=", this->def_.name());
      if (dim_max == 1) shape[off + k] = dim_min;
    }
    const size_t ar = a->shape().size(), br = b->shape().size();
    const TIndex a_k = transa_ ? a->shape()[ar - 2] : a->shape()[ar - 1];
    const TIndex b_k = transb_ ? b->shape()[br - 1] : b->shape()[br - 2];
    BLAZE_CONDITION_THROW(a_k == b_k, "a_k=", a_k, " b_k=", b_k);
    shape[shape.size() - 2] = transa_ ? a->shape()[ar - 1] : a->shape()[ar - 2];
    shape[shape.size() - 1] = transb_ ? b->shape()[br - 2] : b->shape()[br - 1];
    c->Reshape(shape);
  }
  // [B, T, 1]^T x [B, T, C] with the weight = product of two [B, T, 1] tensors, and the sum of the history over T:
  // one launch.  False (nothing launched, no blob touched) when the tensors are not of that form.
  bool RunWeightedPool() {
    Blob* x = this->Input(1);
    Blob* w = pool_mul_ ? pool_mul_->Input(0) : this->Input(0);
    Blob* mask = pool_mul_ ? pool_mul_->Input(1) : nullptr;
    const std::vector<TIndex>& xs = x->shape();
    if (xs.size() != 3 || x->pitch() != 0 || w->pitch() != 0) return false;
    const std::vector<TIndex> col = {xs[0], xs[1], 1};
    if (w->shape() != col || w->data_type() != x->data_type()) return false;
    if (mask && (mask->shape() != col || mask->data_type() != x->data_type() || mask->pitch() != 0)) return false;
    if (x->data_type() != kFloat && x->data_type() != kFloat16) return false;
    if (xs[1] <= 0 || xs[2] <= 0 || xs[1] >= (1ll << 31) || xs[2] >= (1ll << 31)) return false;
    Blob* c = this->Output(0);
    c->set_data_type((DataType)x->data_type());
    Blob* s = pool_sum_ ? pool_sum_->Output(0) : nullptr;
    if (s) s->set_data_type((DataType)x->data_type());
    bz_weighted_pool_desc d;
    memset(&d, 0, sizeof(d));
    // the Concat behind it, when its other input (if any) has the rows of this batch: everything lands in its output
    Blob* other = concat_ && copy_pos_ >= 0 ? concat_->Input(copy_pos_) : nullptr;
    const bool tail = concat_ && (!other || (other->shape().size() == 2 && other->shape()[0] == xs[0] && other->shape()[1] > 0 &&
                                             other->shape()[1] < (1ll << 31) && other->data_type() == x->data_type()));
    if (tail) {
      Blob* out = concat_->Output(0);
      const int n_in = concat_->InputSize();
      TIndex total = 0, col_att = 0, col_sum = 0, col_copy = 0;
      for (int i = 0; i < n_in; ++i) {
        if (i == att_pos_) col_att = total;
        if (i == sum_pos_) col_sum = total;
        if (i == copy_pos_) col_copy = total;
        total += i == copy_pos_ ? other->shape()[1] : xs[2];
      }
      out->set_data_type((DataType)x->data_type());
      out->Reshape({xs[0], total});
      // (the results nobody reads any more keep their shapes and hold no data)
      c->SetShapeOnly({xs[0], 1, xs[2]});
      concat_reshape_->Output(0)->set_data_type((DataType)x->data_type());
      concat_reshape_->Output(0)->SetShapeOnly({xs[0], xs[2]});
      const size_t es = DataTypeSize(x->data_type());
      d.att = (char*)out->data() + col_att * es;
      d.ld_att = total;
      if (s && sum_pos_ >= 0) {
        s->SetShapeOnly({xs[0], xs[2]});
        d.sum = (char*)out->data() + col_sum * es;
        d.ld_sum = total;
      } else if (s) {
        s->Reshape({xs[0], xs[2]});
        d.sum = s->data();
      }
      if (other) {
        d.copy_src = other->data();
        d.ld_copy_src = other->pitch() ? other->pitch() : other->shape()[1];
        d.copy_dst = (char*)out->data() + col_copy * es;
        d.ld_copy_dst = total;
        d.copy_c = (int32_t)other->shape()[1];
      }
    } else {
      c->Reshape({xs[0], 1, xs[2]});
      d.att = c->data();
      if (s) {
        s->Reshape({xs[0], xs[2]});
        d.sum = s->data();
      }
    }
    d.w = w->data();
    d.mask = mask ? mask->data() : nullptr;
    d.x = x->data();
    d.batch = (int64_t)xs[0];
    d.t = (int32_t)xs[1];
    d.c = (int32_t)xs[2];
    d.dtype = BzType(x->data_type());
    BZ_CHECK(bz_weighted_pool(&d, context_.hip_stream()));
    return tail ? true : RunTailConcat();
  }
  bool transa_, transb_, from_deepnet_;
  OperatorBase* pool_mul_ = nullptr;
  OperatorBase* pool_sum_ = nullptr;
  OperatorBase* concat_ = nullptr;          // the Concat behind the weighted pool (AdoptTailConcat) and the Reshape before it
  OperatorBase* concat_reshape_ = nullptr;
  int att_pos_ = -1, sum_pos_ = -1, copy_pos_ = -1;
  int launches_ = 1;
};

REGISTER_HIP_OPERATOR(MatMul, MatMulOp<HIPContext>);

OPERATOR_SCHEMA(MatMul).NumInputs(2).NumOutputs(1).IdenticalTypeOfInput(0).SetDoc("Matrix product that behaves like numpy.matmul");

// ------------------------------------------------------------------------------------------ FusedParallelGemm
template <class Context>
class FusedParallelGemmOp : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  FusedParallelGemmOp(const OperatorDef& def, Workspace* workspace) : Operator<Context>(def, workspace) {
    parallel_num_ = OperatorBase::GetSingleArgument<int>("parallel_num", 2);
    transa_ = OperatorBase::GetSingleArgument<bool>("transA", false);
    transb_ = OperatorBase::GetSingleArgument<bool>("transB", false);
    alpha_ = OperatorBase::GetSingleArgument<float>("alpha", 1.0);
    beta_ = OperatorBase::GetSingleArgument<float>("beta", 1.0);
    BLAZE_CONDITION_THROW(parallel_num_ > 0, "parallel_num=", parallel_num_);
    b_constant_ = workspace->HasConstantBlob(def.input(1));
    if (def.input_size() > 2) c_constant_ = workspace->HasConstantBlob(def.input(2));
    packed_b_.resize(parallel_num_);
  }

  bool RunOnDevice() override {
    CheckValid();
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->InputSize() > 2 ? this->Input(2) : nullptr;
    Blob* y = this->Output(0);
    const auto& a_shape = a->shape();
    const auto& b_shape = b->shape();
    const int P = parallel_num_;
    TIndex M = a_shape.size() == 3 ? a_shape[1] : a_shape[0];
    TIndex K = a_shape.size() == 3 ? a_shape[2] : a_shape[1];
    if (transa_) std::swap(M, K);
    const TIndex N = transb_ ? b_shape[0] / P : b_shape[1];
    TIndex rows = M;
    if (a_shape.size() == 3) {
      y->Reshape({a_shape[0] * P, M, N});
      BLAZE_CONDITION_THROW(!transa_ || a_shape[0] == 1, "3-D FusedParallelGemm with transA is not supported on this device");
      rows = a_shape[0] * M;
    } else {
      y->Reshape({M * P, N});
    }
    hipStream_t st = context_.hip_stream();
    const float* bias = c ? AsFloatParam(c, &bias_f32_, c_constant_, st) : nullptr;
    const bool full_bias = c && c->shape().size() == 2 && c->shape()[0] != (TIndex)P;
    if (full_bias)
      BLAZE_CONDITION_THROW(a_shape.size() != 3 || a_shape[0] == 1, "3-D FusedParallelGemm with a [P*M,N] bias is not supported on this device");
    const size_t es = DataTypeSize(a->data_type());
    // The P sibling FCs share the input; slice p owns weights [K,N] (or [N,K]), bias and output slice p.  The reference
    // hands them to one GemmStridedBatched with stride_a = 0 (fused_parallel_gemm_op.h:115-129); here they are one
    // launch of the FC kernel over P*N columns whose epilogue scatters each slice to its own [rows, N] matrix.  (A
    // launch of at most 8 columns would take the skinny kernel, which computes a softmax-sized head: those few cases
    // run slice by slice.)
    const bool one_launch = P > 1 && (TIndex)P * N > 8;
    launches_ = one_launch ? 1 : P;
    for (int p = 0; p < launches_; ++p) {
      FcCall call;
      call.a = a->data();
      call.a_rows = transa_ ? (int)K : (int)rows;
      call.a_cols = transa_ ? (int)rows : (int)K;
      call.trans_a = transa_;
      call.b_blob = b;
      call.b = (const char*)b->data() + (size_t)p * K * N * es;
      call.b_rows = transb_ ? (int)N : (int)K;
      call.b_cols = transb_ ? (int)K : (int)N;
      call.trans_b = transb_;
      call.b_constant = b_constant_;
      call.dtype = a->data_type();
      call.y = (char*)y->data() + (size_t)p * rows * N * DataTypeSize(y->data_type());
      call.y_dtype = y->data_type();
      call.alpha = alpha_;
      call.beta = beta_;
      if (bias) {
        call.bias = bias + (full_bias ? (size_t)p * rows * N : (size_t)p * N);
        call.bias_rows = full_bias ? (int)rows : 1;
      }
      if (one_launch) {
        call.slices = P;
        call.y_split_stride = (int64_t)rows * N;
        call.b_rows = (int)(transb_ ? N : K) * P;
      }
      RunFc(call, &packed_b_[p], &packed_a_, st);
    }
    return true;
  }

 protected:
  void CheckValid() {
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->InputSize() > 2 ? this->Input(2) : nullptr;
    BLAZE_CONDITION_THROW(a->shape().size() == 2 || a->shape().size() == 3, "a->shape().size()=", a->shape().size());
    BLAZE_CONDITION_THROW(b->shape().size() == 2, "b->shape().size()=", b->shape().size());
    if (c != nullptr) BLAZE_CONDITION_THROW(c->shape().size() <= 2, "c->shape().size()=", c->shape().size());
    const auto& a_shape = a->shape();
    const auto& b_shape = b->shape();
    TIndex a_m = a_shape.size() == 3 ? a_shape[1] : a_shape[0];
    TIndex a_k = a_shape.size() == 3 ? a_shape[2] : a_shape[1];
    if (transa_) std::swap(a_m, a_k);
    // the P weights are stacked on dim 0: [P*K, N], or [P*N, K] under transB
    TIndex b_k = transb_ ? b_shape[1] : b_shape[0] / parallel_num_;
    TIndex b_n = transb_ ? b_shape[0] / parallel_num_ : b_shape[1];
    BLAZE_CONDITION_THROW(a_k == b_k, "a_k=", a_k, " b_k=", b_k);
    if (c != nullptr) {
      if (c->shape().size() == 2) {
        BLAZE_CONDITION_THROW(a_m == c->shape()[0] / parallel_num_, "a_m=", a_m, " c->shape()[0]=", c->shape()[0],
                              " parallel_num_=", parallel_num_);
        BLAZE_CONDITION_THROW(b_n == c->shape()[1], "b_n=", b_n, " c->shape()[1]=", c->shape()[1]);
      } else {
        BLAZE_CONDITION_THROW(b_n == c->shape()[0] / parallel_num_, "b_n=", b_n, " c->shape()[0]=", c->shape()[0]);
      }
    }
  }
  int parallel_num_;
  bool transa_, transb_;
  float alpha_, beta_;
  bool b_constant_ = false, c_constant_ = false;
  std::vector<Derived> packed_b_;
  Derived packed_a_, bias_f32_;
  int launches_ = 0;  // kernel launches of the last run (1 when the slices went out as one)

 public:
  int LaunchesOfLastRun() const override { return launches_; }
};

REGISTER_HIP_OPERATOR(FusedParallelGemm, FusedParallelGemmOp<HIPContext>);

OPERATOR_SCHEMA(FusedParallelGemm)
    .NumInputs(2, 3)
    .NumOutputs(1)
    .IdenticalTypeOfInput(0)
    .SetDoc("parallel_num sibling Gemms that share one input, weights stacked on dim 0");

// ------------------------------------------------------------------------------------------ FusedParallelMatMul
template <class Context>
class FusedParallelMatMulOp : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  FusedParallelMatMulOp(const OperatorDef& def, Workspace* workspace) : Operator<Context>(def, workspace) {
    parallel_num_ = OperatorBase::GetSingleArgument<int>("parallel_num", 2);
    from_deepnet_ = OperatorBase::GetSingleArgument<bool>("from_deepnet", false);
    transa_ = OperatorBase::GetSingleArgument<bool>("transA", false);
    transb_ = OperatorBase::GetSingleArgument<bool>("transB", false);
    BLAZE_CONDITION_THROW(parallel_num_ > 0, "parallel_num=", parallel_num_);
  }

  bool RunOnDevice() override {
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->Output(0);
    if (from_deepnet_) UlfCompatibleReshape(a, b);
    BLAZE_CONDITION_THROW(a->shape().size() >= 2, "a->shape().size()=", a->shape().size());
    BLAZE_CONDITION_THROW(b->shape().size() >= 2, "b->shape().size()=", b->shape().size());
    std::vector<TIndex> a_shape = a->shape(), b_shape = b->shape();
    const int P = parallel_num_;
    BLAZE_CONDITION_THROW(a_shape[0] % P == 0, "a_shape[0]=", a_shape[0], " parallel_num=", P);
    BLAZE_CONDITION_THROW(b_shape[0] % P == 0, "b_shape[0]=", b_shape[0], " parallel_num=", P);
    a_shape[0] /= P;
    b_shape[0] /= P;
    int M = (int)a_shape[a_shape.size() - 2], K = (int)a_shape[a_shape.size() - 1];
    if (transa_) std::swap(M, K);
    const int N = (int)(transb_ ? b_shape[b_shape.size() - 2] : b_shape[b_shape.size() - 1]);
    const TIndex b_k = transb_ ? b_shape[b_shape.size() - 1] : b_shape[b_shape.size() - 2];
    BLAZE_CONDITION_THROW((TIndex)K == b_k, "a_k=", K, " b_k=", b_k);
    a_shape.resize(a_shape.size() - 2);
    b_shape.resize(b_shape.size() - 2);
    BLAZE_CONDITION_THROW(a_shape.size() <= 1 && b_shape.size() <= 1, "Not Implemented BatchedBroadcastGemm!");
    const TIndex a_size = Prod(a_shape), b_size = Prod(b_shape);
    if (a_size != 1 && b_size != 1) BLAZE_CONDITION_THROW(a_size == b_size, "a_size=", a_size, " b_size=", b_size);
    BLAZE_CONDITION_THROW(a_size == b_size || a_size == 1 || b_size == 1, "a_size=", a_size, " b_size=", b_size);
    const TIndex cb = std::max(a_size, b_size);
    c->Reshape({(TIndex)P * cb, (TIndex)M, (TIndex)N});
    const size_t es = DataTypeSize(a->data_type());
    hipStream_t st = context_.hip_stream();
    if (a_size == b_size) {
      // one batch over every slice of every parallel group (math/broadcast.h:282-317)
      StridedBatched(transa_, transb_, M, N, K, 1.f, a->data(), (int64_t)M * K, b->data(), (int64_t)K * N, 0.f, c->data(),
                     (int64_t)M * N, (int)(a_size * P), a->data_type(), st);
    } else {
      // per parallel group, the single matrix of one side is shared by the group's batch (:340-378; the
      // N == 1 shortcut of :319-338 is the same products computed through a transposed Gemm)
      for (int p = 0; p < P; ++p)
        StridedBatched(transa_, transb_, M, N, K, 1.f, (const char*)a->data() + (size_t)p * a_size * M * K * es,
                       a_size == 1 ? 0 : (int64_t)M * K, (const char*)b->data() + (size_t)p * b_size * K * N * es,
                       b_size == 1 ? 0 : (int64_t)K * N, 0.f, (char*)c->data() + (size_t)p * cb * M * N * es, (int64_t)M * N,
                       (int)cb, a->data_type(), st);
    }
    return true;
  }

 protected:
  bool transa_, transb_, from_deepnet_;
  int parallel_num_;
};

REGISTER_HIP_OPERATOR(FusedParallelMatMul, FusedParallelMatMulOp<HIPContext>);

OPERATOR_SCHEMA(FusedParallelMatMul)
    .NumInputs(2)
    .NumOutputs(1)
    .IdenticalTypeOfInput(0)
    .SetDoc("parallel_num sibling MatMuls stacked on dim 0");

}  // namespace blaze
