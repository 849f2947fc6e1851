// misc_ops.cc -- the operators around the Gemms in CTR / DIN graphs: PRelu, Dice, LeakyRelu, Sigmoid, Softmax
// (used stand-alone when they cannot ride in a Gemm epilogue), ConstantFill (weights) and Concat.
//
// Formulas and argument names follow the reference's operators:
//   PRelu        blaze/operator/op/prelu_op.cc:11-73     slope broadcast over the trailing dims
//   Dice         blaze/operator/op/dice_op.{h,cc}        inputs X, gamma, mean, var; arg nosqrt
//   LeakyRelu    blaze/operator/op/leaky_relu_op.cc      arg alpha
//   Sigmoid      blaze/operator/op/sigmoid_op.cc:15-38
//   Softmax      blaze/operator/op/softmax_op.cc:13-78   arg axis (default 1)
//   ConstantFill blaze/operator/op/constant_fill_op.h:13-57  args shape, dtype, value
//   Concat       blaze/operator/op/concat_op.h           arg axis (default 1)
#include "blaze/graph.h"
#include "blaze/op_util.h"
#include "blaze/operator.h"
#include "blaze_hip.h"

#include <algorithm>
#include <type_traits>

namespace blaze {

namespace {

void RunActivation(Blob* x, Blob* y, int act, const float* p0, const float* p1, const float* p2, int act_size, bool nosqrt,
                   float alpha, int64_t rows, int64_t cols, hipStream_t st) {
  bz_act_desc d;
  memset(&d, 0, sizeof(d));
  d.x = x->data();
  d.y = y->data();
  d.p0 = p0;
  d.p1 = p1;
  d.p2 = p2;
  d.rows = rows;
  d.cols = cols;
  d.dtype = BzType(x->data_type());
  d.act = act;
  d.act_size = act_size;
  d.dice_nosqrt = nosqrt ? 1 : 0;
  d.act_alpha = alpha;
  BZ_CHECK(bz_activation(&d, st));
}

}  // namespace

template <class Context>
class PReluOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  PReluOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {}
  bool RunOnDevice() override {
    Blob* X = this->Input(0);
    Blob* W = this->Input(1);
    Blob* Y = this->Output(0);
    BLAZE_CONDITION_THROW(W->size() > 0 && X->size() % W->size() == 0, "X->size()=", X->size(), " W->size()=", W->size());
    Y->Reshape(X->shape());
    if (X->size() == 0) return true;
    hipStream_t st = context_.hip_stream();
    // the slope is the "inner" broadcast: element i uses w[i % W.size] (prelu_op.cc:13-29)
    RunActivation(X, Y, BZ_ACT_PRELU, w_.Get(W, st), nullptr, nullptr, (int)W->size(), false, 0.f, (int64_t)(X->size() / W->size()),
                  (int64_t)W->size(), st);
    return true;
  }

 private:
  ParamF32 w_;
};
REGISTER_HIP_OPERATOR(PRelu, PReluOp<HIPContext>);
OPERATOR_SCHEMA(PRelu).NumInputs(2).NumOutputs(1).AllowInplace({{0, 0}}).IdenticalTypeOfInput(0).SetDoc(
    "f(x) = slope * x for x < 0, f(x) = x for x >= 0");

template <class Context>
class DiceOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  DiceOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    nosqrt_ = OperatorBase::GetSingleArgument<bool>("nosqrt", false);
  }
  bool RunOnDevice() override {
    Blob* x = this->Input(0);
    Blob* gamma = this->Input(1);
    Blob* mean = this->Input(2);
    Blob* var = this->Input(3);
    Blob* y = this->Output(0);
    const int dt[4] = {x->data_type(), gamma->data_type(), mean->data_type(), var->data_type()};
    for (int k = 1; k < 4; ++k)
      BLAZE_CONDITION_THROW(dt[k] == dt[k - 1], "data_type[", k, "]=", dt[k], " data_type[", k - 1, "]=", dt[k - 1]);
    BLAZE_CONDITION_THROW(gamma->size() == mean->size() && mean->size() == var->size(), "size[gamma]=", gamma->size(),
                          " size[mean]=", mean->size(), " size[var]=", var->size());
    BLAZE_CONDITION_THROW(gamma->size() > 0 && x->size() % gamma->size() == 0, "x->size()=", x->size(), " gamma->size()=", gamma->size());
    y->Reshape(x->shape());
    if (x->size() == 0) return true;
    hipStream_t st = context_.hip_stream();
    RunActivation(x, y, BZ_ACT_DICE, p_[0].Get(gamma, st), p_[1].Get(mean, st), p_[2].Get(var, st), (int)gamma->size(), nosqrt_, 0.f,
                  (int64_t)(x->size() / gamma->size()), (int64_t)gamma->size(), st);
    return true;
  }

 private:
  bool nosqrt_ = false;
  ParamF32 p_[3];
};
REGISTER_HIP_OPERATOR(Dice, DiceOp<HIPContext>);
OPERATOR_SCHEMA(Dice).NumInputs(4).NumOutputs(1).AllowInplace({{0, 0}}).IdenticalTypeOfInput(0).SetDoc(
    "Dice activation (https://arxiv.org/pdf/1706.06978.pdf), inference form with fixed mean/var");

template <class Context>
class LeakyReluOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  LeakyReluOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    alpha_ = OperatorBase::GetSingleArgument<float>("alpha", 0.01f);
  }
  bool RunOnDevice() override {
    Blob* X = this->Input(0);
    Blob* Y = this->Output(0);
    Y->Reshape(X->shape());
    if (X->size() == 0) return true;
    RunActivation(X, Y, BZ_ACT_LEAKY_RELU, nullptr, nullptr, nullptr, 0, false, alpha_, 1, (int64_t)X->size(), context_.hip_stream());
    return true;
  }

 private:
  float alpha_;
};
REGISTER_HIP_OPERATOR(LeakyRelu, LeakyReluOp<HIPContext>);
OPERATOR_SCHEMA(LeakyRelu).NumInputs(1).NumOutputs(1).AllowInplace({{0, 0}}).IdenticalTypeOfInput(0).SetDoc(
    "f(x) = alpha * x for x < 0, f(x) = x for x >= 0");

template <class Context>
class SigmoidOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  SigmoidOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {}
  bool RunOnDevice() override {
    Blob* X = this->Input(0);
    Blob* Y = this->Output(0);
    Y->Reshape(X->shape());
    if (X->size() == 0) return true;
    RunActivation(X, Y, BZ_ACT_SIGMOID, nullptr, nullptr, nullptr, 0, false, 0.f, 1, (int64_t)X->size(), context_.hip_stream());
    return true;
  }
};
REGISTER_HIP_OPERATOR(Sigmoid, SigmoidOp<HIPContext>);
OPERATOR_SCHEMA(Sigmoid).NumInputs(1).NumOutputs(1).AllowInplace({{0, 0}}).IdenticalTypeOfInput(0).SetDoc("y = 1 / (1 + exp(-x))");

template <class Context>
class SoftmaxOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  SoftmaxOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    axis_ = OperatorBase::GetSingleArgument<size_t>("axis", 1);
  }
  bool RunOnDevice() override {
    Blob* X = this->Input(0);
    Blob* Y = this->Output(0);
    BLAZE_CONDITION_THROW(axis_ < X->shape().size(), "axis=", axis_, " X->shape().size()=", X->shape().size());
    // softmax over `axis` with W trailing elements (softmax_op.cc:23-26)
    const TIndex W = X->size((int)axis_ + 1, (int)X->shape().size());
    Y->Reshape(X->shape());
    if (X->size() == 0) return true;
    const int64_t C = (int64_t)X->shape()[axis_];
    BZ_CHECK(bz_softmax_axis(X->data(), Y->data(), (int64_t)(X->size() / (C * W)), C, (int64_t)W, BzType(X->data_type()),
                             context_.hip_stream()));
    return true;
  }

 private:
  size_t axis_;
};
REGISTER_HIP_OPERATOR(Softmax, SoftmaxOp<HIPContext>);
OPERATOR_SCHEMA(Softmax).NumInputs(1).NumOutputs(1).AllowInplace({{0, 0}}).IdenticalTypeOfInput(0).SetDoc("softmax over axis");

// ------------------------------------------------------------------------------------------ ConstantFill
template <class Context>
class ConstantFillOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  ConstantFillOp(const OperatorDef& def, Workspace* ws)
      : Operator<Context>(def, ws, false), shape_(OperatorBase::GetRepeatedArgument<TIndex>("shape")) {
    const DataType dtype = (DataType)OperatorBase::GetSingleArgument<int>("dtype", kFloat);
    for (const std::string& out : def.output()) this->outputs_.push_back(ws->CreateConstantBlob(out, this->device_option_));
    Blob* output = this->Output(0);
    output->set_data_type(dtype);
    output->Reshape(shape_);
    const size_t n = output->size();
    std::vector<unsigned char> host(n * DataTypeSize(dtype));
    switch (dtype) {  // CONSTANT_FILL_TYPE_SWITCH
      case kFloat: {
        const auto v = OperatorBase::GetRepeatedArgument<float>("value");
        CheckCount(v.size(), n);
        memcpy(host.data(), v.data(), host.size());
        break;
      }
      case kFloat16: {  // stored as floats in the model, narrowed per element with round-to-nearest-even
        const auto v = OperatorBase::GetRepeatedArgument<float>("value");
        CheckCount(v.size(), n);
        uint16_t* h = (uint16_t*)host.data();
        for (size_t i = 0; i < n; ++i) h[i] = FloatToHalf(v[i]);
        break;
      }
      case kInt32: {
        const auto v = OperatorBase::GetRepeatedArgument<int>("value");
        CheckCount(v.size(), n);
        memcpy(host.data(), v.data(), host.size());
        break;
      }
      case kInt64: {
        const auto v = OperatorBase::GetRepeatedArgument<int64_t>("value");
        CheckCount(v.size(), n);
        memcpy(host.data(), v.data(), host.size());
        break;
      }
      default:
        BLAZE_THROW("Unsupported type: ", dtype);
    }
    // one-time upload, synchronous: the blob is shared by every predictor created afterwards
    if constexpr (std::is_same<Context, HIPContext>::value) {
      context_.Activate();
      HIP_CHECK(hipMemcpy(output->data(), host.data(), host.size(), hipMemcpyHostToDevice));
    } else {
      memcpy(output->data(), host.data(), host.size());
    }
  }
  bool RunOnDevice() override { return true; }

 private:
  void CheckCount(size_t have, size_t want) {
    BLAZE_CONDITION_THROW(have == want, "value.size()=", have, " output->size()=", want, " ", this->def_.DebugString());
  }
  std::vector<TIndex> shape_;
};
REGISTER_HIP_OPERATOR(ConstantFill, ConstantFillOp<HIPContext>);
REGISTER_CPU_OPERATOR(ConstantFill, ConstantFillOp<CPUContext>);
OPERATOR_SCHEMA(ConstantFill).NumInputs(0).NumOutputs(1).SetDoc("a constant tensor: args shape, dtype, value");


// ------------------------------------------------------------------------------------------ Concat
template <class Context>
class ConcatOp final : public Operator<Context>, public ConcatPieceHost, public ConcatForFc {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  ConcatOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    axis_ = OperatorBase::GetSingleArgument<int>("axis", 1);
  }
  void AdoptProducer(int input_idx, OperatorBase* producer, int position) override {
    producers_.push_back({position, input_idx, producer});
    std::sort(producers_.begin(), producers_.end(), [](const Adopted& a, const Adopted& b) { return a.position < b.position; });
  }
  bool DescribeAsPieces(bz_concat_ew_desc* desc) override { return RunWithPieces(desc); }
  // (0 when every input already lives in the output)
  int LaunchesOfLastRun() const override { return launches_; }
  bool RunOnDevice() override {
    launches_ = 0;
    if (!producers_.empty()) {
      if (RunWithPieces(nullptr)) return true;
      // shapes the one-launch form does not take: run the adopted operators after all, in net order, then copy
      for (const Adopted& a : producers_)
        if (!a.op->Run(context_.stream_id())) return false;
    }
    Blob* x0 = this->Input(0);
    const size_t rank = x0->shape().size();
    BLAZE_CONDITION_THROW(axis_ >= 0 && (size_t)axis_ < rank, "axis=", axis_, " rank=", rank);
    std::vector<TIndex> shape = x0->shape();
    TIndex total = 0;
    for (int i = 0; i < this->InputSize(); ++i) {
      Blob* x = this->Input(i);
      BLAZE_CONDITION_THROW(x->shape().size() == rank && x->data_type() == x0->data_type(), "concat input ", i, " has another rank or type");
      for (size_t k = 0; k < rank; ++k)
        if ((int)k != axis_) BLAZE_CONDITION_THROW(x->shape()[k] == shape[k], "concat input ", i, " dim ", k, " mismatch");
      total += x->shape()[axis_];
    }
    shape[axis_] = total;
    Blob* y = this->Output(0);
    y->Reshape(shape);
    const size_t es = DataTypeSize(y->data_type());
    const TIndex outer = y->size(0, axis_), inner = y->size(axis_ + 1, (int)rank);
    hipStream_t st = context_.hip_stream();
    // pieces that already live in the output (column-slice views their producers wrote in place) are skipped;
    // the others are copied, one launch per group of BZ_CONCAT_MAX
    bz_concat_desc d;
    memset(&d, 0, sizeof(d));
    size_t col = 0;
    auto flush = [&]() {
      if (d.n == 0) return;
      d.dst_pitch = (int64_t)(total * inner * es);
      d.rows = (int64_t)outer;
      BZ_CHECK(bz_concat_cols(&d, st));
      ++launches_;
      memset(&d, 0, sizeof(d));
    };
    for (int i = 0; i < this->InputSize(); ++i) {
      Blob* x = this->Input(i);
      const size_t width = (size_t)(x->shape()[axis_] * inner * es);
      const bool in_place = rank == 2 && axis_ == 1 && x->IsColumnSliceOf(y, (TIndex)(col / es));
      if (in_place || d.n == BZ_CONCAT_MAX) flush();
      if (!in_place) {
        BLAZE_CONDITION_THROW(x->pitch() == 0, "concat input ", i, " is a strided view of another tensor");
        if (d.n == 0) d.dst = (char*)y->data() + col;  // this group starts `col` bytes into every output row
        d.src[d.n] = x->data();
        d.width[d.n] = (int64_t)width;
        d.src_pitch[d.n] = (int64_t)width;
        ++d.n;
      }
      col += width;
    }
    flush();
    return true;
  }

 private:
  struct Adopted {
    int position;
    int input_idx;
    OperatorBase* op;
  };
  int launches_ = 0;
  // The inputs as pieces of one bz_concat_ew launch.  False when the shapes do not fit that kernel's model (concat
  // along another axis than the last, an operand broadcast along the last axis, or row dims that do not merge into
  // two coordinates); nothing has been launched then.
  // describe != nullptr: only fill *describe (dst stays null) and give the output its shape, no memory, no launch
  bool RunWithPieces(bz_concat_ew_desc* describe) {
    const int n = this->InputSize();
    if (n > BZ_CEW_MAX) return false;
    std::vector<ConcatPiece> pieces(n);
    std::vector<bool> described(n, false);
    for (const Adopted& a : producers_) {  // net order: a BroadcastTo may take its shape from an earlier piece
      auto* src = dynamic_cast<ConcatPieceSource*>(a.op);
      if (!src || !src->DescribePiece(&pieces[a.input_idx])) return false;
      described[a.input_idx] = true;
    }
    for (int i = 0; i < n; ++i) {
      if (described[i]) continue;
      Blob* x = this->Input(i);
      if (x->pitch() != 0) return false;
      pieces[i].x = x;
      pieces[i].op = BZ_EW_ASSIGN;
      pieces[i].shape = x->shape();
    }
    const size_t rank = pieces[0].shape.size();
    if (rank < 1 || axis_ != (int)rank - 1) return false;
    const int dtype = pieces[0].x->data_type();
    std::vector<TIndex> shape = pieces[0].shape;
    TIndex total = 0;
    for (int i = 0; i < n; ++i) {
      const ConcatPiece& p = pieces[i];
      BLAZE_CONDITION_THROW(p.shape.size() == rank && p.x->data_type() == dtype && (!p.y || p.y->data_type() == dtype),
                            "concat input ", i, " has another rank or type");
      for (size_t k = 0; k + 1 < rank; ++k)
        BLAZE_CONDITION_THROW(p.shape[k] == shape[k], "concat input ", i, " dim ", k, " mismatch");
      if (p.shape[rank - 1] <= 0 || p.shape[rank - 1] >= (1ll << 31)) return false;
      total += p.shape[rank - 1];
    }
    // every operand's dims, right aligned to the piece's rank; `bc[k]` collects, per outer dim, which operands are
    // broadcast along it (one bit per operand): adjacent dims with the same set merge into one row coordinate
    struct Operand {
      std::vector<TIndex> dims;
    };
    std::vector<Operand> ops;
    for (int i = 0; i < n; ++i) {
      for (Blob* b : {pieces[i].x, pieces[i].y}) {
        Operand o;
        if (b) {
          if (b->shape().size() > rank) return false;
          o.dims.assign(rank - b->shape().size(), 1);
          o.dims.insert(o.dims.end(), b->shape().begin(), b->shape().end());
          if (o.dims[rank - 1] != pieces[i].shape[rank - 1]) return false;  // broadcast along the concat axis
        }
        ops.push_back(o);
      }
    }
    std::vector<uint32_t> group_sig;
    std::vector<TIndex> group_size;
    for (size_t k = 0; k + 1 < rank; ++k) {
      if (shape[k] == 1) continue;
      uint32_t sig = 0;
      for (size_t o = 0; o < ops.size(); ++o)
        if (!ops[o].dims.empty() && ops[o].dims[k] == 1) sig |= 1u << o;
      if (!group_sig.empty() && group_sig.back() == sig) {
        group_size.back() *= shape[k];
      } else {
        group_sig.push_back(sig);
        group_size.push_back(shape[k]);
      }
    }
    if (group_sig.size() > 2) return false;
    while (group_sig.size() < 2) {
      group_sig.push_back(0);
      group_size.push_back(1);
    }
    shape[rank - 1] = total;
    Blob* y = this->Output(0);
    y->set_data_type((DataType)dtype);
    if (describe)
      y->SetShapeOnly(shape);
    else
      y->Reshape(shape);
    bz_concat_ew_desc d;
    memset(&d, 0, sizeof(d));
    d.n = n;
    d.dtype = BzType(dtype);
    d.dst = describe ? nullptr : y->data();
    d.dst_pitch = total;
    d.r0 = group_size[0];
    d.r1 = group_size[1];
    for (int i = 0; i < n; ++i) {
      const int64_t w = pieces[i].shape[rank - 1];
      d.op[i] = pieces[i].op;
      d.width[i] = (int32_t)w;
      d.x[i] = pieces[i].x->data();
      d.y[i] = pieces[i].y ? pieces[i].y->data() : nullptr;
      for (int side = 0; side < 2; ++side) {
        if (side == 1 && !pieces[i].y) continue;
        const bool b0 = (group_sig[0] >> (2 * i + side)) & 1, b1 = (group_sig[1] >> (2 * i + side)) & 1;
        int64_t* st = side == 0 ? d.x_stride[i] : d.y_stride[i];
        st[0] = b0 ? 0 : (b1 ? 1 : d.r1) * w;
        st[1] = b1 ? 0 : w;
      }
    }
    if (describe) {
      *describe = d;
      return true;
    }
    BZ_CHECK(bz_concat_ew(&d, context_.hip_stream()));
    launches_ = 1;
    return true;
  }

  int axis_;
  std::vector<Adopted> producers_;  // inputs computed by this operator instead of by their own (sorted by net position)
};
REGISTER_HIP_OPERATOR(Concat, ConcatOp<HIPContext>);
OPERATOR_SCHEMA(Concat).NumInputs(1, INT_MAX).NumOutputs(1).IdenticalTypeOfInput(0).SetDoc("concatenate along axis");

}  // namespace blaze
