// shape_ops.cc -- the shape / elementwise operators that surround the Gemms of a DIN-style graph.
//
// Names, inputs, arguments and shape rules follow the reference's operators:
//   Reshape             blaze/operator/op/reshape_op.h:22-52        input 1 = int32 shape (0 keeps, one -1 inferred); aliases X
//   Add Sub Mul Div     blaze/operator/op/elementwise_op.{h,cc}     multidirectional broadcasting (math/broadcast.h:39-67)
//   BroadcastTo         blaze/operator/op/elementwise_op.h:193-226  to the shape of input 1, or of arg `shape`
//   Where               blaze/operator/op/elementwise_op.h:228-283  condition int32|int64, X, Y
//   ReduceSum           blaze/operator/op/reduce_sum_op.h:17-58     args axis | axes (one entry), keepdims (default 1)
//   Fuse                blaze/operator/op/fuse_op.{h,cc}            arg comm_index: that input's single row is repeated
//   BatchNormalization  blaze/operator/op/batch_normalization_op.{h,cc}  inputs X, gamma, beta, mean, var; args eps, nosqrt
#include "blaze/graph.h"
#include "blaze/op_util.h"
#include "blaze/operator.h"
#include "blaze_hip.h"

#include <algorithm>
#include <climits>

namespace blaze {

namespace {

// MBroadcasting::BroadcastShape
std::vector<TIndex> BroadcastShape(const std::vector<TIndex>& a, const std::vector<TIndex>& b, const OperatorDef& def) {
  const size_t n = std::max(a.size(), b.size());
  std::vector<TIndex> out(n);
  for (size_t i = 0; i < n; ++i) {
    const TIndex ad = i >= n - a.size() ? a[i - (n - a.size())] : 1;
    const TIndex bd = i >= n - b.size() ? b[i - (n - b.size())] : 1;
    BLAZE_CONDITION_THROW(ad == bd || ad == 1 || bd == 1, "a->shape()[", i, "]=", ad, "; b->shape()[", i, "]=", bd,
                          " not equal or meet broadcast rule op=", def.name());
    out[i] = std::max(ad, bd);
  }
  return out;
}

// element strides of a contiguous operand of shape `s` seen through the output's dims (0 where it is broadcast)
void OperandStrides(const std::vector<TIndex>& s, const std::vector<TIndex>& out, int64_t* strides) {
  const size_t n = out.size(), off = n - s.size();
  int64_t st = 1;
  for (size_t k = n; k-- > 0;) {
    if (k < off) {
      strides[k] = 0;
      continue;
    }
    const TIndex d = s[k - off];
    strides[k] = d == 1 ? 0 : st;
    st *= (int64_t)d;
  }
}

void FillDims(bz_bcast_desc* d, const std::vector<TIndex>& out) {
  BLAZE_CONDITION_THROW(!out.empty() && out.size() <= BZ_MAX_RANK, "rank ", out.size(), " outside 1..", BZ_MAX_RANK);
  d->rank = (int)out.size();
  for (size_t k = 0; k < out.size(); ++k) d->dims[k] = (int64_t)out[k];
}

}  // namespace

// ------------------------------------------------------------------------------------------ Reshape
template <class Context>
class ReshapeOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  ReshapeOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {}
  bool RunOnDevice() override {
    Blob* x = this->Input(0);
    Blob* shape_blob = this->Input(1);
    Blob* y = this->Output(0);
    BLAZE_CONDITION_THROW(shape_blob->data_type() == kInt32, "shape->data_type()=", shape_blob->data_type());
    if (shape_src_ != shape_blob->data() || shape_version_ != shape_blob->version() || rshape_.size() != shape_blob->size()) {
      rshape_.resize(shape_blob->size());
      if (shape_blob->device_type() == kCPU) {
        memcpy(rshape_.data(), shape_blob->data(), rshape_.size() * sizeof(int32_t));
      } else {  // a model constant that was placed on the device: fetched once
        context_.Activate();
        HIP_CHECK(hipMemcpy(rshape_.data(), shape_blob->data(), rshape_.size() * sizeof(int32_t), hipMemcpyDeviceToHost));
      }
      shape_src_ = shape_blob->data();
      shape_version_ = shape_blob->version();
    }
    const std::vector<TIndex>& shape = x->shape();
    std::vector<TIndex> new_shape(rshape_.size());
    int unknown_pos = -1;
    TIndex known_size = 1;
    for (size_t i = 0; i < rshape_.size(); ++i) {
      if (rshape_[i] == 0) {
        BLAZE_CONDITION_THROW(i < shape.size(), "shape[", i, "]=0 but the input has rank ", shape.size());
        new_shape[i] = shape[i];
        known_size *= new_shape[i];
      } else if (rshape_[i] < 0) {
        BLAZE_CONDITION_THROW(unknown_pos == -1, "can not support two unknown dims");
        unknown_pos = (int)i;
      } else {
        new_shape[i] = (TIndex)rshape_[i];
        known_size *= new_shape[i];
      }
    }
    if (unknown_pos >= 0) {
      BLAZE_CONDITION_THROW(known_size > 0 && x->size() % known_size == 0, "known_size=", known_size, " x->size()=", x->size());
      new_shape[unknown_pos] = x->size() / known_size;
    } else {
      BLAZE_CONDITION_THROW(known_size == x->size(), "known_size=", known_size, " x->size()=", x->size());
    }
    y->set_data_type((DataType)x->data_type());
    y->RefReshape(new_shape, x->data());
    return true;
  }

 private:
  std::vector<int32_t> rshape_;
  const void* shape_src_ = nullptr;
  uint64_t shape_version_ = 0;
};
REGISTER_HIP_OPERATOR(Reshape, ReshapeOp<HIPContext>);
OPERATOR_SCHEMA(Reshape).NumInputs(2).NumOutputs(1).IdenticalTypeOfInput(0).SetDoc("reshape; the output aliases the input");

// ------------------------------------------------------------------------------------------ Add / Sub / Mul / Div
template <class Context, int OP>
class ElementwiseOp final : public Operator<Context>, public ConcatPieceSource {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  ElementwiseOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {}
  bool DescribePiece(ConcatPiece* piece) override {
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->Output(0);
    if (a->data_type() != b->data_type() || c == a || c == b || a->pitch() != 0 || b->pitch() != 0) return false;
    piece->x = a;
    piece->y = b;
    piece->op = OP;
    piece->shape = BroadcastShape(a->shape(), b->shape(), this->def_);
    c->SetShapeOnly(piece->shape);
    return true;
  }
  bool RunOnDevice() override {
    Blob* a = this->Input(0);
    Blob* b = this->Input(1);
    Blob* c = this->Output(0);
    BLAZE_CONDITION_THROW(a->data_type() == b->data_type(), "a->data_type()=", a->data_type(), " b->data_type()=", b->data_type(),
                          " op=", this->def_.name());
    const std::vector<TIndex> out = BroadcastShape(a->shape(), b->shape(), this->def_);
    // in place is allowed only when the output has the shape of the operand it overwrites
    BLAZE_CONDITION_THROW((c != a || a->shape() == out) && (c != b || b->shape() == out), "in-place output would grow op=",
                          this->def_.name());
    const std::vector<TIndex> as = a->shape(), bs = b->shape();
    c->Reshape(out);
    if (c->size() == 0) return true;
    bz_bcast_desc d;
    memset(&d, 0, sizeof(d));
    d.a = a->data();
    d.b = b->data();
    d.out = c->data();
    FillDims(&d, out);
    OperandStrides(as, out, d.a_stride);
    OperandStrides(bs, out, d.b_stride);
    d.op = OP;
    d.dtype = BzType(a->data_type());
    BZ_CHECK(bz_broadcast_op(&d, context_.hip_stream()));
    return true;
  }
};
#define BLAZE_REGISTER_ELEMENTWISE(Name, OP, doc)                          \
  using Name##HipOp = ElementwiseOp<HIPContext, OP>;                       \
  REGISTER_HIP_OPERATOR(Name, Name##HipOp);                                \
  OPERATOR_SCHEMA(Name).NumInputs(2).NumOutputs(1).IdenticalTypeOfInput(0).AllowInplace({{0, 0}, {1, 0}}).SetDoc(doc)
BLAZE_REGISTER_ELEMENTWISE(Add, BZ_EW_ADD, "a + b = c");
BLAZE_REGISTER_ELEMENTWISE(Sub, BZ_EW_SUB, "a - b = c");
BLAZE_REGISTER_ELEMENTWISE(Mul, BZ_EW_MUL, "a * b = c");
BLAZE_REGISTER_ELEMENTWISE(Div, BZ_EW_DIV, "a / b = c");

// ------------------------------------------------------------------------------------------ BroadcastTo
template <class Context>
class BroadcastToOp final : public Operator<Context>, public ConcatPieceSource {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  BroadcastToOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    broadcast_shape_ = OperatorBase::GetRepeatedArgument<int>("shape");
  }
  bool DescribePiece(ConcatPiece* piece) override {
    Blob* a = this->Input(0);
    Blob* y = this->Output(0);
    if (y == a || a->pitch() != 0) return false;
    piece->x = a;
    piece->y = nullptr;
    piece->op = BZ_EW_ASSIGN;
    piece->shape = TargetShape();
    y->SetShapeOnly(piece->shape);
    return true;
  }
  bool RunOnDevice() override {
    Blob* a = this->Input(0);
    Blob* y = this->Output(0);
    const std::vector<TIndex> as = a->shape();
    const std::vector<TIndex> out = TargetShape();
    BLAZE_CONDITION_THROW(y != a || as == out, "in-place output would grow op=", this->def_.name());
    y->Reshape(out);
    if (y->size() == 0) return true;
    bz_bcast_desc d;
    memset(&d, 0, sizeof(d));
    d.a = a->data();
    d.out = y->data();
    FillDims(&d, out);
    OperandStrides(as, out, d.a_stride);
    d.op = BZ_EW_ASSIGN;
    d.dtype = BzType(a->data_type());
    BZ_CHECK(bz_broadcast_op(&d, context_.hip_stream()));
    return true;
  }

 private:
  // the shape of the second input, or the input's own with the positive entries of `shape` put in
  std::vector<TIndex> TargetShape() {
    const std::vector<TIndex> as = this->Input(0)->shape();
    std::vector<TIndex> out;
    if (this->InputSize() > 1) {
      out = this->Input(1)->shape();
    } else {
      BLAZE_CONDITION_THROW(as.size() == broadcast_shape_.size(), "a->shape().size()=", as.size(),
                            " broadcast_shape_.size()=", broadcast_shape_.size());
      out = as;
      for (size_t i = 0; i < broadcast_shape_.size(); ++i) {
        BLAZE_CONDITION_THROW(broadcast_shape_[i] >= 0, "can not support dim < 0");
        if (broadcast_shape_[i] > 0) out[i] = (TIndex)broadcast_shape_[i];
      }
    }
    BLAZE_CONDITION_THROW(BroadcastShape(as, out, this->def_) == out, "input does not broadcast to the target shape op=",
                          this->def_.name());
    return out;
  }
  std::vector<int> broadcast_shape_;
};
REGISTER_HIP_OPERATOR(BroadcastTo, BroadcastToOp<HIPContext>);
OPERATOR_SCHEMA(BroadcastTo).NumInputs(1, 2).NumOutputs(1).IdenticalTypeOfInput(0).SetDoc("c = BroadcastTo(a)");

// ------------------------------------------------------------------------------------------ Where
template <class Context>
class WhereOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  WhereOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {}
  bool RunOnDevice() override {
    Blob* cond = this->Input(0);
    Blob* x = this->Input(1);
    Blob* y = this->Input(2);
    Blob* z = this->Output(0);
    BLAZE_CONDITION_THROW(x->data_type() == y->data_type(), "x->data_type()=", x->data_type(), " y->data_type()=", y->data_type(),
                          " op=", this->def_.name());
    BLAZE_CONDITION_THROW(cond->data_type() == kInt32 || cond->data_type() == kInt64, "Unsupported type", cond->data_type());
    BLAZE_CONDITION_THROW(z != cond && z != x && z != y, "Where does not run in place");
    const std::vector<TIndex> out = BroadcastShape(BroadcastShape(cond->shape(), x->shape(), this->def_), y->shape(), this->def_);
    z->Reshape(out);
    if (z->size() == 0) return true;
    bz_bcast_desc d;
    memset(&d, 0, sizeof(d));
    d.a = cond->data();
    d.b = x->data();
    d.c = y->data();
    d.out = z->data();
    FillDims(&d, out);
    OperandStrides(cond->shape(), out, d.a_stride);
    OperandStrides(x->shape(), out, d.b_stride);
    OperandStrides(y->shape(), out, d.c_stride);
    d.op = BZ_EW_WHERE;
    d.dtype = BzType(x->data_type());
    d.cond_dtype = BzType(cond->data_type());
    BZ_CHECK(bz_broadcast_op(&d, context_.hip_stream()));
    return true;
  }
};
REGISTER_HIP_OPERATOR(Where, WhereOp<HIPContext>);
OPERATOR_SCHEMA(Where).NumInputs(3).NumOutputs(1).IdenticalTypeOfInput(1).SetDoc(
    "Return elements, either from X or Y, depending on condition");

// ------------------------------------------------------------------------------------------ ReduceSum
template <class Context>
class ReduceSumOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  ReduceSumOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    if (OperatorBase::HasArgument("axes")) {
      const std::vector<int> axes = OperatorBase::GetRepeatedArgument<int>("axes");
      BLAZE_CONDITION_THROW(axes.size() == 1, "axes.size()=", axes.size());
      axis_ = (size_t)axes[0];
    } else {
      axis_ = (size_t)OperatorBase::GetSingleArgument<int>("axis", 0);
    }
    keepdims_ = OperatorBase::GetSingleArgument<int>("keepdims", 1);
  }
  bool RunOnDevice() override {
    Blob* x = this->Input(0);
    Blob* y = this->Output(0);
    const std::vector<TIndex> shape = x->shape();
    BLAZE_CONDITION_THROW(axis_ < shape.size(), "axis_=", axis_, " shape.size()=", shape.size(), " ", this->def_.name());
    BLAZE_CONDITION_THROW(y != x, "ReduceSum does not run in place");
    std::vector<TIndex> new_shape;
    TIndex outer = 1, K = 1, N = 1;
    for (size_t i = 0; i < shape.size(); ++i) {
      if (i == axis_) {
        if (keepdims_) new_shape.push_back(1);
      } else {
        new_shape.push_back(shape[i]);
      }
      if (i < axis_)
        outer *= shape[i];
      else if (i == axis_)
        K = shape[i];
      else
        N *= shape[i];
    }
    y->Reshape(new_shape);
    BZ_CHECK(bz_reduce_sum(x->data(), y->data(), (int64_t)outer, (int64_t)K, (int64_t)N, BzType(x->data_type()),
                           context_.hip_stream()));
    return true;
  }

 private:
  size_t axis_;
  int keepdims_;
};
REGISTER_HIP_OPERATOR(ReduceSum, ReduceSumOp<HIPContext>);
OPERATOR_SCHEMA(ReduceSum).NumInputs(1).NumOutputs(1).IdenticalTypeOfInput(0).SetDoc("sum over one axis");

// ------------------------------------------------------------------------------------------ Gather
// blaze/operator/op/gather_op.h:25-87, gather_op.cc:9-45: output shape = data.shape[:axis] + indices.shape +
// data.shape[axis+1:], y[.., j, ..] = data[.., indices[j], ..]; integer indices (int32 | int64).
template <class Context>
class GatherOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  GatherOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    axis_ = OperatorBase::GetSingleArgument<size_t>("axis", 0);
  }
  bool RunOnDevice() override {
    Blob* data = this->Input(0);
    Blob* indices = this->Input(1);
    Blob* y = this->Output(0);
    BLAZE_CONDITION_THROW(indices->data_type() == kInt32 || indices->data_type() == kInt64, "indices->data_type()=",
                          indices->data_type());
    const std::vector<TIndex> shape = data->shape();
    BLAZE_CONDITION_THROW(axis_ < shape.size(), "axis_=", axis_, " shape.size()=", shape.size(), " ", this->def_.name());
    BLAZE_CONDITION_THROW(y != data && y != indices, "Gather does not run in place");
    std::vector<TIndex> o_shape;
    TIndex outer = 1, inner = 1, n_idx = 1;
    for (size_t i = 0; i < axis_; ++i) {
      o_shape.push_back(shape[i]);
      outer *= shape[i];
    }
    for (TIndex d : indices->shape()) {
      o_shape.push_back(d);
      n_idx *= d;
    }
    for (size_t i = axis_ + 1; i < shape.size(); ++i) {
      o_shape.push_back(shape[i]);
      inner *= shape[i];
    }
    if (y->data_type() != data->data_type()) y->set_data_type((DataType)data->data_type());
    y->Reshape(o_shape);
    BZ_CHECK(bz_gather_rows(data->data(), indices->data(), indices->data_type() == kInt32 ? BZ_I32 : BZ_I64, y->data(), (int64_t)outer,
                            (int64_t)shape[axis_], (int64_t)(inner * DataTypeSize(data->data_type())), (int64_t)n_idx,
                            context_.hip_stream()));
    return true;
  }

 private:
  size_t axis_;
};
REGISTER_HIP_OPERATOR(Gather, GatherOp<HIPContext>);
OPERATOR_SCHEMA(Gather).NumInputs(2).NumOutputs(1).IdenticalTypeOfInput(0).SetDoc("Gather a tensor base on indices.");

// ------------------------------------------------------------------------------------------ Slice
// blaze/operator/op/slice_op.h:30-153, slice_op.cc:9-46: one axis, [start, end) given as axis | axes[1] and start, end |
// starts[1], ends[1] (defaults 0, 0, 1); any other argument name is ignored, as there.  A strided copy: outer rows of
// (end - start) * inner elements.
template <class Context>
class SliceOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  SliceOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    if (OperatorBase::HasArgument("axes")) {
      const std::vector<size_t> axes = OperatorBase::GetRepeatedArgument<size_t>("axes");
      BLAZE_CONDITION_THROW(axes.size() == 1, "axes.size()=", axes.size());
      axis_ = axes[0];
    } else {
      axis_ = OperatorBase::GetSingleArgument<size_t>("axis", 0);
    }
    if (OperatorBase::HasArgument("starts")) {
      const std::vector<size_t> starts = OperatorBase::GetRepeatedArgument<size_t>("starts");
      const std::vector<size_t> ends = OperatorBase::GetRepeatedArgument<size_t>("ends");
      BLAZE_CONDITION_THROW(starts.size() == 1 && ends.size() == 1, "starts.size()=", starts.size(), " ends.size()=", ends.size());
      start_ = starts[0];
      end_ = ends[0];
    } else {
      start_ = OperatorBase::GetSingleArgument<size_t>("start", 0);
      end_ = OperatorBase::GetSingleArgument<size_t>("end", 1);
    }
    BLAZE_CONDITION_THROW(start_ < end_, "Slice start=", start_, " end=", end_);
  }
  bool RunOnDevice() override {
    Blob* x = this->Input(0);
    Blob* y = this->Output(0);
    const std::vector<TIndex> shape = x->shape();
    BLAZE_CONDITION_THROW(axis_ < shape.size(), "axis_=", axis_, " shape.size()=", shape.size(), " ", this->def_.name());
    BLAZE_CONDITION_THROW(end_ <= (size_t)shape[axis_], "axis=", axis_, " shape.size()=", shape.size(), " end_=", end_,
                          " shape[exes_]=", shape[axis_]);
    BLAZE_CONDITION_THROW(y != x, "Slice does not run in place");
    TIndex outer = 1, inner = 1;
    for (size_t i = 0; i < axis_; ++i) outer *= shape[i];
    for (size_t i = axis_ + 1; i < shape.size(); ++i) inner *= shape[i];
    std::vector<TIndex> y_shape = shape;
    y_shape[axis_] = (TIndex)(end_ - start_);
    if (y->data_type() != x->data_type()) y->set_data_type((DataType)x->data_type());
    y->Reshape(y_shape);
    const int64_t es = (int64_t)DataTypeSize(x->data_type());
    bz_concat_desc d;
    memset(&d, 0, sizeof(d));
    d.src[0] = (const char*)x->data() + (int64_t)start_ * inner * es;
    d.width[0] = (int64_t)(end_ - start_) * inner * es;
    d.src_pitch[0] = (int64_t)shape[axis_] * inner * es;
    d.dst = y->data();
    d.dst_pitch = d.width[0];
    d.rows = (int64_t)outer;
    d.n = 1;
    BZ_CHECK(bz_concat_cols(&d, context_.hip_stream()));
    return true;
  }

 private:
  size_t axis_, start_, end_;
};
REGISTER_HIP_OPERATOR(Slice, SliceOp<HIPContext>);
OPERATOR_SCHEMA(Slice).NumInputs(1).NumOutputs(1).IdenticalTypeOfInput(0).SetDoc("Procuce a slice of the input tensor along one axis");

// ------------------------------------------------------------------------------------------ Split
// blaze/operator/op/split_op.h:33-132, split_op.cc:11-44.  Equal parts along axis 0 are views of the input (the
// reference's RefReshape: the optimizer's FusedParallelGemm + Split pair costs no copy); any other split copies each
// part out with one strided copy.
template <class Context>
class SplitOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  SplitOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    axis_ = OperatorBase::GetSingleArgument<size_t>("axis", 1);
    if (OperatorBase::HasArgument("split")) {
      splits_ = OperatorBase::GetRepeatedArgument<size_t>("split");
      BLAZE_CONDITION_THROW(splits_.size() == (size_t)this->OutputSize(), "splits_.size()=", splits_.size(),
                            " this->output_size()=", this->OutputSize());
    }
  }
  int LaunchesOfLastRun() const override { return launches_; }
  bool RunOnDevice() override {
    Blob* x = this->Input(0);
    const int n_out = this->OutputSize();
    const std::vector<TIndex> shape0 = x->shape();
    launches_ = 0;
    BLAZE_CONDITION_THROW(x->pitch() == 0, "Split of a strided view of another tensor");
    if (splits_.empty() && axis_ == 0) {
      BLAZE_CONDITION_THROW(!shape0.empty() && shape0[0] % n_out == 0, "shape[0]=", shape0.empty() ? 0 : shape0[0]);
      std::vector<TIndex> shape = shape0;
      shape[0] /= n_out;
      const size_t part = (size_t)(x->size() / n_out) * DataTypeSize(x->data_type());
      for (int i = 0; i < n_out; ++i) {
        Blob* y = this->Output(i);
        y->set_data_type((DataType)x->data_type());
        y->RefReshape(shape, (char*)x->data() + part * i);
      }
      return true;
    }
    BLAZE_CONDITION_THROW(axis_ < shape0.size(), "axis_=", axis_, " shape0.size()=", shape0.size());
    if (splits_.empty()) {
      BLAZE_CONDITION_THROW(shape0[axis_] % n_out == 0, "shape0[", axis_, "]=", shape0[axis_], " output_size=", n_out,
                            " op=", this->def_.name());
    } else {
      size_t sum_axis = 0;
      for (auto sp : splits_) sum_axis += sp;
      BLAZE_CONDITION_THROW(sum_axis == (size_t)shape0[axis_], "sum_axis=", sum_axis, " shape0[", axis_, "]=", shape0[axis_]);
    }
    const size_t es = DataTypeSize(x->data_type());
    const TIndex outer = x->size(0, (int)axis_), inner = x->size((int)axis_ + 1, (int)shape0.size());
    size_t offset = 0;
    std::vector<TIndex> shape = shape0;
    for (int k = 0; k < n_out; ++k) {
      shape[axis_] = splits_.empty() ? shape0[axis_] / n_out : (TIndex)splits_[k];
      Blob* y = this->Output(k);
      y->set_data_type((DataType)x->data_type());
      y->Reshape(shape);
      if (y->size() > 0) {
        bz_concat_desc d;
        memset(&d, 0, sizeof(d));
        d.n = 1;
        d.src[0] = (const char*)x->data() + offset * inner * es;
        d.width[0] = (int64_t)(shape[axis_] * inner * es);
        d.src_pitch[0] = (int64_t)(shape0[axis_] * inner * es);
        d.dst = y->data();
        d.dst_pitch = d.width[0];
        d.rows = (int64_t)outer;
        BZ_CHECK(bz_concat_cols(&d, context_.hip_stream()));
        ++launches_;
      }
      offset += shape[axis_];
    }
    return true;
  }

 private:
  size_t axis_;
  std::vector<size_t> splits_;
  int launches_ = 0;
};
REGISTER_HIP_OPERATOR(Split, SplitOp<HIPContext>);
OPERATOR_SCHEMA(Split).NumInputs(1).NumOutputs(1, INT_MAX).IdenticalTypeOfInput(0).SetDoc("Split a tensor into many tensors.");

// ------------------------------------------------------------------------------------------ Fuse
template <class Context>
class FuseOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  FuseOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    comm_index_ = OperatorBase::GetSingleArgument<int>("comm_index", 0);
  }
  bool RunOnDevice() override {
    BLAZE_CONDITION_THROW(comm_index_ >= 0 && comm_index_ <= 1, "comm_index_=", comm_index_);
    Blob* x[2] = {this->Input(0), this->Input(1)};
    Blob* y = this->Output(0);
    for (int i = 0; i < 2; ++i) {
      BLAZE_CONDITION_THROW(x[i]->shape().size() == 2, "x->shape().size()=", x[i]->shape().size(), " i=", i);
      if (comm_index_ == i)
        BLAZE_CONDITION_THROW(x[i]->shape()[0] == 1, "x->shape()[0]=", x[i]->shape()[0], " i=", i, " ", this->def_.name());
    }
    BLAZE_CONDITION_THROW(x[0]->data_type() == x[1]->data_type(), "Fuse inputs differ in type");
    const TIndex m0 = x[0]->shape()[0], m1 = x[1]->shape()[0], n0 = x[0]->shape()[1], n1 = x[1]->shape()[1];
    const TIndex ym = std::max(m0, m1);
    // fuse_op.cc:14-21: when input 0 has one row it is the repeated one, otherwise input 1's first row is
    const bool repeat0 = m0 == 1;
    BLAZE_CONDITION_THROW(repeat0 ? (m1 == ym) : (m0 == ym), "Fuse: row counts ", m0, " and ", m1);
    y->Reshape({ym, n0 + n1});
    const size_t es = DataTypeSize(y->data_type());
    bz_concat_desc d;
    memset(&d, 0, sizeof(d));
    d.n = 2;
    d.src[0] = x[0]->data();
    d.src[1] = x[1]->data();
    d.width[0] = (int64_t)(n0 * es);
    d.width[1] = (int64_t)(n1 * es);
    d.src_pitch[0] = repeat0 ? 0 : d.width[0];
    d.src_pitch[1] = repeat0 ? d.width[1] : 0;
    d.dst = y->data();
    d.dst_pitch = (int64_t)((n0 + n1) * es);
    d.rows = (int64_t)ym;
    BZ_CHECK(bz_concat_cols(&d, context_.hip_stream()));
    return true;
  }

 private:
  int comm_index_;
};
REGISTER_HIP_OPERATOR(Fuse, FuseOp<HIPContext>);
OPERATOR_SCHEMA(Fuse).NumInputs(2).NumOutputs(1).IdenticalTypeOfInput(0).SetDoc("fuse operation.");

// ------------------------------------------------------------------------------------------ BatchNormalization
template <class Context>
class BatchNormalizationOp final : public Operator<Context> {
 public:
  USE_OPERATOR_FUNCTIONS(Context);
  BatchNormalizationOp(const OperatorDef& def, Workspace* ws) : Operator<Context>(def, ws) {
    nosqrt_ = OperatorBase::GetSingleArgument<bool>("nosqrt", false);
    eps_ = OperatorBase::GetSingleArgument<float>("eps", 0.001f);  // kBnEpsilon, operator/common_helper.h:89
  }
  bool RunOnDevice() override {
    Blob* x = this->Input(0);
    Blob* p[4] = {this->Input(1), this->Input(2), this->Input(3), this->Input(4)};  // gamma, beta, mean, var
    Blob* y = this->Output(0);
    for (int k = 1; k < 4; ++k) {
      BLAZE_CONDITION_THROW(p[k]->data_type() == p[k - 1]->data_type(), "data_type[", k, "]=", p[k]->data_type(), " data_type[", k - 1,
                            "]=", p[k - 1]->data_type());
      BLAZE_CONDITION_THROW(p[k]->size() == p[k - 1]->size(), "size[", k, "]=", p[k]->size(), "size[", k - 1, "]=", p[k - 1]->size());
    }
    BLAZE_CONDITION_THROW(p[0]->size() > 0, "gamma is empty");
    y->Reshape(x->shape());
    if (x->size() == 0) return true;
    hipStream_t st = context_.hip_stream();
    bz_bn_desc d;
    memset(&d, 0, sizeof(d));
    d.x = x->data();
    d.y = y->data();
    d.gamma = f32_[0].Get(p[0], st);
    d.beta = f32_[1].Get(p[1], st);
    d.mean = f32_[2].Get(p[2], st);
    d.var = f32_[3].Get(p[3], st);
    d.size = (int64_t)x->size();
    d.channels = (int64_t)p[0]->size();
    d.dtype = BzType(x->data_type());
    d.nosqrt = nosqrt_ ? 1 : 0;
    d.eps = eps_;
    BZ_CHECK(bz_batch_norm(&d, st));
    return true;
  }

 private:
  bool nosqrt_ = false;
  float eps_;
  ParamF32 f32_[4];
};
REGISTER_HIP_OPERATOR(BatchNormalization, BatchNormalizationOp<HIPContext>);
OPERATOR_SCHEMA(BatchNormalization).NumInputs(5).NumOutputs(1).AllowInplace({{0, 0}}).IdenticalTypeOfInput(0).SetDoc(
    "batch normalization, inference form");

}  // namespace blaze
