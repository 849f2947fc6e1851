// optimizer.cc -- see optimizer.h.
#include "blaze/optimizer.h"

#include <map>
#include <set>

namespace blaze {

namespace {

// what CanFusion compares (parallel_gemm_fusion_pattern_impl.cc:116-140)
struct GemmInfo {
  int idx = -1;           // position of the Gemm in net->op_
  int weight = -1;        // position of the ConstantFill that makes input(1)
  int bias = -1;          // position of the ConstantFill that makes input(2); -1: the Gemm has no bias
  bool trans_a = false, trans_b = false;
  float alpha = 1.f, beta = 1.f;
  std::vector<int64_t> shape, bias_shape;
  int64_t weight_dtype = kFloat, bias_dtype = kFloat;
};

int ProducerOf(const NetDef& net, const std::string& name, int before) {
  for (int j = before - 1; j >= 0; --j)
    for (const auto& out : net.op_[j].output_)
      if (out == name) return j;
  return -1;
}

int Readers(const NetDef& net, const std::string& name) {
  int n = 0;
  for (const auto& op : net.op_)
    for (const auto& in : op.input_) n += (in == name);
  for (const auto& eo : net.external_output_) n += (eo.name_ == name);
  return n;
}

bool SameKind(const GemmInfo& m, const GemmInfo& n) {
  if (m.weight_dtype != n.weight_dtype || m.trans_a != n.trans_a || m.trans_b != n.trans_b) return false;
  if (m.alpha != n.alpha || m.beta != n.beta) return false;
  if (m.shape.size() != 2 || n.shape.size() != 2 || m.shape != n.shape) return false;
  // the reference fills a missing bias with zeros; here a group is all with bias or all without
  if ((m.bias < 0) != (n.bias < 0)) return false;
  if (m.bias >= 0) {
    if (m.bias_dtype != n.bias_dtype || m.bias_shape != n.bias_shape || m.bias_shape.empty() || m.bias_shape.size() > 2) return false;
    const size_t diff = m.shape.size() - m.bias_shape.size();
    for (size_t i = 0; i < m.bias_shape.size(); ++i)
      if (m.shape[i + diff] != m.bias_shape[i]) return false;
  }
  return true;
}

Argument* FindArg(OperatorDef* op, const std::string& name) {
  for (auto& a : op->arg_)
    if (a.name == name) return &a;
  return nullptr;
}

// values of a ConstantFill as the reference stores them: `value` floats for the float types
bool AppendValues(OperatorDef* dst, const OperatorDef& src) {
  Argument* d = FindArg(dst, "value");
  const Argument* s = ArgumentHelper::Find(src.arg_, "value");
  if (d == nullptr || s == nullptr) return false;
  d->floats.insert(d->floats.end(), s->floats.begin(), s->floats.end());
  d->ints.insert(d->ints.end(), s->ints.begin(), s->ints.end());
  return true;
}

}  // namespace

int FuseParallelGemms(NetDef* net) {
  int fused = 0;
  for (;;) {
    // Gemms grouped by the tensor they read; every member has constant operands
    std::map<std::string, std::vector<GemmInfo>> by_input;
    std::vector<std::string> order;
    for (int i = 0; i < net->op_size(); ++i) {
      const OperatorDef& op = net->op_[i];
      if (op.type_ != "Gemm" || op.input_size() < 2 || op.input_size() > 3 || op.output_size() != 1) continue;
      GemmInfo g;
      g.idx = i;
      g.weight = ProducerOf(*net, op.input(1), i);
      if (g.weight < 0 || net->op_[g.weight].type_ != "ConstantFill" || Readers(*net, op.input(1)) != 1) continue;
      const auto& wargs = net->op_[g.weight].arg_;
      g.shape = ArgumentHelper::GetRepeated<int64_t>(wargs, "shape");
      g.weight_dtype = ArgumentHelper::GetSingle<int64_t>(wargs, "dtype", kFloat);
      if (op.input_size() == 3) {
        g.bias = ProducerOf(*net, op.input(2), i);
        if (g.bias < 0 || net->op_[g.bias].type_ != "ConstantFill" || Readers(*net, op.input(2)) != 1) continue;
        g.bias_shape = ArgumentHelper::GetRepeated<int64_t>(net->op_[g.bias].arg_, "shape");
        g.bias_dtype = ArgumentHelper::GetSingle<int64_t>(net->op_[g.bias].arg_, "dtype", kFloat);
      }
      g.trans_a = ArgumentHelper::GetSingle<int64_t>(op.arg_, "transA", 0) != 0;
      g.trans_b = ArgumentHelper::GetSingle<int64_t>(op.arg_, "transB", 0) != 0;
      g.alpha = ArgumentHelper::GetSingle<float>(op.arg_, "alpha", 1.f);
      g.beta = ArgumentHelper::GetSingle<float>(op.arg_, "beta", 1.f);
      // the shared input must be the same tensor for all members: nobody writes its name between them (checked below)
      if (!by_input.count(op.input(0))) order.push_back(op.input(0));
      by_input[op.input(0)].push_back(g);
    }
    // first group of at least two compatible Gemms (GenerateFusionCandidate: greedy, in net order)
    std::vector<GemmInfo> group;
    for (const auto& name : order) {
      const auto& all = by_input[name];
      for (size_t i = 0; i < all.size() && group.empty(); ++i) {
        std::vector<GemmInfo> cand = {all[i]};
        for (size_t j = i + 1; j < all.size(); ++j)
          if (SameKind(all[i], all[j])) cand.push_back(all[j]);
        if (cand.size() < 2) continue;
        bool clean = true;  // no operator between the first and the last member writes the shared input or a member's output
        for (int k = cand.front().idx + 1; k < cand.back().idx && clean; ++k)
          for (const auto& out : net->op_[k].output_) {
            clean &= (out != name);
            for (const auto& g : cand) clean &= (k == g.idx || out != net->op_[g.idx].output(0));
          }
        // an operator between the first and a later member must not read that member's output before it existed: true
        // by construction (names are written before they are read), and the fused operator sits at the first member's
        // place, which is after the shared input's producer
        if (clean) group = cand;
      }
      if (!group.empty()) break;
    }
    if (group.empty()) return fused;
    ++fused;
    const std::string fname = "fused_parallel_gemm_" + std::to_string(fused);
    const int P = (int)group.size();
    // stacked weight and bias live in the first member's constants
    OperatorDef* w0 = &net->op_[group[0].weight];
    for (int p = 1; p < P; ++p) AppendValues(w0, net->op_[group[p].weight]);
    if (Argument* sh = FindArg(w0, "shape")) sh->ints[0] *= P;
    if (group[0].bias >= 0) {
      OperatorDef* b0 = &net->op_[group[0].bias];
      for (int p = 1; p < P; ++p) AppendValues(b0, net->op_[group[p].bias]);
      if (Argument* sh = FindArg(b0, "shape")) sh->ints[0] *= P;
    }
    const OperatorDef first = net->op_[group[0].idx];
    OperatorDef gemm;
    gemm.type_ = "FusedParallelGemm";
    gemm.name_ = fname;
    gemm.arg_ = first.arg_;
    Argument pn;
    pn.name = "parallel_num";
    pn.i = P;
    pn.has_i = true;
    gemm.arg_.push_back(pn);
    gemm.input_ = first.input_;
    gemm.output_ = {fname};
    gemm.device_option_ = first.device_option_;
    gemm.has_device_option_ = first.has_device_option_;
    OperatorDef split;
    split.type_ = "Split";
    split.name_ = "fused_parallel_gemm_split_" + std::to_string(fused);
    split.input_ = {fname};
    for (const auto& g : group) split.output_.push_back(net->op_[g.idx].output(0));
    Argument ax;
    ax.name = "axis";
    ax.i = 0;
    ax.has_i = true;
    split.arg_.push_back(ax);
    split.device_option_ = first.device_option_;
    split.has_device_option_ = first.has_device_option_;
    // rebuild the operator list: the pair takes the first member's place, the members and the constants only they
    // read disappear
    std::set<int> drop;
    for (int p = 0; p < P; ++p) {
      drop.insert(group[p].idx);
      if (p > 0) {
        drop.insert(group[p].weight);
        if (group[p].bias >= 0) drop.insert(group[p].bias);
      }
    }
    std::vector<OperatorDef> ops;
    for (int i = 0; i < net->op_size(); ++i) {
      if (i == group[0].idx) {
        ops.push_back(gemm);
        ops.push_back(split);
      }
      if (!drop.count(i)) ops.push_back(net->op_[i]);
    }
    net->op_.swap(ops);
  }
}

}  // namespace blaze
