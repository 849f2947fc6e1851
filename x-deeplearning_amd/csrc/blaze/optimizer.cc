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

namespace {

struct Constant {
  int idx = -1;
  std::vector<int64_t> shape;
  int64_t dtype = kFloat;
  std::vector<float> value;
};

// the ConstantFill that makes `name` for operator `before`, with float values of the expected count
bool ReadConstant(const NetDef& net, const std::string& name, int before, Constant* c) {
  c->idx = ProducerOf(net, name, before);
  if (c->idx < 0 || net.op_[c->idx].type_ != "ConstantFill") return false;
  const auto& args = net.op_[c->idx].arg_;
  c->shape = ArgumentHelper::GetRepeated<int64_t>(args, "shape");
  c->dtype = ArgumentHelper::GetSingle<int64_t>(args, "dtype", kFloat);
  c->value = ArgumentHelper::GetRepeated<float>(args, "value");
  if (c->dtype != kFloat && c->dtype != kFloat16) return false;
  int64_t n = 1;
  for (int64_t d : c->shape) n *= d;
  return !c->shape.empty() && n > 0 && (int64_t)c->value.size() == n;
}

void WriteConstant(OperatorDef* op, const std::vector<int64_t>& shape, int64_t dtype, const std::vector<float>& value) {
  auto arg = [&](const char* name) {
    Argument* a = FindArg(op, name);
    if (a == nullptr) {
      op->arg_.push_back(Argument());
      a = &op->arg_.back();
      a->name = name;
    }
    return a;
  };
  Argument* s = arg("shape");
  s->ints.assign(shape.begin(), shape.end());
  Argument* d = arg("dtype");
  d->i = dtype;
  d->has_i = true;
  Argument* v = arg("value");
  v->floats = value;
  v->ints.clear();
}

// C[m, n] = scale * op(A)[m, k] * op(B)[k, n], row major, fp32 sums in k order
std::vector<float> MatMul(const std::vector<float>& a, bool ta, const std::vector<float>& b, bool tb, int64_t m, int64_t n, int64_t k,
                          float scale) {
  std::vector<float> c((size_t)(m * n));
  for (int64_t i = 0; i < m; ++i)
    for (int64_t j = 0; j < n; ++j) {
      float acc = 0.f;
      for (int64_t q = 0; q < k; ++q) acc += (ta ? a[q * m + i] : a[i * k + q]) * (tb ? b[j * k + q] : b[q * n + j]);
      c[i * n + j] = scale * acc;
    }
  return c;
}

}  // namespace

int FuseGemmChains(NetDef* net) {
  int fused = 0;
  for (;;) {
    bool changed = false;
    for (int i = 0; i < net->op_size() && !changed; ++i) {
      const OperatorDef second = net->op_[i];
      if (second.type_ != "Gemm" || second.input_size() < 2 || second.input_size() > 3 || second.output_size() != 1) continue;
      const int j = ProducerOf(*net, second.input(0), i);
      if (j < 0) continue;
      const OperatorDef first = net->op_[j];
      if (first.type_ != "Gemm" || first.input_size() < 2 || first.input_size() > 3 || first.output_size() != 1) continue;
      if (Readers(*net, first.output(0)) != 1) continue;  // somebody else wants the layer between the two
      bool clean = true;  // the second Gemm will read the first one's input: nothing in between may overwrite that name
      for (int q = j + 1; q < i; ++q)
        for (const auto& out : net->op_[q].output_) clean &= (out != first.input(0));
      if (!clean) continue;
      // (the reference looks at the second Gemm's transA only and drops the first one's; both are refused here)
      if (ArgumentHelper::GetSingle<int64_t>(first.arg_, "transA", 0) != 0 || ArgumentHelper::GetSingle<int64_t>(second.arg_, "transA", 0) != 0)
        continue;
      const bool tb0 = ArgumentHelper::GetSingle<int64_t>(first.arg_, "transB", 0) != 0;
      const bool tb1 = ArgumentHelper::GetSingle<int64_t>(second.arg_, "transB", 0) != 0;
      const float alpha0 = ArgumentHelper::GetSingle<float>(first.arg_, "alpha", 1.f), beta0 = ArgumentHelper::GetSingle<float>(first.arg_, "beta", 1.f);
      const float alpha1 = ArgumentHelper::GetSingle<float>(second.arg_, "alpha", 1.f), beta1 = ArgumentHelper::GetSingle<float>(second.arg_, "beta", 1.f);
      Constant w0, w1, b0, b1;
      if (!ReadConstant(*net, first.input(1), j, &w0) || !ReadConstant(*net, second.input(1), i, &w1)) continue;
      if (w0.shape.size() != 2 || w1.shape.size() != 2 || w0.dtype != w1.dtype) continue;
      // constants that are rewritten must belong to this pair alone
      if (Readers(*net, second.input(1)) != 1) continue;
      const bool has_b0 = first.input_size() == 3, has_b1 = second.input_size() == 3;
      if (has_b0 && (!ReadConstant(*net, first.input(2), j, &b0) || b0.dtype != w1.dtype)) continue;
      if (has_b1 && (!ReadConstant(*net, second.input(2), i, &b1) || b1.dtype != w1.dtype || Readers(*net, second.input(2)) != 1)) continue;
      if (has_b0 && !has_b1 && Readers(*net, first.input(2)) != 1) continue;
      int64_t m = w0.shape[0], k0 = w0.shape[1], k1 = w1.shape[0], n = w1.shape[1];
      if (tb0) std::swap(m, k0);
      if (tb1) std::swap(k1, n);
      if (k0 != k1) continue;
      // biases: a row [K] / [N], or one row per sample [M0, K] / [M0, N] on both sides
      std::vector<int64_t> bias_shape;
      std::vector<float> bias;
      if (has_b0) {
        const int64_t rows = b0.shape.size() == 1 ? 1 : b0.shape[0];
        if (b0.shape.size() > 2 || b0.shape.back() != k1) continue;
        // alpha1 * (alpha0 * A * W0 + beta0 * b0) * W1: the first bias passes through the second product and its alpha
        // (the reference's CalcNewBias leaves alpha1 out, gemm_gemm_fusion_pattern_impl.cc; its fixtures have alpha1 = 1)
        bias = MatMul(b0.value, false, w1.value, tb1, rows, n, k1, alpha1 * beta0);
        bias_shape = b0.shape.size() == 1 ? std::vector<int64_t>{n} : std::vector<int64_t>{rows, n};
      }
      if (has_b1) {
        if (b1.shape.size() > 2 || b1.shape.back() != n) continue;
        if (!has_b0) {
          bias_shape = b1.shape;
          bias.assign(b1.value.size(), 0.f);
        } else if (b1.shape.size() > bias_shape.size()) {  // a row against a matrix: the row repeats
          std::vector<float> wide(b1.value.size());
          for (size_t q = 0; q < wide.size(); ++q) wide[q] = bias[q % bias.size()];
          bias.swap(wide);
          bias_shape = b1.shape;
        } else if (b1.shape.size() == 2 && b1.shape != bias_shape) {
          continue;
        }
        for (size_t q = 0; q < bias.size(); ++q) bias[q] += beta1 * b1.value[q % b1.value.size()];
      }
      // rewrite: weight into the second Gemm's constant, bias into the surviving bias constant
      WriteConstant(&net->op_[w1.idx], {m, n}, w1.dtype, MatMul(w0.value, tb0, w1.value, tb1, m, n, k0, 1.f));
      OperatorDef gemm = second;
      gemm.input_ = {first.input(0), second.input(1)};
      if (has_b1 || has_b0) {
        const Constant& keep = has_b1 ? b1 : b0;
        WriteConstant(&net->op_[keep.idx], bias_shape, w1.dtype, bias);
        gemm.input_.push_back(has_b1 ? second.input(2) : first.input(2));
      }
      gemm.arg_.clear();
      Argument a;
      a.name = "alpha";
      a.f = alpha0 * alpha1;
      a.has_f = true;
      gemm.arg_.push_back(a);
      a.name = "beta";
      a.f = 1.f;
      gemm.arg_.push_back(a);
      net->op_[i] = gemm;
      // the first Gemm goes, and with it the constants nobody reads any more
      std::set<int> drop = {j};
      net->op_[j].input_.clear();  // (so that Readers below no longer counts it)
      if (Readers(*net, first.input(1)) == 0) drop.insert(w0.idx);
      if (has_b0 && has_b1 && Readers(*net, first.input(2)) == 0) drop.insert(b0.idx);
      std::vector<OperatorDef> ops;
      for (int q = 0; q < net->op_size(); ++q)
        if (!drop.count(q)) ops.push_back(net->op_[q]);
      net->op_.swap(ops);
      ++fused;
      changed = true;
    }
    if (!changed) return fused;
  }
}

}  // namespace blaze
