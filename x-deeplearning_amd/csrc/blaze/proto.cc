#include "blaze/proto.h"

#include <stdio.h>
#include <stdlib.h>

#include <fstream>
#include <functional>

namespace blaze {

// ================================================================================ text format
namespace {

struct TextNode;
struct TextValue {
  std::string scalar;                // unquoted token or unescaped string
  std::shared_ptr<TextNode> message; // set for nested messages
};
struct TextNode {
  std::vector<std::pair<std::string, TextValue>> fields;  // in file order
};

class TextParser {
 public:
  explicit TextParser(const std::string& s) : s_(s) {}
  std::shared_ptr<TextNode> ParseTop() {
    auto n = ParseFields('\0');
    return n;
  }

 private:
  void SkipSpace() {
    while (pos_ < s_.size()) {
      char c = s_[pos_];
      if (c == '#') {
        while (pos_ < s_.size() && s_[pos_] != '\n') ++pos_;
      } else if (c == ' ' || c == '\t' || c == '\n' || c == '\r' || c == ',' || c == ';') {
        ++pos_;
      } else {
        break;
      }
    }
  }
  std::string Ident() {
    size_t b = pos_;
    while (pos_ < s_.size() && (isalnum((unsigned char)s_[pos_]) || s_[pos_] == '_' || s_[pos_] == '.' || s_[pos_] == '-' ||
                                s_[pos_] == '+'))
      ++pos_;
    BLAZE_CONDITION_THROW(pos_ > b, "text proto: expected a token at offset ", b);
    return s_.substr(b, pos_ - b);
  }
  std::string Quoted() {
    char q = s_[pos_++];
    std::string out;
    while (pos_ < s_.size() && s_[pos_] != q) {
      char c = s_[pos_++];
      if (c == '\\' && pos_ < s_.size()) {
        char e = s_[pos_++];
        switch (e) {
          case 'n': out += '\n'; break;
          case 't': out += '\t'; break;
          case 'r': out += '\r'; break;
          case '\\': out += '\\'; break;
          case '"': out += '"'; break;
          case '\'': out += '\''; break;
          default:
            if (e >= '0' && e <= '7') {  // octal escape
              int v = e - '0';
              for (int k = 0; k < 2 && pos_ < s_.size() && s_[pos_] >= '0' && s_[pos_] <= '7'; ++k) v = v * 8 + (s_[pos_++] - '0');
              out += (char)v;
            } else {
              out += e;
            }
        }
      } else {
        out += c;
      }
    }
    BLAZE_CONDITION_THROW(pos_ < s_.size(), "text proto: unterminated string");
    ++pos_;
    return out;
  }
  std::shared_ptr<TextNode> ParseFields(char close) {
    auto node = std::make_shared<TextNode>();
    while (true) {
      SkipSpace();
      if (pos_ >= s_.size()) {
        BLAZE_CONDITION_THROW(close == '\0', "text proto: missing '", close, "'");
        return node;
      }
      if (s_[pos_] == close) {
        ++pos_;
        return node;
      }
      std::string name = Ident();
      SkipSpace();
      bool colon = false;
      if (pos_ < s_.size() && s_[pos_] == ':') {
        colon = true;
        ++pos_;
        SkipSpace();
      }
      BLAZE_CONDITION_THROW(pos_ < s_.size(), "text proto: value missing for ", name);
      TextValue v;
      if (s_[pos_] == '{' || s_[pos_] == '<') {
        char c = s_[pos_] == '{' ? '}' : '>';
        ++pos_;
        v.message = ParseFields(c);
      } else {
        BLAZE_CONDITION_THROW(colon, "text proto: ':' expected after ", name);
        if (s_[pos_] == '"' || s_[pos_] == '\'') {
          v.scalar = Quoted();
          SkipSpace();
          while (pos_ < s_.size() && (s_[pos_] == '"' || s_[pos_] == '\'')) {  // adjacent strings concatenate
            v.scalar += Quoted();
            SkipSpace();
          }
        } else {
          v.scalar = Ident();
        }
      }
      node->fields.emplace_back(std::move(name), std::move(v));
    }
  }
  const std::string& s_;
  size_t pos_ = 0;
};

int64_t ToInt(const std::string& s) {
  if (s == "true") return 1;
  if (s == "false") return 0;
  char* end = nullptr;
  long long v = strtoll(s.c_str(), &end, 0);
  if (*end != '\0') {  // "1.0" in an integer field: accept integral floats like TextFormat does not; be strict
    unsigned long long u = strtoull(s.c_str(), &end, 0);
    BLAZE_CONDITION_THROW(*end == '\0', "text proto: bad integer '", s, "'");
    return (int64_t)u;
  }
  return v;
}
float ToFloat(std::string s) {
  if (!s.empty() && (s.back() == 'f' || s.back() == 'F')) s.pop_back();
  char* end = nullptr;
  float v = strtof(s.c_str(), &end);
  BLAZE_CONDITION_THROW(end != s.c_str() && *end == '\0', "text proto: bad float '", s, "'");
  return v;
}
int EnumOrInt(const std::string& s, const std::map<std::string, int>& names) {
  auto it = names.find(s);
  return it != names.end() ? it->second : (int)ToInt(s);
}

const std::map<std::string, int> kDataTypeNames = {{"kFloat", 1}, {"kInt32", 2}, {"kByte", 3}, {"kString", 4},
                                                   {"kBool", 5},  {"kUInt8", 6}, {"kInt8", 7}, {"kUInt16", 8},
                                                   {"kInt16", 9}, {"kInt64", 10}, {"kFloat16", 12}, {"kDouble", 13}};
const std::map<std::string, int> kInputTypeNames = {{"kInputDense", 0}, {"kInputSparseIds", 1}, {"kInputSparseValues", 2},
                                                    {"kInputSparseSegments", 3}, {"kInputIndicator", 4}};
const std::map<std::string, int> kTruncNames = {{"kInorder", 0}, {"kReverse", 1}};

void FromText(const TextNode& n, Argument* a) {
  for (const auto& f : n.fields) {
    const std::string& k = f.first;
    const std::string& v = f.second.scalar;
    if (k == "name") a->name = v;
    else if (k == "f") { a->f = ToFloat(v); a->has_f = true; }
    else if (k == "i") { a->i = ToInt(v); a->has_i = true; }
    else if (k == "s") { a->s = v; a->has_s = true; }
    else if (k == "floats") a->floats.push_back(ToFloat(v));
    else if (k == "ints") a->ints.push_back(ToInt(v));
    else if (k == "strings") a->strings.push_back(v);
  }
}
void FromText(const TextNode& n, DeviceOption* d) {
  for (const auto& f : n.fields) {
    if (f.first == "device_type") d->device_type_ = (int)ToInt(f.second.scalar);
    else if (f.first == "device_id") d->device_id_ = (int)ToInt(f.second.scalar);
    else if (f.first == "is_pipe") d->is_pipe_ = ToInt(f.second.scalar) != 0;
  }
}
void FromText(const TextNode& n, OperatorDef* o) {
  for (const auto& f : n.fields) {
    const std::string& k = f.first;
    if (k == "type") o->type_ = f.second.scalar;
    else if (k == "name") o->name_ = f.second.scalar;
    else if (k == "input") o->input_.push_back(f.second.scalar);
    else if (k == "output") o->output_.push_back(f.second.scalar);
    else if (k == "doc_string") o->doc_string_ = f.second.scalar;
    else if (k == "arg" && f.second.message) { o->arg_.emplace_back(); FromText(*f.second.message, &o->arg_.back()); }
    else if (k == "device_option" && f.second.message) { o->has_device_option_ = true; FromText(*f.second.message, &o->device_option_); }
  }
}
void FromText(const TextNode& n, ValueInfo* v) {
  for (const auto& f : n.fields) {
    const std::string& k = f.first;
    if (k == "name") v->name_ = f.second.scalar;
    else if (k == "dtype") v->dtype_ = EnumOrInt(f.second.scalar, kDataTypeNames);
    else if (k == "doc_string") v->doc_string_ = f.second.scalar;
    else if (k == "level") v->level_ = (int)ToInt(f.second.scalar);
    else if (k == "input_type") v->input_type_ = EnumOrInt(f.second.scalar, kInputTypeNames);
    else if (k == "feature_name") v->feature_name_ = f.second.scalar;
    else if (k == "tensor_shape" && f.second.message)
      for (const auto& d : f.second.message->fields)
        if (d.first == "dims") v->tensor_shape_.dims.push_back(ToInt(d.second.scalar));
  }
}

}  // namespace

void ParseNetDefText(const std::string& text, NetDef* out) {
  TextParser p(text);
  auto top = p.ParseTop();
  *out = NetDef();
  for (const auto& f : top->fields) {
    const std::string& k = f.first;
    if (k == "name") out->name_ = f.second.scalar;
    else if (k == "run_mode") out->run_mode_ = f.second.scalar;
    else if (k == "version") out->version_ = (int)ToInt(f.second.scalar);
    else if (k == "model_str") out->model_str_ = f.second.scalar;
    else if (k == "op" && f.second.message) { out->op_.emplace_back(); FromText(*f.second.message, &out->op_.back()); }
    else if (k == "arg" && f.second.message) { out->arg_.emplace_back(); FromText(*f.second.message, &out->arg_.back()); }
    else if (k == "device_option" && f.second.message) { out->has_device_option_ = true; FromText(*f.second.message, &out->device_option_); }
    else if (k == "external_input" && f.second.message) { out->external_input_.emplace_back(); FromText(*f.second.message, &out->external_input_.back()); }
    else if (k == "external_output" && f.second.message) { out->external_output_.emplace_back(); FromText(*f.second.message, &out->external_output_.back()); }
  }
}

void ParseEmbeddingConfigText(const std::string& text, EmbeddingConfig* out) {
  TextParser p(text);
  auto top = p.ParseTop();
  *out = EmbeddingConfig();
  for (const auto& f : top->fields) {
    if (f.first == "feature_group_config" && f.second.message) {
      EmbeddingFeatureGroupConfig c;
      bool has_fg = false, has_table = false;
      for (const auto& g : f.second.message->fields) {
        if (g.first == "feature_group") { c.feature_group = g.second.scalar; has_fg = true; }
        else if (g.first == "table_name") { c.table_name = g.second.scalar; has_table = true; }
        else if (g.first == "dim") c.dim = (int)ToInt(g.second.scalar);
      }
      BLAZE_CONDITION_THROW(has_fg && has_table, "feature_group_config needs feature_group and table_name (required fields)");
      out->feature_group_config.push_back(c);
    } else if (f.first == "block_config" && f.second.message) {
      EmbeddingBlockConfig b;
      for (const auto& g : f.second.message->fields) {
        if (g.first == "stride") b.stride = (uint64_t)ToInt(g.second.scalar);
        else if (g.first == "embedding_block_config_item" && g.second.message) {
          EmbeddingBlockConfigItem it;
          bool has_fg = false;
          for (const auto& h : g.second.message->fields) {
            if (h.first == "feature_group") { it.feature_group = h.second.scalar; has_fg = true; }
            else if (h.first == "udf_type") it.udf_type = (int)ToInt(h.second.scalar);
            else if (h.first == "trunc_direction") it.trunc_direction = EnumOrInt(h.second.scalar, kTruncNames);
            else if (h.first == "trunc_num") it.trunc_num = (int)ToInt(h.second.scalar);
            else if (h.first == "offset") it.offset = (uint64_t)ToInt(h.second.scalar);
          }
          BLAZE_CONDITION_THROW(has_fg, "embedding_block_config_item needs feature_group (required field)");
          b.embedding_block_config_item.push_back(it);
        }
      }
      out->block_config.push_back(b);
    }
  }
}

// ================================================================================ wire format
namespace {

struct Reader {
  const uint8_t* p;
  const uint8_t* end;
  bool ok = true;
  bool Done() const { return p >= end; }
  uint64_t Varint() {
    uint64_t v = 0;
    int shift = 0;
    while (p < end && shift < 64) {
      uint8_t b = *p++;
      v |= (uint64_t)(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
      shift += 7;
    }
    ok = false;
    return 0;
  }
  uint32_t Fixed32() {
    if (end - p < 4) { ok = false; return 0; }
    uint32_t v;
    memcpy(&v, p, 4);
    p += 4;
    return v;
  }
  Reader Sub() {
    uint64_t n = Varint();
    if (!ok || (uint64_t)(end - p) < n) { ok = false; return Reader{p, p}; }
    Reader r{p, p + n};
    p += n;
    return r;
  }
  void Skip(int wt) {
    switch (wt) {
      case 0: Varint(); break;
      case 1: if (end - p < 8) ok = false; else p += 8; break;
      case 2: Sub(); break;
      case 5: Fixed32(); break;
      default: ok = false;
    }
  }
};
std::string Str(Reader r) { return std::string((const char*)r.p, (size_t)(r.end - r.p)); }
float AsFloat(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

bool Decode(Reader r, Argument* a) {
  while (r.ok && !r.Done()) {
    uint64_t key = r.Varint();
    int fn = (int)(key >> 3), wt = (int)(key & 7);
    if (fn == 1 && wt == 2) a->name = Str(r.Sub());
    else if (fn == 2 && wt == 5) { a->f = AsFloat(r.Fixed32()); a->has_f = true; }
    else if (fn == 3 && wt == 0) { a->i = (int64_t)r.Varint(); a->has_i = true; }
    else if (fn == 4 && wt == 2) { a->s = Str(r.Sub()); a->has_s = true; }
    else if (fn == 5 && wt == 2) { Reader s = r.Sub(); while (s.ok && !s.Done()) a->floats.push_back(AsFloat(s.Fixed32())); r.ok &= s.ok; }
    else if (fn == 5 && wt == 5) a->floats.push_back(AsFloat(r.Fixed32()));
    else if (fn == 6 && wt == 2) { Reader s = r.Sub(); while (s.ok && !s.Done()) a->ints.push_back((int64_t)s.Varint()); r.ok &= s.ok; }
    else if (fn == 6 && wt == 0) a->ints.push_back((int64_t)r.Varint());
    else if (fn == 7 && wt == 2) a->strings.push_back(Str(r.Sub()));
    else r.Skip(wt);
  }
  return r.ok;
}
bool Decode(Reader r, DeviceOption* d) {
  while (r.ok && !r.Done()) {
    uint64_t key = r.Varint();
    int fn = (int)(key >> 3), wt = (int)(key & 7);
    if (fn == 1 && wt == 0) d->device_type_ = (int32_t)r.Varint();
    else if (fn == 2 && wt == 0) d->device_id_ = (int32_t)r.Varint();
    else if (fn == 3 && wt == 0) d->is_pipe_ = r.Varint() != 0;
    else r.Skip(wt);
  }
  return r.ok;
}
bool Decode(Reader r, OperatorDef* o) {
  while (r.ok && !r.Done()) {
    uint64_t key = r.Varint();
    int fn = (int)(key >> 3), wt = (int)(key & 7);
    if (fn == 1 && wt == 2) o->type_ = Str(r.Sub());
    else if (fn == 2 && wt == 2) o->name_ = Str(r.Sub());
    else if (fn == 3 && wt == 2) o->input_.push_back(Str(r.Sub()));
    else if (fn == 4 && wt == 2) o->output_.push_back(Str(r.Sub()));
    else if (fn == 5 && wt == 2) { o->arg_.emplace_back(); r.ok &= Decode(r.Sub(), &o->arg_.back()); }
    else if (fn == 6 && wt == 2) { o->has_device_option_ = true; r.ok &= Decode(r.Sub(), &o->device_option_); }
    else if (fn == 7 && wt == 2) o->doc_string_ = Str(r.Sub());
    else r.Skip(wt);
  }
  return r.ok;
}
bool Decode(Reader r, ValueInfo* v) {
  while (r.ok && !r.Done()) {
    uint64_t key = r.Varint();
    int fn = (int)(key >> 3), wt = (int)(key & 7);
    if (fn == 1 && wt == 2) v->name_ = Str(r.Sub());
    else if (fn == 2 && wt == 0) v->dtype_ = (int32_t)r.Varint();
    else if (fn == 3 && wt == 2) v->doc_string_ = Str(r.Sub());
    else if (fn == 4 && wt == 0) v->level_ = (int32_t)r.Varint();
    else if (fn == 5 && wt == 0) v->input_type_ = (int32_t)r.Varint();
    else if (fn == 6 && wt == 2) v->feature_name_ = Str(r.Sub());
    else if (fn == 7 && wt == 2) {
      Reader s = r.Sub();
      while (s.ok && !s.Done()) {
        uint64_t k2 = s.Varint();
        if ((k2 >> 3) == 1 && (k2 & 7) == 0) v->tensor_shape_.dims.push_back((int64_t)s.Varint());
        else if ((k2 >> 3) == 1 && (k2 & 7) == 2) { Reader t = s.Sub(); while (t.ok && !t.Done()) v->tensor_shape_.dims.push_back((int64_t)t.Varint()); s.ok &= t.ok; }
        else s.Skip((int)(k2 & 7));
      }
      r.ok &= s.ok;
    } else r.Skip(wt);
  }
  return r.ok;
}

struct Writer {
  std::string* out;
  void Varint(uint64_t v) {
    while (v >= 0x80) { out->push_back((char)(v | 0x80)); v >>= 7; }
    out->push_back((char)v);
  }
  void Key(int fn, int wt) { Varint(((uint64_t)fn << 3) | wt); }
  void Bytes(int fn, const std::string& s) { Key(fn, 2); Varint(s.size()); out->append(s); }
  void Int(int fn, int64_t v) { Key(fn, 0); Varint((uint64_t)v); }
  void Float(int fn, float f) { Key(fn, 5); out->append((const char*)&f, 4); }
};
void Encode(const Argument& a, std::string* out) {
  Writer w{out};
  if (!a.name.empty()) w.Bytes(1, a.name);
  if (a.has_f) w.Float(2, a.f);
  if (a.has_i) w.Int(3, a.i);
  if (a.has_s) w.Bytes(4, a.s);
  if (!a.floats.empty()) w.Bytes(5, std::string((const char*)a.floats.data(), a.floats.size() * 4));
  if (!a.ints.empty()) {
    std::string packed;
    Writer pw{&packed};
    for (int64_t v : a.ints) pw.Varint((uint64_t)v);
    w.Bytes(6, packed);
  }
  for (const auto& s : a.strings) w.Bytes(7, s);
}
void Encode(const DeviceOption& d, std::string* out) {
  Writer w{out};
  w.Int(1, d.device_type_);
  w.Int(2, d.device_id_);
  if (d.is_pipe_) w.Int(3, 1);
}
void Encode(const OperatorDef& o, std::string* out) {
  Writer w{out};
  w.Bytes(1, o.type_);
  if (!o.name_.empty()) w.Bytes(2, o.name_);
  for (const auto& s : o.input_) w.Bytes(3, s);
  for (const auto& s : o.output_) w.Bytes(4, s);
  for (const auto& a : o.arg_) { std::string sub; Encode(a, &sub); w.Bytes(5, sub); }
  if (o.has_device_option_) { std::string sub; Encode(o.device_option_, &sub); w.Bytes(6, sub); }
  if (!o.doc_string_.empty()) w.Bytes(7, o.doc_string_);
}
void Encode(const ValueInfo& v, std::string* out) {
  Writer w{out};
  w.Bytes(1, v.name_);
  w.Int(2, v.dtype_);
  if (!v.doc_string_.empty()) w.Bytes(3, v.doc_string_);
  w.Int(4, v.level_);
  w.Int(5, v.input_type_);
  if (!v.feature_name_.empty()) w.Bytes(6, v.feature_name_);
  if (!v.tensor_shape_.dims.empty()) {
    std::string sub;
    Writer sw{&sub};
    for (int64_t d : v.tensor_shape_.dims) sw.Int(1, d);
    w.Bytes(7, sub);
  }
}

}  // namespace

bool ParseNetDefBinary(const void* data, size_t len, NetDef* out) {
  *out = NetDef();
  Reader r{(const uint8_t*)data, (const uint8_t*)data + len};
  bool saw_op = false;
  while (r.ok && !r.Done()) {
    uint64_t key = r.Varint();
    int fn = (int)(key >> 3), wt = (int)(key & 7);
    if (fn == 0) return false;
    if (fn == 1 && wt == 2) out->name_ = Str(r.Sub());
    else if (fn == 2 && wt == 2) { out->op_.emplace_back(); r.ok &= Decode(r.Sub(), &out->op_.back()); saw_op = true; }
    else if (fn == 3 && wt == 2) out->run_mode_ = Str(r.Sub());
    else if (fn == 4 && wt == 2) { out->arg_.emplace_back(); r.ok &= Decode(r.Sub(), &out->arg_.back()); }
    else if (fn == 5 && wt == 2) { out->has_device_option_ = true; r.ok &= Decode(r.Sub(), &out->device_option_); }
    else if (fn == 6 && wt == 2) { out->external_input_.emplace_back(); r.ok &= Decode(r.Sub(), &out->external_input_.back()); }
    else if (fn == 7 && wt == 2) { out->external_output_.emplace_back(); r.ok &= Decode(r.Sub(), &out->external_output_.back()); }
    else if (fn == 8 && wt == 2) out->model_str_ = Str(r.Sub());
    else if (fn == 9 && wt == 0) out->version_ = (int32_t)r.Varint();
    else r.Skip(wt);
  }
  for (const auto& op : out->op_)
    if (op.type_.empty()) return false;  // `type` is a required field of OperatorDef
  return r.ok && (saw_op || len == 0 || !out->name_.empty());
}

void SerializeNetDefBinary(const NetDef& net, std::string* out) {
  out->clear();
  Writer w{out};
  if (!net.name_.empty()) w.Bytes(1, net.name_);
  for (const auto& o : net.op_) { std::string sub; Encode(o, &sub); w.Bytes(2, sub); }
  w.Bytes(3, net.run_mode_);
  for (const auto& a : net.arg_) { std::string sub; Encode(a, &sub); w.Bytes(4, sub); }
  if (net.has_device_option_) { std::string sub; Encode(net.device_option_, &sub); w.Bytes(5, sub); }
  for (const auto& v : net.external_input_) { std::string sub; Encode(v, &sub); w.Bytes(6, sub); }
  for (const auto& v : net.external_output_) { std::string sub; Encode(v, &sub); w.Bytes(7, sub); }
  if (!net.model_str_.empty()) w.Bytes(8, net.model_str_);
  w.Int(9, net.version_);
}

namespace {
std::string Quote(const std::string& s) {
  std::string o = "\"";
  for (unsigned char c : s) {
    if (c == '"' || c == '\\') { o += '\\'; o += (char)c; }
    else if (c == '\n') o += "\\n";
    else if (c < 32 || c >= 127) { char b[8]; snprintf(b, sizeof(b), "\\%03o", c); o += b; }
    else o += (char)c;
  }
  return o + "\"";
}
void TextArg(const Argument& a, const std::string& ind, std::stringstream& ss) {
  ss << ind << "arg {\n";
  ss << ind << "  name: " << Quote(a.name) << "\n";
  char b[64];
  if (a.has_f) { snprintf(b, sizeof(b), "%.9g", a.f); ss << ind << "  f: " << b << "\n"; }
  if (a.has_i) ss << ind << "  i: " << a.i << "\n";
  if (a.has_s) ss << ind << "  s: " << Quote(a.s) << "\n";
  for (float f : a.floats) { snprintf(b, sizeof(b), "%.9g", f); ss << ind << "  floats: " << b << "\n"; }
  for (int64_t v : a.ints) ss << ind << "  ints: " << v << "\n";
  for (const auto& v : a.strings) ss << ind << "  strings: " << Quote(v) << "\n";
  ss << ind << "}\n";
}
void TextValueInfo(const char* field, const ValueInfo& v, std::stringstream& ss) {
  ss << field << " {\n  name: " << Quote(v.name_) << "\n  dtype: " << v.dtype_ << "\n";
  if (!v.doc_string_.empty()) ss << "  doc_string: " << Quote(v.doc_string_) << "\n";
  ss << "  level: " << v.level_ << "\n  input_type: " << v.input_type_ << "\n";
  if (!v.feature_name_.empty()) ss << "  feature_name: " << Quote(v.feature_name_) << "\n";
  if (!v.tensor_shape_.dims.empty()) {
    ss << "  tensor_shape {\n";
    for (int64_t d : v.tensor_shape_.dims) ss << "    dims: " << d << "\n";
    ss << "  }\n";
  }
  ss << "}\n";
}
}  // namespace

void SerializeNetDefText(const NetDef& net, std::string* out) {
  std::stringstream ss;
  if (!net.name_.empty()) ss << "name: " << Quote(net.name_) << "\n";
  for (const auto& o : net.op_) {
    ss << "op {\n  type: " << Quote(o.type_) << "\n";
    if (!o.name_.empty()) ss << "  name: " << Quote(o.name_) << "\n";
    for (const auto& i : o.input_) ss << "  input: " << Quote(i) << "\n";
    for (const auto& i : o.output_) ss << "  output: " << Quote(i) << "\n";
    for (const auto& a : o.arg_) TextArg(a, "  ", ss);
    if (o.has_device_option_)
      ss << "  device_option {\n    device_type: " << o.device_option_.device_type_ << "\n    device_id: "
         << o.device_option_.device_id_ << "\n  }\n";
    if (!o.doc_string_.empty()) ss << "  doc_string: " << Quote(o.doc_string_) << "\n";
    ss << "}\n";
  }
  ss << "run_mode: " << Quote(net.run_mode_) << "\n";
  for (const auto& a : net.arg_) TextArg(a, "", ss);
  if (net.has_device_option_)
    ss << "device_option {\n  device_type: " << net.device_option_.device_type_ << "\n  device_id: "
       << net.device_option_.device_id_ << "\n}\n";
  for (const auto& v : net.external_input_) TextValueInfo("external_input", v, ss);
  for (const auto& v : net.external_output_) TextValueInfo("external_output", v, ss);
  if (!net.model_str_.empty()) ss << "model_str: " << Quote(net.model_str_) << "\n";
  ss << "version: " << net.version_ << "\n";
  *out = ss.str();
}

bool LoadNetDefFromFile(const char* path, NetDef* out, std::string* err) {
  std::ifstream is(path, std::ios::binary);
  if (!is.is_open()) {
    if (err) *err = std::string("can not open ") + path;
    return false;
  }
  std::string data((std::istreambuf_iterator<char>(is)), std::istreambuf_iterator<char>());
  if (ParseNetDefBinary(data.data(), data.size(), out) && out->op_size() > 0) return true;
  try {
    ParseNetDefText(data, out);
    if (out->op_size() > 0) return true;
    if (err) *err = "no operators found";
  } catch (std::exception& e) {
    if (err) *err = e.what();
  }
  return false;
}

// ================================================================================ arguments
std::string OperatorDef::DebugString() const {
  std::stringstream ss;
  ss << "op { type: \"" << type_ << "\" name: \"" << name_ << "\"";
  for (const auto& i : input_) ss << " input: \"" << i << "\"";
  for (const auto& o : output_) ss << " output: \"" << o << "\"";
  ss << " }";
  return ss.str();
}

#define BZ_SINGLE(T, expr)                                                                                       \
  template <>                                                                                                    \
  T ArgumentHelper::GetSingle<T>(const std::vector<Argument>& args, const std::string& name, const T& def) {     \
    const Argument* a = Find(args, name);                                                                        \
    if (!a) return def;                                                                                          \
    return expr;                                                                                                 \
  }
BZ_SINGLE(float, a->has_f ? a->f : (a->has_i ? (float)a->i : def))
BZ_SINGLE(double, a->has_f ? (double)a->f : (a->has_i ? (double)a->i : def))
BZ_SINGLE(bool, a->has_i ? a->i != 0 : def)
BZ_SINGLE(int, a->has_i ? (int)a->i : def)
BZ_SINGLE(int64_t, a->has_i ? a->i : def)
BZ_SINGLE(size_t, a->has_i ? (size_t)a->i : def)
BZ_SINGLE(std::string, a->has_s ? a->s : def)
#undef BZ_SINGLE

#define BZ_REPEATED(T, field, conv)                                                                               \
  template <>                                                                                                     \
  std::vector<T> ArgumentHelper::GetRepeated<T>(const std::vector<Argument>& args, const std::string& name,       \
                                                const std::vector<T>& def) {                                      \
    const Argument* a = Find(args, name);                                                                         \
    if (!a) return def;                                                                                           \
    std::vector<T> out;                                                                                           \
    out.reserve(a->field.size());                                                                                 \
    for (const auto& v : a->field) out.push_back(conv(v));                                                        \
    return out;                                                                                                   \
  }
BZ_REPEATED(float, floats, (float))
BZ_REPEATED(double, floats, (double))
BZ_REPEATED(int, ints, (int))
BZ_REPEATED(int64_t, ints, (int64_t))
BZ_REPEATED(size_t, ints, (size_t))
BZ_REPEATED(std::string, strings, std::string)
#undef BZ_REPEATED

}  // namespace blaze
