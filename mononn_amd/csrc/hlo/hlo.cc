#include "hlo/hlo.h"

#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <set>
#include <sstream>

#include "common/json.h"
#include "common/status.h"

namespace mononn {
namespace hlo {

namespace {
struct DTypeInfo {
  DType t;
  const char* name;
  int bytes;
  const char* ctype;
};
const DTypeInfo kDTypes[] = {
    {DType::kPred, "pred", 1, "bool"},       {DType::kS8, "s8", 1, "int8_t"},
    {DType::kS16, "s16", 2, "int16_t"},      {DType::kS32, "s32", 4, "int32_t"},
    {DType::kS64, "s64", 8, "int64_t"},      {DType::kU8, "u8", 1, "uint8_t"},
    {DType::kU16, "u16", 2, "uint16_t"},     {DType::kU32, "u32", 4, "uint32_t"},
    {DType::kU64, "u64", 8, "uint64_t"},     {DType::kF16, "f16", 2, "_Float16"},
    {DType::kF32, "f32", 4, "float"},        {DType::kF64, "f64", 8, "double"},
    {DType::kBF16, "bf16", 2, "__bf16"},
};

// Opcode set of mononn_engine/core/op/op_type.h:20-58 plus `fusion`; everything else is rejected
// the way ir_parser_fused.cc:311 does.  A few harmless extras XLA prints in the same position
// (`sqrt`, `power`, `and`, `or`, `not`) are accepted because the emitter handles them.
const std::set<std::string>& known_opcodes() {
  static const std::set<std::string> s = {
      "abs", "add", "bitcast", "broadcast", "clamp", "compare", "concatenate", "constant", "convert",
      "convolution", "copy", "custom-call", "divide", "dot", "dynamic-slice", "dynamic-update-slice",
      "exponential", "gather", "get-tuple-element", "iota", "log", "maximum", "minimum", "multiply",
      "negate", "pad", "parameter", "reduce", "reduce-window", "reshape", "rsqrt", "select", "sign",
      "slice", "subtract", "tanh", "transpose", "tuple", "fusion", "sqrt", "power", "and", "or", "not"};
  return s;
}
}  // namespace

const char* dtype_name(DType t) {
  for (auto& d : kDTypes)
    if (d.t == t) return d.name;
  return t == DType::kTuple ? "tuple" : "invalid";
}
int dtype_bytes(DType t) {
  for (auto& d : kDTypes)
    if (d.t == t) return d.bytes;
  return 0;
}
const char* dtype_ctype(DType t) {
  for (auto& d : kDTypes)
    if (d.t == t) return d.ctype;
  return "void";
}
DType dtype_from_name(const std::string& s) {
  for (auto& d : kDTypes)
    if (s == d.name) return d.t;
  return DType::kInvalid;
}

std::string Shape::to_string() const {
  if (is_tuple()) {
    std::string s = "(";
    for (size_t i = 0; i < tuple.size(); ++i) s += (i ? ", " : "") + tuple[i].to_string();
    return s + ")";
  }
  std::string s = std::string(dtype_name(dtype)) + "[";
  for (size_t i = 0; i < dims.size(); ++i) s += (i ? "," : "") + std::to_string(dims[i]);
  return s + "]";
}

std::string canonical_name(const std::string& n) {
  std::string s = n;
  if (!s.empty() && s[0] == '%') s.erase(0, 1);
  for (auto& c : s)
    if (c == '.' || c == '-') c = '_';
  return s;
}

std::string module_short_name(const std::string& module_name) {
  const std::string prefix = "cluster_";
  MONONN_CHECK(module_name.compare(0, prefix.size(), prefix) == 0, kInvalidArgument)
      << "module name '" << module_name << "' does not start with cluster_<id>";
  size_t i = prefix.size();
  while (i < module_name.size() && isdigit(static_cast<unsigned char>(module_name[i]))) ++i;
  MONONN_CHECK(i > prefix.size(), kInvalidArgument) << "module name '" << module_name << "' has no cluster id";
  return module_name.substr(0, i);
}

// ------------------------------------------------------------------------------------------
namespace {

class Lexer {
 public:
  explicit Lexer(const std::string& s) : s_(s) {}
  size_t pos = 0;
  int line = 1;

  bool eof() {
    skip_ws();
    return pos >= s_.size();
  }
  void skip_ws() {
    while (pos < s_.size()) {
      char c = s_[pos];
      if (c == '\n') {
        ++line;
        ++pos;
      } else if (c == ' ' || c == '\t' || c == '\r') {
        ++pos;
      } else if (c == '/' && pos + 1 < s_.size() && s_[pos + 1] == '/') {
        while (pos < s_.size() && s_[pos] != '\n') ++pos;
      } else if (c == '/' && pos + 1 < s_.size() && s_[pos + 1] == '*') {
        size_t e = s_.find("*/", pos + 2);
        if (e == std::string::npos) fail("unterminated comment");
        for (size_t i = pos; i < e; ++i)
          if (s_[i] == '\n') ++line;
        pos = e + 2;
      } else {
        break;
      }
    }
  }
  char peek() {
    skip_ws();
    return pos < s_.size() ? s_[pos] : '\0';
  }
  bool consume(char c) {
    if (peek() == c) {
      ++pos;
      return true;
    }
    return false;
  }
  void expect(char c) {
    if (!consume(c)) fail(std::string("expected '") + c + "'");
  }
  bool consume_word(const std::string& w) {
    skip_ws();
    if (s_.compare(pos, w.size(), w) == 0) {
      size_t e = pos + w.size();
      if (e >= s_.size() || !(isalnum(static_cast<unsigned char>(s_[e])) || s_[e] == '_')) {
        pos = e;
        return true;
      }
    }
    return false;
  }
  // identifier characters used by HLO names and opcodes
  std::string ident() {
    skip_ws();
    size_t st = pos;
    if (pos < s_.size() && s_[pos] == '%') ++pos;
    while (pos < s_.size()) {
      char c = s_[pos];
      if (isalnum(static_cast<unsigned char>(c)) || c == '_' || c == '.' || c == '-' || c == '$') ++pos;
      else break;
    }
    if (st == pos) fail("expected identifier");
    return s_.substr(st, pos - st);
  }
  // balanced blob starting at an opening bracket, returned including the brackets
  std::string balanced() {
    skip_ws();
    size_t st = pos;
    int depth = 0;
    bool in_q = false;
    while (pos < s_.size()) {
      char c = s_[pos];
      if (in_q) {
        if (c == '\\') ++pos;
        else if (c == '"') in_q = false;
      } else if (c == '"') {
        in_q = true;
      } else if (c == '(' || c == '{' || c == '[') {
        ++depth;
      } else if (c == ')' || c == '}' || c == ']') {
        --depth;
        if (depth == 0) {
          ++pos;
          return s_.substr(st, pos - st);
        }
      } else if (c == '\n') {
        ++line;
      }
      ++pos;
    }
    fail("unbalanced brackets");
  }
  std::string quoted() {
    skip_ws();
    if (pos >= s_.size() || s_[pos] != '"') fail("expected string");
    ++pos;
    std::string out;
    while (pos < s_.size() && s_[pos] != '"') {
      if (s_[pos] == '\\' && pos + 1 < s_.size()) {
        ++pos;
        out.push_back(s_[pos]);
      } else {
        out.push_back(s_[pos]);
      }
      ++pos;
    }
    if (pos >= s_.size()) fail("unterminated string");
    ++pos;
    return out;
  }
  // attribute value: balanced blob, quoted string, or bare token up to a top-level ',' / newline
  std::string attr_value() {
    char c = peek();
    if (c == '{' || c == '(' || c == '[') return balanced();
    if (c == '"') return quoted();
    size_t st = pos;
    while (pos < s_.size() && s_[pos] != ',' && s_[pos] != '\n' && s_[pos] != ' ' && s_[pos] != '}') ++pos;
    return s_.substr(st, pos - st);
  }
  [[noreturn]] void fail(const std::string& what) {
    MONONN_FAIL(kParseError) << "HLO text line " << line << ": " << what;
  }
  const std::string& text() const { return s_; }

 private:
  const std::string& s_;
};

std::vector<int64_t> ints_of(const std::string& s) {
  std::vector<int64_t> v;
  size_t i = 0;
  while (i < s.size()) {
    if (isdigit(static_cast<unsigned char>(s[i])) || (s[i] == '-' && i + 1 < s.size() && isdigit(static_cast<unsigned char>(s[i + 1])))) {
      size_t st = i++;
      while (i < s.size() && isdigit(static_cast<unsigned char>(s[i]))) ++i;
      v.push_back(std::strtoll(s.substr(st, i - st).c_str(), nullptr, 10));
    } else {
      ++i;
    }
  }
  return v;
}

Shape parse_shape(Lexer& lx) {
  Shape sh;
  if (lx.peek() == '(') {
    lx.expect('(');
    sh.dtype = DType::kTuple;
    if (lx.peek() != ')') {
      do {
        sh.tuple.push_back(parse_shape(lx));
        if (sh.tuple.back().is_tuple()) MONONN_FAIL(kUnsupported) << "nested tuple shapes are not supported";
      } while (lx.consume(','));
    }
    lx.expect(')');
    return sh;
  }
  std::string t = lx.ident();
  sh.dtype = dtype_from_name(t);
  if (sh.dtype == DType::kInvalid) MONONN_FAIL(kUnsupported) << "line " << lx.line << ": unsupported element type '" << t << "'";
  lx.expect('[');
  while (lx.peek() != ']') {
    lx.skip_ws();
    if (lx.peek() == '<' || lx.peek() == '?') MONONN_FAIL(kUnsupported) << "line " << lx.line << ": dynamic dimensions are not supported";
    std::string num;
    while (isdigit(static_cast<unsigned char>(lx.text()[lx.pos]))) num.push_back(lx.text()[lx.pos++]);
    if (num.empty()) lx.fail("expected dimension");
    sh.dims.push_back(std::strtoll(num.c_str(), nullptr, 10));
    lx.consume(',');
  }
  lx.expect(']');
  // optional layout directly attached: {1,0} ; tiling / element size / memory space annotations rejected
  if (lx.pos < lx.text().size() && lx.text()[lx.pos] == '{') {
    std::string lay = lx.balanced();
    if (lay.find(':') != std::string::npos) MONONN_FAIL(kUnsupported) << "line " << lx.line << ": tiled or annotated layouts are not supported: " << lay;
    for (auto v : ints_of(lay)) sh.minor_to_major.push_back(static_cast<int>(v));
    MONONN_CHECK(sh.minor_to_major.size() == sh.dims.size(), kParseError) << "layout rank mismatch in " << lay;
    std::vector<bool> seen(sh.dims.size(), false);
    for (int d : sh.minor_to_major) {
      MONONN_CHECK(d >= 0 && d < static_cast<int>(sh.dims.size()) && !seen[d], kParseError) << "line " << lx.line << ": layout " << lay << " is not a permutation of the dimensions";
      seen[d] = true;
    }
  } else {
    for (int i = static_cast<int>(sh.dims.size()) - 1; i >= 0; --i) sh.minor_to_major.push_back(i);
  }
  return sh;
}

void decode_gemm_config(Instr* ins) {
  auto it = ins->attrs.find("backend_config");
  MONONN_CHECK(it != ins->attrs.end(), kParseError) << ins->hlo_name << ": __cublas$gemm without backend_config";
  Json top = Json::parse(it->second);
  // newer XLA nests the fields: {"gemm_backend_config": {...}}
  const Json& j = top.contains("gemm_backend_config") ? top.at("gemm_backend_config") : top;
  GemmConfig& g = ins->gemm;
  g.alpha_real = j.at("alpha_real").as_double();
  if (j.contains("alpha_imag")) g.alpha_imag = j.at("alpha_imag").as_double();
  g.beta = j.at("beta").as_double();
  const Json& dn = j.at("dot_dimension_numbers");
  const Json& lc = dn.at("lhs_contracting_dimensions");
  const Json& rc = dn.at("rhs_contracting_dimensions");
  MONONN_CHECK(lc.size() == 1 && rc.size() == 1, kUnsupported) << ins->hlo_name << ": exactly one contracting dimension per operand is supported";
  g.lhs_contracting = static_cast<int>(lc.at(size_t(0)).as_int());
  g.rhs_contracting = static_cast<int>(rc.at(size_t(0)).as_int());
  g.batch_size = j.contains("batch_size") ? j.at("batch_size").as_int() : 1;
  if (dn.contains("lhs_batch_dimensions"))
    for (auto& v : dn.at("lhs_batch_dimensions").items()) g.lhs_batch.push_back(static_cast<int>(v.as_int()));
  if (dn.contains("rhs_batch_dimensions"))
    for (auto& v : dn.at("rhs_batch_dimensions").items()) g.rhs_batch.push_back(static_cast<int>(v.as_int()));
  if (j.contains("lhs_stride")) g.lhs_stride = j.at("lhs_stride").as_int();
  if (j.contains("rhs_stride")) g.rhs_stride = j.at("rhs_stride").as_int();
  if (j.contains("selected_algorithm")) {
    const Json& a = j.at("selected_algorithm");
    g.selected_algorithm = a.is_string() ? a.as_string() : std::to_string(a.as_int());
  }
}

// __cublas$lt$matmul(a, b[, c][, bias]): what newer XLA versions print instead of __cublas$gemm.  Same
// gemm_backend_config plus `epilogue`; operand c is present when beta != 0, the bias vector (one value per result
// column) when the epilogue names it; the result may come as a (matrix, workspace) tuple.  The reference knows only
// __cublas$gemm (core/op/custom_call.cc:96-100, :165-167) and applies alpha / beta as gemm_impl.cc:182-231 reads
// them; the epilogue semantics here are cuBLASLt's as XLA's GEMM rewriter uses them, reconstructed without a dump of
// such a module at hand: D = act(alpha * A.B + beta * C + bias), act = identity, max(x, 0) or tanh-GELU.
void decode_lt_matmul_config(Instr* ins) {
  decode_gemm_config(ins);
  auto it = ins->attrs.find("backend_config");
  Json top = Json::parse(it->second);
  const Json& j = top.contains("gemm_backend_config") ? top.at("gemm_backend_config") : top;
  std::string ep = "DEFAULT";
  if (j.contains("epilogue")) {
    const Json& e = j.at("epilogue");
    static const char* by_number[] = {"DEFAULT", "BIAS", "RELU", "BIAS_RELU", "GELU", "BIAS_GELU", "GELU_AUX", "BIAS_GELU_AUX"};
    if (e.is_string()) ep = e.as_string();
    else {
      const int64_t k = e.as_int();
      MONONN_CHECK(k >= 0 && k < 8, kUnsupported) << ins->hlo_name << ": unknown epilogue number " << k;
      ep = by_number[k];
    }
  }
  MONONN_CHECK(ep == "DEFAULT" || ep == "BIAS" || ep == "RELU" || ep == "GELU" || ep == "BIAS_RELU" || ep == "BIAS_GELU", kUnsupported)
      << ins->hlo_name << ": epilogue " << ep << " of __cublas$lt$matmul is not supported (an auxiliary output has no place in the one-result call)";
  ins->gemm.epilogue = ep;
  const size_t want = 2 + (ins->gemm.beta != 0 ? 1 : 0) + (ep.rfind("BIAS", 0) == 0 ? 1 : 0);
  MONONN_CHECK(ins->operands.size() == want, kParseError)
      << ins->hlo_name << ": __cublas$lt$matmul with beta " << ins->gemm.beta << " and epilogue " << ep << " takes " << want << " operands, got " << ins->operands.size();
  if (ins->shape.is_tuple()) {
    MONONN_CHECK(!ins->shape.tuple.empty() && !ins->shape.tuple[0].is_tuple(), kParseError) << ins->hlo_name << ": __cublas$lt$matmul yields (matrix, workspace)";
    Shape arr = ins->shape.tuple[0];
    ins->shape = arr;
    ins->lt_tuple_result = true;
  }
}

// window={size=16x16 stride=16x16 pad=1_1x1_1}: fields separated by blanks, dimensions by 'x'
std::map<std::string, std::vector<std::string>> window_fields(const std::string& raw) {
  std::map<std::string, std::vector<std::string>> out;
  std::string s = raw;
  for (char& c : s)
    if (c == '{' || c == '}') c = ' ';
  std::istringstream is(s);
  std::string field;
  while (is >> field) {
    size_t eq = field.find('=');
    if (eq == std::string::npos) continue;
    std::vector<std::string> dims;
    std::string v = field.substr(eq + 1);
    size_t st = 0;
    while (st <= v.size()) {
      size_t e = v.find('x', st);
      dims.push_back(v.substr(st, e == std::string::npos ? std::string::npos : e - st));
      if (e == std::string::npos) break;
      st = e + 1;
    }
    out[field.substr(0, eq)] = dims;
  }
  return out;
}

void decode_conv_config(Instr* ins) {
  auto attr = [&](const char* k) -> std::string {
    auto it = ins->attrs.find(k);
    return it == ins->attrs.end() ? std::string() : it->second;
  };
  MONONN_CHECK(ins->operands.size() == 2, kUnsupported) << ins->hlo_name << ": convolution with a side input / bias operand is not supported";
  MONONN_CHECK(ins->shape.is_tuple() && ins->shape.tuple.size() == 2, kParseError) << ins->hlo_name << ": __cudnn$convForward yields (output, scratch)";
  std::string labels = attr("dim_labels");
  labels.erase(std::remove_if(labels.begin(), labels.end(), [](char c) { return isspace(static_cast<unsigned char>(c)); }), labels.end());
  // the lowering assumes N,H,W,C / K,R,S,C / N,P,Q,K in memory (conv_impl.cc:295-298); with the row-major layouts
  // this parser accepts, that is exactly this labelling
  MONONN_CHECK(labels == "b01f_o01i->b01f", kUnsupported) << ins->hlo_name << ": dim_labels '" << labels << "' (only b01f_o01i->b01f is supported)";
  const std::string fg = attr("feature_group_count");
  MONONN_CHECK(fg.empty() || std::strtoll(fg.c_str(), nullptr, 10) == 1, kUnsupported) << ins->hlo_name << ": grouped convolution is not supported";
  const hlo::Shape &in = ins->operands[0]->shape, &flt = ins->operands[1]->shape, &out = ins->shape.tuple[0];
  MONONN_CHECK(in.rank() == 4 && flt.rank() == 4 && out.rank() == 4, kUnsupported) << ins->hlo_name << ": only 2-d convolutions are supported";
  MONONN_CHECK(is_half_float(in.dtype) && flt.dtype == in.dtype && out.dtype == in.dtype, kUnsupported)
      << ins->hlo_name << ": a convolution's input, filter and output must all be f16 or all be bf16";
  ConvConfig& c = ins->conv;
  c.N = in.dims[0], c.H = in.dims[1], c.W = in.dims[2], c.C = in.dims[3];
  c.K = flt.dims[0], c.R = flt.dims[1], c.S = flt.dims[2];
  c.P = out.dims[1], c.Q = out.dims[2];
  MONONN_CHECK(flt.dims[3] == c.C, kInvalidArgument) << ins->hlo_name << ": channel extents of input and filter differ";
  MONONN_CHECK(out.dims[0] == c.N && out.dims[3] == c.K, kInvalidArgument) << ins->hlo_name << ": output shape does not match the operands";
  auto w = window_fields(attr("window"));
  auto two = [&](const char* key, int64_t dflt, int64_t* a, int64_t* b) {
    auto it = w.find(key);
    if (it == w.end()) {
      *a = *b = dflt;
      return;
    }
    MONONN_CHECK(it->second.size() == 2, kUnsupported) << ins->hlo_name << ": window field " << key << " must have two dimensions";
    *a = std::strtoll(it->second[0].c_str(), nullptr, 10);
    *b = std::strtoll(it->second[1].c_str(), nullptr, 10);
  };
  int64_t sr = 0, ss = 0, d0 = 1, d1 = 1;
  two("size", 0, &sr, &ss);
  MONONN_CHECK(sr == c.R && ss == c.S, kInvalidArgument) << ins->hlo_name << ": window size does not match the filter";
  two("stride", 1, &c.stride_h, &c.stride_w);
  two("lhs_dilate", 1, &d0, &d1);
  MONONN_CHECK(d0 == 1 && d1 == 1, kUnsupported) << ins->hlo_name << ": dilated convolution is not supported";
  two("rhs_dilate", 1, &d0, &d1);
  MONONN_CHECK(d0 == 1 && d1 == 1, kUnsupported) << ins->hlo_name << ": dilated convolution is not supported";
  auto pit = w.find("pad");
  if (pit != w.end()) {
    MONONN_CHECK(pit->second.size() == 2, kUnsupported) << ins->hlo_name << ": pad must have two dimensions";
    int64_t lo[2], hi[2];
    for (int i = 0; i < 2; ++i) {
      const std::string& v = pit->second[i];
      size_t us = v.find('_');
      MONONN_CHECK(us != std::string::npos, kParseError) << ins->hlo_name << ": bad pad field";
      lo[i] = std::strtoll(v.substr(0, us).c_str(), nullptr, 10);
      hi[i] = std::strtoll(v.substr(us + 1).c_str(), nullptr, 10);
      // only symmetric padding (ir_parser_fused.cc:782-798)
      MONONN_CHECK(lo[i] == hi[i] && lo[i] >= 0, kUnsupported) << ins->hlo_name << ": only symmetric, non-negative padding is supported";
    }
    c.pad_h = lo[0];
    c.pad_w = lo[1];
  }
  MONONN_CHECK(c.stride_h >= 1 && c.stride_w >= 1, kInvalidArgument) << ins->hlo_name << ": bad stride";
  MONONN_CHECK((c.H + 2 * c.pad_h - c.R) / c.stride_h + 1 == c.P && (c.W + 2 * c.pad_w - c.S) / c.stride_w + 1 == c.Q, kInvalidArgument)
      << ins->hlo_name << ": output extents do not follow from input, window, stride and padding";
  auto bc = ins->attrs.find("backend_config");
  if (bc != ins->attrs.end()) {
    Json j = Json::parse(bc->second);
    if (j.contains("conv_result_scale")) c.result_scale = j.at("conv_result_scale").as_double();
    if (j.contains("side_input_scale")) {
      MONONN_CHECK(j.at("side_input_scale").as_double() == 0, kUnsupported) << ins->hlo_name << ": side input is not supported";
    }
    if (j.contains("activation_mode")) {
      const Json& a = j.at("activation_mode");
      const std::string mode = a.is_string() ? a.as_string() : std::to_string(a.as_int());
      // conv_impl.cc:245-247 aborts on any other mode
      MONONN_CHECK(mode == "0", kUnsupported) << ins->hlo_name << ": activation mode " << mode << " inside the convolution call is not supported";
    }
  }
  // from here on the call is an array-valued instruction; its get-tuple-element index 0 is an alias of it
  Shape arr = out;
  ins->shape = arr;
}

// dot(lhs, rhs), lhs_batch_dims={0,1}, lhs_contracting_dims={3}, rhs_batch_dims={0,1}, rhs_contracting_dims={2}
// -> the same GemmConfig a __cublas$gemm call carries (alpha 1, beta 0)
void decode_dot_config(Instr* ins) {
  auto dims = [&](const char* k) {
    auto it = ins->attrs.find(k);
    return it == ins->attrs.end() ? std::vector<int64_t>() : ints_of(it->second);
  };
  MONONN_CHECK(ins->operands.size() == 2, kParseError) << ins->hlo_name << ": dot takes two operands";
  auto lc = dims("lhs_contracting_dims"), rc = dims("rhs_contracting_dims"), lb = dims("lhs_batch_dims"), rb = dims("rhs_batch_dims");
  MONONN_CHECK(lc.size() == 1 && rc.size() == 1, kUnsupported) << ins->hlo_name << ": exactly one contracting dimension per operand is supported";
  MONONN_CHECK(lb == rb, kUnsupported) << ins->hlo_name << ": batch dimensions of the two operands must be the same";
  for (size_t i = 0; i < lb.size(); ++i)
    MONONN_CHECK(lb[i] == static_cast<int64_t>(i), kUnsupported) << ins->hlo_name << ": batch dimensions must be the leading dimensions, in order";
  MONONN_CHECK(static_cast<int>(lb.size()) == ins->operands[0]->shape.rank() - 2, kUnsupported)
      << ins->hlo_name << ": every operand must have exactly two non-batch dimensions";
  GemmConfig& g = ins->gemm;
  g.alpha_real = 1;
  g.beta = 0;
  g.lhs_contracting = static_cast<int>(lc[0]);
  g.rhs_contracting = static_cast<int>(rc[0]);
  g.batch_size = 1;
  for (size_t i = 0; i < lb.size(); ++i) {
    g.lhs_batch.push_back(static_cast<int>(lb[i]));
    g.rhs_batch.push_back(static_cast<int>(rb[i]));
    g.batch_size *= ins->operands[0]->shape.dims[lb[i]];
  }
}

// Operand counts, attribute lengths and extents that every later stage relies on (index maps subscript these
// vectors without further checks): a module that gets past here is consistent, whatever text it came from.
void validate_shapes(const Instr* ins) {
  const std::string& op = ins->opcode;
  const Shape& sh = ins->shape;
  auto arity = [&](size_t lo, size_t hi) {
    MONONN_CHECK(ins->operands.size() >= lo && ins->operands.size() <= hi, kParseError)
        << ins->hlo_name << " (" << op << "): " << ins->operands.size() << " operands, expected " << lo << (hi == lo ? "" : " to " + std::to_string(hi));
  };
  auto array_operand = [&](size_t i) -> const Shape& {
    MONONN_CHECK(!ins->operands[i]->shape.is_tuple(), kParseError) << ins->hlo_name << ": operand " << i << " is a tuple";
    return ins->operands[i]->shape;
  };
  auto in_range = [&](int64_t v, int64_t n, const char* what) {
    MONONN_CHECK(v >= 0 && v < n, kParseError) << ins->hlo_name << ": " << what << " " << v << " out of range [0, " << n << ")";
  };
  static const std::set<std::string> unary = {"abs", "convert", "copy", "exponential", "log", "negate", "not", "rsqrt", "sign", "sqrt", "tanh"};
  static const std::set<std::string> binary = {"add", "and", "divide", "maximum", "minimum", "multiply", "or", "power", "subtract", "compare"};
  if (unary.count(op)) {
    arity(1, 1);
    MONONN_CHECK(array_operand(0).dims == sh.dims, kParseError) << ins->hlo_name << ": operand and result shapes differ";
  } else if (binary.count(op)) {
    arity(2, 2);
    MONONN_CHECK(array_operand(0).dims == sh.dims && array_operand(1).dims == sh.dims, kParseError) << ins->hlo_name << ": operand and result shapes differ";
  } else if (op == "select" || op == "clamp") {
    arity(3, 3);
    for (size_t i = 0; i < 3; ++i)
      MONONN_CHECK(array_operand(i).dims == sh.dims || array_operand(i).rank() == 0, kParseError) << ins->hlo_name << ": operand " << i << " does not match the result shape";
  } else if (op == "bitcast" || op == "reshape") {
    arity(1, 1);
    if (!ins->operands[0]->shape.is_tuple())
      MONONN_CHECK(array_operand(0).num_elements() == sh.num_elements(), kParseError) << ins->hlo_name << ": element count changes";
  } else if (op == "broadcast") {
    arity(1, 1);
    const Shape& x = array_operand(0);
    MONONN_CHECK(static_cast<int>(ins->dimensions.size()) == x.rank(), kParseError) << ins->hlo_name << ": dimensions={} must name one result dimension per operand dimension";
    for (int i = 0; i < x.rank(); ++i) {
      in_range(ins->dimensions[i], sh.rank(), "broadcast dimension");
      MONONN_CHECK(sh.dims[ins->dimensions[i]] == x.dims[i], kParseError) << ins->hlo_name << ": broadcast extent mismatch in operand dimension " << i;
    }
  } else if (op == "transpose") {
    arity(1, 1);
    const Shape& x = array_operand(0);
    MONONN_CHECK(static_cast<int>(ins->dimensions.size()) == x.rank() && sh.rank() == x.rank(), kParseError) << ins->hlo_name << ": dimensions={} must be a permutation of the operand's dimensions";
    std::vector<bool> seen(x.rank(), false);
    for (int i = 0; i < x.rank(); ++i) {
      in_range(ins->dimensions[i], x.rank(), "transpose dimension");
      MONONN_CHECK(!seen[ins->dimensions[i]] && sh.dims[i] == x.dims[ins->dimensions[i]], kParseError) << ins->hlo_name << ": not a permutation of the operand's shape";
      seen[ins->dimensions[i]] = true;
    }
  } else if (op == "slice") {
    arity(1, 1);
    const Shape& x = array_operand(0);
    MONONN_CHECK(static_cast<int>(ins->slice_starts.size()) == x.rank() && sh.rank() == x.rank(), kParseError) << ins->hlo_name << ": slice={} must have one range per dimension";
    for (int i = 0; i < x.rank(); ++i)
      MONONN_CHECK(ins->slice_starts[i] >= 0 && ins->slice_limits[i] <= x.dims[i] && ins->slice_limits[i] - ins->slice_starts[i] == sh.dims[i], kParseError)
          << ins->hlo_name << ": slice range of dimension " << i << " does not fit the operand / result";
  } else if (op == "concatenate") {
    arity(1, 1u << 20);
    MONONN_CHECK(ins->dimensions.size() == 1, kParseError) << ins->hlo_name << ": concatenate needs dimensions={d}";
    in_range(ins->dimensions[0], sh.rank(), "concatenate dimension");
    int64_t total = 0;
    for (size_t k = 0; k < ins->operands.size(); ++k) {
      const Shape& x = array_operand(k);
      MONONN_CHECK(x.rank() == sh.rank(), kParseError) << ins->hlo_name << ": operand " << k << " has another rank";
      for (int i = 0; i < sh.rank(); ++i)
        if (i != ins->dimensions[0]) MONONN_CHECK(x.dims[i] == sh.dims[i], kParseError) << ins->hlo_name << ": operand " << k << " differs outside the concatenated dimension";
      total += x.dims[ins->dimensions[0]];
    }
    MONONN_CHECK(total == sh.dims[ins->dimensions[0]], kParseError) << ins->hlo_name << ": operand extents do not add up to the result";
  } else if (op == "pad") {
    arity(2, 2);
    const Shape& x = array_operand(0);
    MONONN_CHECK(static_cast<int>(ins->pad_low.size()) == x.rank() && sh.rank() == x.rank() && array_operand(1).rank() == 0, kParseError)
        << ins->hlo_name << ": padding= must have one entry per dimension and a scalar padding value";
    for (int i = 0; i < x.rank(); ++i)
      MONONN_CHECK(ins->pad_low[i] + x.dims[i] + ins->pad_high[i] == sh.dims[i], kParseError) << ins->hlo_name << ": padded extent of dimension " << i << " does not match the result";
  } else if (op == "iota") {
    arity(0, 0);
    in_range(ins->iota_dimension, std::max(sh.rank(), 1), "iota_dimension");
  } else if (op == "reduce") {
    MONONN_CHECK(ins->operands.size() >= 2 && ins->operands.size() % 2 == 0, kParseError) << ins->hlo_name << ": reduce takes N operands and N init values";
    const Shape& x = array_operand(0);
    MONONN_CHECK(!ins->dimensions.empty(), kParseError) << ins->hlo_name << ": reduce needs dimensions={..}";
    for (auto d : ins->dimensions) in_range(d, x.rank(), "reduced dimension");
    const size_t n = ins->operands.size() / 2;
    MONONN_CHECK(ins->called && ins->called->params.size() == 2 * n, kParseError) << ins->hlo_name << ": the reducer must take " << 2 * n << " parameters";
    MONONN_CHECK(sh.is_tuple() ? sh.tuple.size() == n : n == 1, kParseError) << ins->hlo_name << ": result arity does not match the operands";
    const Shape& out = sh.is_tuple() ? sh.tuple[0] : sh;
    MONONN_CHECK(out.rank() == x.rank() - static_cast<int>(ins->dimensions.size()), kParseError) << ins->hlo_name << ": result rank does not follow from the reduced dimensions";
    for (size_t k = 0; k < n; ++k) MONONN_CHECK(array_operand(k).dims == x.dims && array_operand(n + k).rank() == 0, kParseError) << ins->hlo_name << ": operands must share a shape, init values must be scalars";
  } else if (op == "dynamic-slice") {
    MONONN_CHECK(!ins->operands.empty(), kParseError) << ins->hlo_name << ": no operand";
    const Shape& x = array_operand(0);
    MONONN_CHECK(static_cast<int>(ins->operands.size()) == 1 + x.rank() && static_cast<int>(ins->dynamic_slice_sizes.size()) == x.rank() && sh.rank() == x.rank(), kParseError)
        << ins->hlo_name << ": dynamic-slice takes one scalar start index and one size per dimension";
    for (int i = 0; i < x.rank(); ++i)
      MONONN_CHECK(ins->dynamic_slice_sizes[i] == sh.dims[i] && sh.dims[i] <= x.dims[i] && array_operand(1 + i).rank() == 0, kParseError) << ins->hlo_name << ": slice size of dimension " << i << " does not fit";
  } else if (op == "gather") {
    arity(2, 2);
    array_operand(0);
    array_operand(1);
  } else if (op == "get-tuple-element") {
    arity(1, 1);
    if (ins->operands[0]->shape.is_tuple()) in_range(ins->tuple_index, static_cast<int64_t>(ins->operands[0]->shape.tuple.size()), "tuple index");
  } else if (op == "fusion") {
    MONONN_CHECK(ins->called && ins->called->params.size() == ins->operands.size(), kParseError)
        << ins->hlo_name << ": " << ins->operands.size() << " operands for a computation of " << (ins->called ? ins->called->params.size() : 0) << " parameters";
    for (size_t i = 0; i < ins->operands.size(); ++i)
      MONONN_CHECK(ins->called->params[i]->shape.dims == ins->operands[i]->shape.dims && ins->called->params[i]->shape.dtype == ins->operands[i]->shape.dtype, kParseError)
          << ins->hlo_name << ": operand " << i << " does not match parameter " << i << " of " << ins->called->hlo_name;
  }
}

void decode_attrs(Instr* ins, Module* mod) {
  auto has = [&](const char* k) { return ins->attrs.count(k) > 0; };
  auto get = [&](const char* k) -> const std::string& { return ins->attrs.at(k); };
  auto need = [&](const char* k) -> const std::string& {
    MONONN_CHECK(has(k), kParseError) << ins->hlo_name << " (" << ins->opcode << "): missing attribute " << k;
    return get(k);
  };
  auto comp_ref = [&](const std::string& raw) -> Computation* {
    auto it = mod->by_name.find(canonical_name(raw));
    MONONN_CHECK(it != mod->by_name.end(), kParseError) << ins->hlo_name << ": unknown computation " << raw;
    return it->second;
  };
  const std::string& op = ins->opcode;
  if (op == "broadcast" || op == "transpose" || op == "reduce" || op == "concatenate") {
    if (op != "broadcast" || has("dimensions")) ins->dimensions = ints_of(need("dimensions"));
  }
  if (op == "fusion") {
    ins->called = comp_ref(need("calls"));
    ins->fusion_kind = need("kind");
    MONONN_CHECK(ins->fusion_kind == "kLoop" || ins->fusion_kind == "kInput", kUnsupported)
        << ins->hlo_name << ": fusion kind " << ins->fusion_kind << " is not supported";
  }
  if (op == "reduce" || op == "reduce-window") ins->called = comp_ref(need("to_apply"));
  if (op == "compare") ins->comparison = need("direction");
  if (op == "get-tuple-element") {
    ins->tuple_index = std::strtoll(need("index").c_str(), nullptr, 10);
    if (!ins->operands.empty() && ins->operands[0]->is_conv()) {
      // (output, scratch) of the convolution call: element 0 aliases the call (which has been given the array
      // shape), the scratch buffer is never read (the reference wires only element 0, ir_parser_fused.cc:802-821)
      MONONN_CHECK(ins->tuple_index == 0, kUnsupported) << ins->hlo_name << ": the scratch result of a convolution call cannot be used";
      ins->opcode = "bitcast";
    }
    if (!ins->operands.empty() && ins->operands[0]->lt_tuple_result) {
      MONONN_CHECK(ins->tuple_index == 0, kUnsupported) << ins->hlo_name << ": the workspace of a __cublas$lt$matmul call cannot be used";
      ins->opcode = "bitcast";
    }
  }
  if (op == "iota") ins->iota_dimension = std::strtoll(need("iota_dimension").c_str(), nullptr, 10);
  if (op == "slice") {
    // slice={[0:8192], [2:4:1]}
    const std::string& s = need("slice");
    size_t i = 0;
    while ((i = s.find('[', i)) != std::string::npos) {
      size_t e = s.find(']', i);
      MONONN_CHECK(e != std::string::npos, kParseError) << ins->hlo_name << ": bad slice attribute";
      auto v = ints_of(s.substr(i, e - i));
      MONONN_CHECK(v.size() == 2 || v.size() == 3, kParseError) << ins->hlo_name << ": bad slice attribute";
      ins->slice_starts.push_back(v[0]);
      ins->slice_limits.push_back(v[1]);
      ins->slice_strides.push_back(v.size() == 3 ? v[2] : 1);
      // stride-1 slices only (ir_parser_fused.cc:1321-1327)
      MONONN_CHECK(ins->slice_strides.back() == 1, kUnsupported) << ins->hlo_name << ": strided slice is not supported";
      i = e;
    }
  }
  if (op == "pad") {
    // padding=0_0x1_2 or with interior 0_0_0 ; no interior, non-negative edges (ir_parser_fused.cc:1143-1147)
    const std::string& s = need("padding");
    size_t st = 0;
    while (st <= s.size()) {
      size_t e = s.find('x', st);
      std::string part = s.substr(st, e == std::string::npos ? std::string::npos : e - st);
      std::vector<int64_t> v;
      size_t p = 0;
      while (p <= part.size()) {
        size_t q = part.find('_', p);
        v.push_back(std::strtoll(part.substr(p, q == std::string::npos ? std::string::npos : q - p).c_str(), nullptr, 10));
        if (q == std::string::npos) break;
        p = q + 1;
      }
      MONONN_CHECK(v.size() >= 2, kParseError) << ins->hlo_name << ": bad padding attribute";
      MONONN_CHECK(v[0] >= 0 && v[1] >= 0 && (v.size() < 3 || v[2] == 0), kUnsupported)
          << ins->hlo_name << ": negative or interior padding is not supported";
      ins->pad_low.push_back(v[0]);
      ins->pad_high.push_back(v[1]);
      ins->pad_interior.push_back(0);
      if (e == std::string::npos) break;
      st = e + 1;
    }
  }
  if (op == "dynamic-slice") ins->dynamic_slice_sizes = ints_of(need("dynamic_slice_sizes"));
  if (op == "dynamic-update-slice") {
    MONONN_CHECK(ins->operands.size() >= 2 && static_cast<int>(ins->operands.size()) == 2 + ins->shape.rank() &&
                     ins->operands[0]->shape.dims == ins->shape.dims && ins->operands[1]->shape.rank() == ins->shape.rank(),
                 kUnsupported)
        << ins->hlo_name << ": dynamic-update-slice takes the operand, the update and one scalar start index per dimension";
    for (int i = 0; i < ins->shape.rank(); ++i)
      MONONN_CHECK(ins->operands[1]->shape.dims[i] <= ins->shape.dims[i], kInvalidArgument) << ins->hlo_name << ": the update is larger than the operand";
  }
  if (op == "reduce-window") {
    // one operand and its init value, no dilation (ir_parser_fused.cc:1218-1222, :1246-1250)
    MONONN_CHECK(ins->operands.size() == 2 && !ins->shape.is_tuple(), kUnsupported) << ins->hlo_name << ": reduce-window takes one operand and one init value";
    auto w = window_fields(need("window"));
    MONONN_CHECK(!w.count("lhs_dilate") && !w.count("rhs_dilate"), kUnsupported) << ins->hlo_name << ": window dilation is not supported";
    const hlo::Shape& x = ins->operands[0]->shape;
    const size_t r = static_cast<size_t>(x.rank());
    MONONN_CHECK(w.count("size") && w["size"].size() == r && ins->shape.rank() == x.rank(), kParseError) << ins->hlo_name << ": window size does not match the operand's rank";
    for (size_t i = 0; i < r; ++i) {
      ins->window_size.push_back(std::strtoll(w["size"][i].c_str(), nullptr, 10));
      ins->window_stride.push_back(w.count("stride") && w["stride"].size() == r ? std::strtoll(w["stride"][i].c_str(), nullptr, 10) : 1);
      int64_t lo = 0, hi = 0;
      if (w.count("pad") && w["pad"].size() == r) {
        const std::string& pd = w["pad"][i];
        size_t us = pd.find('_');
        MONONN_CHECK(us != std::string::npos, kParseError) << ins->hlo_name << ": bad window padding '" << pd << "'";
        lo = std::strtoll(pd.substr(0, us).c_str(), nullptr, 10);
        hi = std::strtoll(pd.substr(us + 1).c_str(), nullptr, 10);
      }
      ins->window_pad_low.push_back(lo);
      ins->window_pad_high.push_back(hi);
      MONONN_CHECK(ins->window_size[i] >= 1 && ins->window_stride[i] >= 1 && lo >= 0 && hi >= 0, kUnsupported) << ins->hlo_name << ": negative window padding is not supported";
      const int64_t span = x.dims[i] + lo + hi - ins->window_size[i];
      MONONN_CHECK(span >= 0 && ins->shape.dims[i] == span / ins->window_stride[i] + 1, kInvalidArgument)
          << ins->hlo_name << ": output extent " << ins->shape.dims[i] << " of dimension " << i << " does not follow from the window";
    }
  }
  if (op == "gather") {
    ins->offset_dims = ints_of(need("offset_dims"));
    ins->collapsed_slice_dims = ints_of(need("collapsed_slice_dims"));
    ins->start_index_map = ints_of(need("start_index_map"));
    ins->index_vector_dim = std::strtoll(need("index_vector_dim").c_str(), nullptr, 10);
    ins->slice_sizes = ints_of(need("slice_sizes"));
  }
  if (op == "custom-call") {
    ins->custom_call_target = need("custom_call_target");
    if (ins->custom_call_target == "__cublas$gemm") {
      decode_gemm_config(ins);
    } else if (ins->custom_call_target == "__cublas$lt$matmul") {
      decode_lt_matmul_config(ins);
    } else if (ins->custom_call_target == "__cudnn$convForward") {
      decode_conv_config(ins);
    } else {
      // any other target aborts in the reference (core/op/custom_call.cc:96-100)
      MONONN_FAIL(kUnsupported) << ins->hlo_name << ": custom-call target '" << ins->custom_call_target << "' is not supported";
    }
  }
  if (op == "dot") decode_dot_config(ins);
  if (op == "convolution") {
    // a bare convolution aborts in the reference as well (ir_parser_fused.cc:728-732)
    MONONN_FAIL(kUnsupported) << ins->hlo_name << ": bare convolution is not supported; expected custom-call __cudnn$convForward";
  }
  validate_shapes(ins);
}

// ---- layouts --------------------------------------------------------------------------------------------------------
// Every operation of the dialect is defined on logical indices, so a value's minor-to-major order matters only where
// memory is handed over or reinterpreted: entry parameters, constants whose bytes the host supplies, the results, and
// `bitcast` (same bytes, another shape).  A value with dims L and order m lies in memory as the row-major array
// transpose(value, perm) with perm[i] = m[rank-1-i]; the reference turns the same list into per-dimension positions
// (ir_parser_fused.cc:132-152) and carries them through its index arithmetic.  Here the four places get explicit
// transposes instead, and every instruction leaves with the descending order the rest of the compiler assumes.
bool is_descending(const std::vector<int>& m) {
  for (size_t i = 0; i < m.size(); ++i)
    if (m[i] != static_cast<int>(m.size() - 1 - i)) return false;
  return true;
}

void reset_layout(Shape& s) {
  s.minor_to_major.clear();
  for (int i = s.rank() - 1; i >= 0; --i) s.minor_to_major.push_back(i);
  for (auto& t : s.tuple) reset_layout(t);
}

std::vector<int64_t> major_to_minor(const std::vector<int>& m) { return std::vector<int64_t>(m.rbegin(), m.rend()); }

std::vector<int64_t> inverse_permutation(const std::vector<int64_t>& p) {
  std::vector<int64_t> inv(p.size());
  for (size_t i = 0; i < p.size(); ++i) inv[p[i]] = static_cast<int64_t>(i);
  return inv;
}

std::vector<int64_t> permuted(const std::vector<int64_t>& dims, const std::vector<int64_t>& p) {
  std::vector<int64_t> out(p.size());
  for (size_t i = 0; i < p.size(); ++i) out[i] = dims[p[i]];
  return out;
}

void unlink_user(Instr* operand, const Instr* user) {
  auto& u = operand->users;
  u.erase(std::remove(u.begin(), u.end(), user), u.end());
}

// transposes that exchange the two minor dimensions and keep the leading (batch) ones
bool swaps_minor_pair(const Instr* t) {
  const int r = static_cast<int>(t->dimensions.size());
  if (t->opcode != "transpose" || r < 2 || t->dimensions[r - 1] != r - 2 || t->dimensions[r - 2] != r - 1) return false;
  for (int i = 0; i < r - 2; ++i)
    if (t->dimensions[i] != i) return false;
  return true;
}

void renumber(Computation* comp) {
  for (size_t i = 0; i < comp->instrs.size(); ++i) comp->instrs[i]->index_in_comp = static_cast<int>(i);
}

void normalize_layouts(Computation* comp, std::set<const Instr*>* made) {
  std::map<const Instr*, std::vector<int>> order;   // as written, non-tuple values only
  bool any = false;
  for (auto& up : comp->instrs) {
    if (!up->shape.is_tuple()) {
      order[up.get()] = up->shape.minor_to_major;
      any = any || !is_descending(up->shape.minor_to_major);
    }
    reset_layout(up->shape);
  }
  if (!any) return;
  std::set<std::string> names;
  for (auto& up : comp->instrs) names.insert(up->name);
  auto fresh = [&](const std::string& base) {
    std::string n = base;
    for (int k = 1; names.count(n); ++k) n = base + "_" + std::to_string(k);
    names.insert(n);
    return n;
  };
  std::vector<std::unique_ptr<Instr>> old = std::move(comp->instrs), out;
  // a new one-operand instruction, appended to `out`
  auto make = [&](const std::string& base, const char* opcode, std::vector<int64_t> dims, std::vector<int64_t> dimensions, Instr* operand) {
    auto ins = std::make_unique<Instr>();
    ins->name = ins->hlo_name = fresh(base);
    ins->opcode = opcode;
    ins->shape.dtype = operand->shape.dtype;
    ins->shape.dims = std::move(dims);
    reset_layout(ins->shape);
    ins->dimensions = std::move(dimensions);
    ins->operands = {operand};
    ins->parent = comp;
    operand->users.push_back(ins.get());
    if (ins->opcode == "transpose") made->insert(ins.get());
    out.push_back(std::move(ins));
    return out.back().get();
  };
  std::map<const Instr*, Instr*> memory_of;   // logical value -> an instruction whose row-major array is its memory image
  // the memory image of `x` as a row-major value; appended to `out` when it has to be computed
  auto image = [&](Instr* x, const std::string& base) -> Instr* {
    auto it = order.find(x);
    if (it == order.end() || is_descending(it->second)) return x;
    auto mo = memory_of.find(x);
    if (mo != memory_of.end()) return mo->second;
    const auto p = major_to_minor(it->second);
    return memory_of[x] = make(base, "transpose", permuted(x->shape.dims, p), p, x);
  };
  Instr* old_root = comp->root;
  for (auto& up : old) {
    Instr* ins = up.get();
    auto it = order.find(ins);
    const bool plain = it == order.end() || is_descending(it->second);
    const std::vector<int64_t> p = plain ? std::vector<int64_t>() : major_to_minor(it->second);
    if (comp->is_entry && ins == old_root) {
      // results leave as memory images
      if (ins->opcode == "tuple") {
        for (size_t i = 0; i < ins->operands.size(); ++i) {
          Instr* x = ins->operands[i];
          Instr* y = image(x, x->name + "_memory");
          if (y == x) continue;
          unlink_user(x, ins);   // every position that holds x gets the same image
          ins->operands[i] = y;
          if (std::find(y->users.begin(), y->users.end(), ins) == y->users.end()) y->users.push_back(ins);
          ins->shape.tuple[i].dims = y->shape.dims;
        }
      }
    }
    if (ins->opcode == "bitcast") {
      Instr* x = ins->operands[0];
      Instr* in = image(x, ins->name + "_operand_memory");
      if (in != x) {
        unlink_user(x, ins);
        ins->operands[0] = in;
        in->users.push_back(ins);
      }
      if (!plain) {
        // the instruction keeps its name and its users and becomes the way back from the new bitcast's row-major
        // array to logical order
        Instr* raw = make(ins->name + "_memory", "bitcast", permuted(ins->shape.dims, p), {}, in);
        unlink_user(in, ins);
        ins->opcode = "transpose";
        ins->operands = {raw};
        raw->users.push_back(ins);
        ins->dimensions = inverse_permutation(p);
        memory_of[ins] = raw;
        made->insert(ins);
      }
      out.push_back(std::move(up));
      continue;
    }
    const bool buffer = (ins->opcode == "parameter" && comp->is_entry) || (ins->opcode == "constant" && ins->literal_elided);
    out.push_back(std::move(up));
    if (buffer && !plain) {
      // the host hands over the memory image: that is what this instruction now is, and its users read the
      // transpose back to logical order
      const std::vector<int64_t> logical = ins->shape.dims;
      std::vector<Instr*> users = ins->users;
      ins->users.clear();
      ins->shape.dims = permuted(logical, p);
      Instr* t = make(ins->name + "_logical", "transpose", logical, inverse_permutation(p), ins);
      for (Instr* u : users) {
        for (auto& o : u->operands)
          if (o == ins) o = t;
        t->users.push_back(u);
      }
      order[t] = it->second;
      memory_of[t] = ins;
      order.erase(ins);
    }
  }
  if (comp->is_entry && old_root->opcode != "tuple") {
    Instr* y = image(old_root, old_root->name + "_memory");
    if (y != old_root) {
      old_root->is_root = false;
      y->is_root = true;
      comp->root = y;
    }
  }
  comp->instrs = std::move(out);
  renumber(comp);
}

void erase_instr(Computation* comp, Instr* dead) {
  for (Instr* o : dead->operands) unlink_user(o, dead);
  auto& v = comp->instrs;
  v.erase(std::remove_if(v.begin(), v.end(), [&](const std::unique_ptr<Instr>& u) { return u.get() == dead; }), v.end());
}

// The transposes above next to a GEMM go into the call itself, as the reference's GEMM takes either order of each
// operand and a column-major result by exchanging the operands (gemm_impl.cc:345-351, :408-469):
//   gemm(transpose(X), B) = gemm(X, B) contracting X's other minor dimension (same for the right operand);
//   transpose(gemm(A, B)) = gemm(B, A) with the roles of the contracting and batch dimensions exchanged, taken only
//   when that leaves the new left operand contiguous along k (the order the MFMA tiles read).
void fold_layout_transposes_into_gemms(Computation* comp, std::set<const Instr*>* made) {
  for (auto& up : comp->instrs) {
    Instr* g = up.get();
    if (!g->is_gemm() || g->operands.size() < 2) continue;
    const int r = g->shape.rank();
    for (int side = 0; side < 2; ++side) {
      Instr* t = g->operands[side];
      if (!made->count(t) || !swaps_minor_pair(t) || t->shape.rank() != r) continue;
      Instr* x = t->operands[0];
      unlink_user(t, g);
      g->operands[side] = x;
      x->users.push_back(g);
      if (g->operands[0] == t || g->operands[1] == t) t->users.push_back(g);   // still read by the other side
      int& c = side == 0 ? g->gemm.lhs_contracting : g->gemm.rhs_contracting;
      c = c == r - 1 ? r - 2 : (c == r - 2 ? r - 1 : c);
    }
  }
  for (auto& up : comp->instrs) {
    Instr* t = up.get();
    if (!made->count(t) || !swaps_minor_pair(t)) continue;
    Instr* g = t->operands[0];
    const int r = g->shape.rank();
    if (!g->is_gemm() || g->operands.size() != 2 || g->users.size() != 1 || g == comp->root || g->gemm.rhs_contracting != r - 1) continue;
    Instr *a = g->operands[0], *b = g->operands[1];
    unlink_user(g, t);
    unlink_user(a, g);
    unlink_user(b, g);
    g->operands.clear();
    t->opcode = g->opcode;
    t->custom_call_target = g->custom_call_target;
    t->attrs = g->attrs;
    t->dimensions.clear();
    t->gemm = g->gemm;
    std::swap(t->gemm.lhs_contracting, t->gemm.rhs_contracting);
    std::swap(t->gemm.lhs_batch, t->gemm.rhs_batch);
    std::swap(t->gemm.lhs_stride, t->gemm.rhs_stride);
    t->operands = {b, a};
    b->users.push_back(t);
    a->users.push_back(t);
    made->erase(t);
  }
  // what the rewrites left without a reader
  for (bool again = true; again;) {
    again = false;
    for (auto& up : comp->instrs) {
      Instr* d = up.get();
      const bool candidate = made->count(d) || (d->is_gemm() && d->operands.empty());
      if (!candidate || !d->users.empty() || d == comp->root) continue;
      made->erase(d);
      erase_instr(comp, d);
      again = true;
      break;
    }
  }
  renumber(comp);
}

}  // namespace

// The epilogue of a __cublas$lt$matmul call (bias vector, ReLU, tanh-GELU) becomes what the older dialect writes for
// it: a kLoop fusion behind the call, computed in f32 and rounded to the result type.  The GEMM-epilogue fusion of the
// compiler then runs it on the accumulator tile like any other element-wise consumer of a GEMM.
void lower_lt_matmul_epilogues(Module* mod) {
  int serial = 0;
  for (size_t ci = 0; ci < mod->computations.size(); ++ci) {
    Computation* comp = mod->computations[ci].get();
    for (size_t at = 0; at < comp->instrs.size(); ++at) {
      Instr* call = comp->instrs[at].get();
      if (call->opcode != "custom-call" || call->custom_call_target != "__cublas$lt$matmul" || call->gemm.epilogue == "DEFAULT") continue;
      const std::string ep = call->gemm.epilogue;
      const bool has_bias = ep.rfind("BIAS", 0) == 0;
      const bool relu = ep.find("RELU") != std::string::npos, gelu = ep.find("GELU") != std::string::npos;
      Instr* bias = nullptr;
      if (has_bias) {
        bias = call->operands.back();
        MONONN_CHECK(bias->shape.rank() == 1 && !call->shape.dims.empty() && bias->shape.dims[0] == call->shape.dims.back(), kInvalidArgument)
            << call->hlo_name << ": the bias of __cublas$lt$matmul must be a vector with one value per result column";
        unlink_user(bias, call);
        call->operands.pop_back();
      }
      MONONN_CHECK(is_float(call->shape.dtype), kUnsupported) << call->hlo_name << ": epilogue on a non-float result";
      auto body = std::make_unique<Computation>();
      body->hlo_name = body->name = "lt_matmul_epilogue_" + std::to_string(serial++);
      while (mod->by_name.count(body->name)) body->hlo_name = body->name = "lt_matmul_epilogue_" + std::to_string(serial++);
      Computation* bc = body.get();
      int counter = 0;
      auto add = [&](const char* opcode, DType t, const std::vector<int64_t>& dims, std::vector<Instr*> operands) {
        auto ins = std::make_unique<Instr>();
        ins->hlo_name = ins->name = std::string(opcode == std::string("parameter") ? "param_" : "lt_") + std::to_string(counter++);
        ins->opcode = opcode;
        ins->shape.dtype = t;
        ins->shape.dims = dims;
        for (int i = static_cast<int>(dims.size()) - 1; i >= 0; --i) ins->shape.minor_to_major.push_back(i);
        ins->operands = std::move(operands);
        for (auto* o : ins->operands) o->users.push_back(ins.get());
        ins->parent = bc;
        ins->index_in_comp = static_cast<int>(bc->instrs.size());
        bc->instrs.push_back(std::move(ins));
        return bc->instrs.back().get();
      };
      const std::vector<int64_t>& dims = call->shape.dims;
      const DType rt = call->shape.dtype;
      Instr* p0 = add("parameter", rt, dims, {});
      p0->parameter_number = 0;
      bc->params.push_back(p0);
      Instr* p1 = nullptr;
      if (has_bias) {
        p1 = add("parameter", bias->shape.dtype, bias->shape.dims, {});
        p1->parameter_number = 1;
        bc->params.push_back(p1);
      }
      auto constant = [&](const char* text) {
        Instr* c = add("constant", DType::kF32, {}, {});
        c->literal = text;
        Instr* b = add("broadcast", DType::kF32, dims, {c});
        return b;
      };
      auto f32 = [&](Instr* v) { return v->shape.dtype == DType::kF32 ? v : add("convert", DType::kF32, v->shape.dims, {v}); };
      Instr* x = f32(p0);
      if (has_bias) {
        Instr* b = add("broadcast", DType::kF32, dims, {f32(p1)});
        b->dimensions = {static_cast<int64_t>(dims.size()) - 1};
        x = add("add", DType::kF32, dims, {x, b});
      }
      if (relu) x = add("maximum", DType::kF32, dims, {x, constant("0")});
      if (gelu) {
        // 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3)))
        Instr* x3 = add("multiply", DType::kF32, dims, {add("multiply", DType::kF32, dims, {x, x}), x});
        Instr* inner = add("add", DType::kF32, dims, {x, add("multiply", DType::kF32, dims, {constant("0.044715"), x3})});
        Instr* t = add("tanh", DType::kF32, dims, {add("multiply", DType::kF32, dims, {constant("0.7978845608028654"), inner})});
        x = add("multiply", DType::kF32, dims, {add("multiply", DType::kF32, dims, {constant("0.5"), x}), add("add", DType::kF32, dims, {constant("1"), t})});
      }
      if (rt != DType::kF32) x = add("convert", rt, dims, {x});
      x->is_root = true;
      bc->root = x;
      // the fusion takes the call's place for every user
      auto fus = std::make_unique<Instr>();
      Instr* f = fus.get();
      f->hlo_name = f->name = call->name + "_epilogue";
      f->opcode = "fusion";
      f->fusion_kind = "kLoop";
      f->called = bc;
      f->shape = call->shape;
      f->parent = comp;
      std::vector<Instr*> users = call->users;
      call->users.clear();
      for (Instr* u : users)
        for (auto& o : u->operands)
          if (o == call) {
            o = f;
            if (std::find(f->users.begin(), f->users.end(), u) == f->users.end()) f->users.push_back(u);
          }
      f->operands = {call};
      call->users.push_back(f);
      if (has_bias) {
        f->operands.push_back(bias);
        bias->users.push_back(f);
      }
      if (comp->root == call) {
        comp->root = f;
        f->is_root = true;
        call->is_root = false;
      }
      comp->instrs.insert(comp->instrs.begin() + static_cast<long>(at) + 1, std::move(fus));
      for (size_t i = 0; i < comp->instrs.size(); ++i) comp->instrs[i]->index_in_comp = static_cast<int>(i);
      mod->by_name[bc->name] = bc;
      mod->computations.push_back(std::move(body));
      comp = mod->computations[ci].get();
    }
  }
}

std::unique_ptr<Module> parse_module(const std::string& text) {
  auto mod = std::make_unique<Module>();
  Lexer lx(text);
  if (!lx.consume_word("HloModule")) lx.fail("expected 'HloModule'");
  {
    std::string n = lx.ident();
    mod->name = n;
    // skip the rest of the header line (module attributes)
    while (lx.pos < text.size() && text[lx.pos] != '\n') ++lx.pos;
  }
  struct Pending {
    Instr* ins;
    std::vector<std::string> operand_names;
    int line;
  };
  while (!lx.eof()) {
    auto comp = std::make_unique<Computation>();
    comp->is_entry = lx.consume_word("ENTRY");
    comp->hlo_name = lx.ident();
    comp->name = canonical_name(comp->hlo_name);
    // optional signature "(p: f32[..]) -> f32[..]"
    if (lx.peek() == '(') {
      lx.balanced();
      lx.skip_ws();
      if (text.compare(lx.pos, 2, "->") == 0) {
        lx.pos += 2;
        parse_shape(lx);
      }
    }
    lx.expect('{');
    std::map<std::string, Instr*> local;
    std::vector<Pending> pend;
    while (lx.peek() != '}') {
      if (lx.eof()) lx.fail("unterminated computation");
      auto ins = std::make_unique<Instr>();
      ins->parent = comp.get();
      ins->is_root = lx.consume_word("ROOT");
      ins->hlo_name = lx.ident();
      ins->name = canonical_name(ins->hlo_name);
      lx.expect('=');
      ins->shape = parse_shape(lx);
      ins->opcode = lx.ident();
      int line = lx.line;
      if (!known_opcodes().count(ins->opcode))
        MONONN_FAIL(kUnsupported) << "line " << line << ": opcode '" << ins->opcode << "' is not supported";
      std::string body = lx.balanced();
      body = body.substr(1, body.size() - 2);
      Pending p{ins.get(), {}, line};
      if (ins->opcode == "parameter") {
        ins->parameter_number = std::strtoll(body.c_str(), nullptr, 10);
      } else if (ins->opcode == "constant") {
        ins->literal = body;
        std::string squeezed;
        for (char c : body)
          if (!isspace(static_cast<unsigned char>(c))) squeezed.push_back(c);
        ins->literal_elided = squeezed == "{...}";
      } else {
        // operands: "[shape] %name" separated by top-level commas
        Lexer ol(body);
        while (!ol.eof()) {
          // skip an optional shape prefix: anything before the final identifier of this operand
          size_t start = ol.pos;
          int depth = 0;
          size_t i = start;
          for (; i < body.size(); ++i) {
            char c = body[i];
            if (c == '(' || c == '{' || c == '[') ++depth;
            else if (c == ')' || c == '}' || c == ']') --depth;
            else if (c == ',' && depth == 0) break;
          }
          std::string piece = body.substr(start, i - start);
          while (!piece.empty() && isspace(static_cast<unsigned char>(piece.back()))) piece.pop_back();
          size_t sp = piece.find_last_of(" \t");
          std::string nm = sp == std::string::npos ? piece : piece.substr(sp + 1);
          size_t lead = nm.find_first_not_of(" \t\n");
          nm = lead == std::string::npos ? "" : nm.substr(lead);
          if (nm.empty()) MONONN_FAIL(kParseError) << "line " << line << ": empty operand";
          p.operand_names.push_back(canonical_name(nm));
          ol.pos = i < body.size() ? i + 1 : body.size();
        }
      }
      // attributes
      while (lx.consume(',')) {
        std::string key = lx.ident();
        lx.expect('=');
        ins->attrs[key] = lx.attr_value();
      }
      ins->index_in_comp = static_cast<int>(comp->instrs.size());
      MONONN_CHECK(!local.count(ins->name), kParseError) << "line " << line << ": duplicate instruction name " << ins->hlo_name;
      local[ins->name] = ins.get();
      if (ins->is_root) comp->root = ins.get();
      pend.push_back(std::move(p));
      comp->instrs.push_back(std::move(ins));
    }
    lx.expect('}');
    MONONN_CHECK(!comp->instrs.empty(), kParseError) << "computation " << comp->hlo_name << " is empty";
    if (!comp->root) comp->root = comp->instrs.back().get();
    for (auto& p : pend) {
      for (auto& on : p.operand_names) {
        auto it = local.find(on);
        MONONN_CHECK(it != local.end(), kParseError) << "line " << p.line << ": operand '" << on << "' of " << p.ins->hlo_name << " is not defined";
        MONONN_CHECK(it->second->index_in_comp < p.ins->index_in_comp, kParseError) << "line " << p.line << ": operand '" << on << "' is used before its definition";
        p.ins->operands.push_back(it->second);
        it->second->users.push_back(p.ins);
      }
      decode_attrs(p.ins, mod.get());
      if (p.ins->opcode == "parameter") {
        MONONN_CHECK(p.ins->parameter_number >= 0, kParseError) << "bad parameter number for " << p.ins->hlo_name;
        if (comp->params.size() <= static_cast<size_t>(p.ins->parameter_number)) comp->params.resize(p.ins->parameter_number + 1, nullptr);
        comp->params[p.ins->parameter_number] = p.ins;
      }
    }
    for (auto* pp : comp->params) MONONN_CHECK(pp != nullptr, kParseError) << "computation " << comp->hlo_name << " has a gap in its parameter numbers";
    MONONN_CHECK(!mod->by_name.count(comp->name), kParseError) << "duplicate computation " << comp->hlo_name;
    mod->by_name[comp->name] = comp.get();
    if (comp->is_entry) {
      MONONN_CHECK(mod->entry == nullptr, kParseError) << "more than one ENTRY computation";
      mod->entry = comp.get();
    }
    mod->computations.push_back(std::move(comp));
  }
  MONONN_CHECK(mod->entry != nullptr, kParseError) << "module has no ENTRY computation";
  lower_lt_matmul_epilogues(mod.get());
  std::set<const Instr*> layout_transposes;
  for (auto& comp : mod->computations) {
    normalize_layouts(comp.get(), &layout_transposes);
    if (!layout_transposes.empty()) fold_layout_transposes_into_gemms(comp.get(), &layout_transposes);
  }
  return mod;
}

}  // namespace hlo
}  // namespace mononn
