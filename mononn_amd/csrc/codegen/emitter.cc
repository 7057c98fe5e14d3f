#include "codegen/emitter.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <sstream>

#include "common/status.h"

namespace mononn {
namespace codegen {

using hlo::DType;
using hlo::Instr;

// ------------------------------------------------------------------------------------------
void CodeBuffer::line(const std::string& s) {
  text_.append(static_cast<size_t>(indent_) * 2, ' ');
  text_ += s;
  text_.push_back('\n');
}
void CodeBuffer::open(const std::string& header) {
  line(header + " {");
  ++indent_;
}
void CodeBuffer::close(const std::string& tail) {
  --indent_;
  line("}" + tail);
}

std::string PointerTable::input(const Instr* root, DType as) {
  for (auto& e : entries)
    if (e.root == root && !e.is_output) return e.name;
  int n = 0;
  for (auto& e : entries) n += e.is_output ? 0 : 1;
  entries.push_back({root, false, "in" + std::to_string(n), as == DType::kInvalid ? root->shape.dtype : as});
  return entries.back().name;
}
std::string PointerTable::output(const Instr* root, DType as) {
  for (auto& e : entries)
    if (e.root == root && e.is_output) return e.name;
  int n = 0;
  for (auto& e : entries) n += e.is_output ? 1 : 0;
  entries.push_back({root, true, "out" + std::to_string(n), as == DType::kInvalid ? root->shape.dtype : as});
  return entries.back().name;
}

LinExpr physical_offset(const graph::Program& prog, const Instr* root, const Index& idx, const VarTable* vars) {
  auto tile = prog.physical_tile.find(root);
  if (tile != prog.physical_tile.end()) {
    MONONN_CHECK(vars != nullptr, kInternal) << root->hlo_name << ": fragment-order buffer addressed without a variable table";
    Index pi = idx;
    std::vector<int64_t> pd = root->shape.dims;
    auto perm = prog.physical_perm.find(root);
    if (perm != prog.physical_perm.end()) {
      pi.clear();
      pd.clear();
      for (int d : perm->second) {
        pi.push_back(idx[d]);
        pd.push_back(root->shape.dims[d]);
      }
    }
    const int64_t K = tile->second.k, R = root->shape.num_elements() / K;
    if (tile->second.order == graph::Program::TileOrder::kRunsOf8) {
      Index d = delinearize(linearize(pi, pd), {R / 16, 16, K / 32, 4, 8}, *vars);
      return linearize({d[0], d[2], d[3], d[1], d[4]}, {R / 16, K / 32, 4, 16, 8});
    }
    // k % 32 = 16 * half + 4 * g + e  ->  lane group g, element 4 * half + e
    Index d = delinearize(linearize(pi, pd), {R / 16, 16, K / 32, 2, 4, 4}, *vars);
    return linearize({d[0], d[2], d[4], d[1], d[3], d[5]}, {R / 16, K / 32, 4, 16, 2, 4});
  }
  auto it = prog.physical_perm.find(root);
  if (it == prog.physical_perm.end()) return linearize(idx, root->shape.dims);
  Index pi;
  std::vector<int64_t> pd;
  for (int d : it->second) {
    pi.push_back(idx[d]);
    pd.push_back(root->shape.dims[d]);
  }
  return linearize(pi, pd);
}

// ------------------------------------------------------------------------------------------
Emitter::Emitter(const graph::Program& prog, const std::vector<const Instr*>& members, CodeBuffer& out,
                 VarTable& vars, PointerTable& ptrs)
    : prog_(prog), member_order_(members), out_(out), vars_(vars), ptrs_(ptrs) {
  for (auto* m : members) {
    members_.insert(m);
    if (m->opcode == "fusion") caller_[m->called] = m;
  }
  scopes_.emplace_back();
}

void Emitter::push_scope() { scopes_.emplace_back(); }
void Emitter::pop_scope() { scopes_.pop_back(); }
std::string Emitter::fresh(const std::string& prefix) { return prefix + std::to_string(counter_++); }

void Emitter::bind(const Instr* ins, const Index& idx, const std::string& expr) { bound_[ins] = {idx, expr}; }
void Emitter::unbind(const Instr* ins) { bound_.erase(ins); }

std::string Emitter::key(const Instr* ins, const Index& idx) const {
  char buf[32];
  std::snprintf(buf, sizeof buf, "%p", static_cast<const void*>(ins));
  std::string k = buf;
  for (auto& e : idx) k += "|" + e.str(vars_);
  return k;
}

std::string Emitter::def(DType t, const std::string& rhs) {
  // Value numbering: every definition is a pure function of the variables named in `rhs` (inputs of
  // a node are never written by it), so an identical right-hand side already in scope is the same
  // value.  This merges the copies of a sub-expression that XLA duplicated into several fusions
  // (the soft-max logits, the centred LayerNorm input) once those fusions share a loop body.
  std::string k = std::string("=") + hlo::dtype_ctype(t) + "|" + rhs;
  for (auto it = scopes_.rbegin(); it != scopes_.rend(); ++it) {
    auto f = it->find(k);
    if (f != it->end()) return f->second;
  }
  std::string v = fresh();
  out_.line(std::string("const ") + hlo::dtype_ctype(t) + " " + v + " = " + rhs + ";");
  scopes_.back()[k] = v;
  return v;
}

const Instr* Emitter::resolve_output(const Instr* v) const {
  if (v->opcode == "get-tuple-element") {
    const Instr* f = v->operands[0];
    MONONN_CHECK(f->opcode == "fusion" && f->called->root->opcode == "tuple", kUnsupported)
        << v->hlo_name << ": get-tuple-element of something other than a multi-output fusion";
    return f->called->root->operands[v->tuple_index];
  }
  if (v->opcode == "fusion") return v->called->root;
  return v;
}

std::vector<const Instr*> Emitter::collect_reduces() const {
  std::vector<const Instr*> out;
  for (auto* m : member_order_) {
    if (m->opcode == "fusion") {
      for (auto& i : m->called->instrs)
        if (i->opcode == "reduce") out.push_back(i.get());
    } else if (m->opcode == "reduce") {
      out.push_back(m);
    }
  }
  return out;
}

std::string Emitter::literal_of(DType t, const std::string& text_in) {
  std::string text;
  for (char c : text_in)
    if (!isspace(static_cast<unsigned char>(c))) text.push_back(c);
  if (t == DType::kPred) return (text == "true" || text == "1") ? "true" : "false";
  if (hlo::is_float(t)) {
    std::string body;
    if (text == "inf" || text == "+inf") body = "__builtin_inff()";
    else if (text == "-inf") body = "(-__builtin_inff())";
    else if (text == "nan" || text == "-nan") body = "__builtin_nanf(\"\")";
    else {
      char* end = nullptr;
      double v = std::strtod(text.c_str(), &end);
      MONONN_CHECK(end && *end == 0 && !text.empty(), kParseError) << "bad floating literal '" << text_in << "'";
      char buf[64];
      if (t == DType::kF64) {
        std::snprintf(buf, sizeof buf, "%.17g", v);
        body = buf;
        if (body.find_first_of(".e") == std::string::npos && body.find("inf") == std::string::npos) body += ".0";
        return "(" + body + ")";
      }
      float f = static_cast<float>(v);
      if (std::isinf(f)) body = f > 0 ? "__builtin_inff()" : "(-__builtin_inff())";
      else {
        std::snprintf(buf, sizeof buf, "%.9g", static_cast<double>(f));
        body = buf;
        if (body.find_first_of(".e") == std::string::npos) body += ".0";
        body += "f";
      }
    }
    if (t == DType::kF16) return "((_Float16)" + body + ")";
    if (t == DType::kBF16) return "((__bf16)" + body + ")";
    if (t == DType::kF64) return "((double)" + body + ")";
    return "(" + body + ")";
  }
  char* end = nullptr;
  long long v = std::strtoll(text.c_str(), &end, 10);
  MONONN_CHECK(end && *end == 0 && !text.empty(), kParseError) << "bad integer literal '" << text_in << "'";
  std::string s = std::to_string(v);
  if (t == DType::kS64 || t == DType::kU64) s += "ll";
  return std::string("((") + hlo::dtype_ctype(t) + ")" + s + ")";
}

std::string Emitter::literal(const Instr* c) { return literal_of(c->shape.dtype, c->literal); }

std::string Emitter::reducer_expr(const Instr* reduce, const std::string& a, const std::string& b) {
  const hlo::Computation* c = reduce->called;
  MONONN_CHECK(c != nullptr, kInternal) << reduce->hlo_name << ": reduce without reducer";
  const Instr* r = c->root;
  // a scalar binary computation over its two parameters (add / maximum / minimum / multiply / and / or),
  // the shapes produced for soft-max and LayerNorm (reduction_functor_generator.cc:224-294)
  bool direct = r->operands.size() == 2 && r->operands[0]->opcode == "parameter" && r->operands[1]->opcode == "parameter";
  MONONN_CHECK(direct, kUnsupported) << reduce->hlo_name << ": reducer computation '" << c->hlo_name
                                     << "' is not a single binary op over its parameters";
  DType t = r->shape.dtype;
  const std::string& op = r->opcode;
  if (op == "add") return "(" + a + " + " + b + ")";
  if (op == "multiply") return "(" + a + " * " + b + ")";
  if (op == "maximum") return t == DType::kF32 ? "fmaxf(" + a + ", " + b + ")" : "((" + a + ") > (" + b + ") ? (" + a + ") : (" + b + "))";
  if (op == "minimum") return t == DType::kF32 ? "fminf(" + a + ", " + b + ")" : "((" + a + ") < (" + b + ") ? (" + a + ") : (" + b + "))";
  if (op == "and") return t == DType::kPred ? "(" + a + " && " + b + ")" : "(" + a + " & " + b + ")";
  if (op == "or") return t == DType::kPred ? "(" + a + " || " + b + ")" : "(" + a + " | " + b + ")";
  MONONN_FAIL(kUnsupported) << reduce->hlo_name << ": reducer op '" << op << "' is not supported";
}

std::string Emitter::reducer_functor(const Instr* reduce) {
  std::string t = hlo::dtype_ctype(reduce->called->root->shape.dtype);
  return "[](" + t + " x, " + t + " y) { return (" + t + ")" + reducer_expr(reduce, "x", "y") + "; }";
}

// ------------------------------------------------------------------------------------------
std::string Emitter::value(const Instr* ins, const Index& idx) {
  MONONN_CHECK(static_cast<int>(idx.size()) == ins->shape.rank(), kInternal)
      << "index rank " << idx.size() << " does not match " << ins->hlo_name << " " << ins->shape.to_string();
  auto b = bound_.find(ins);
  if (b != bound_.end()) {
    LinExpr want = linearize(b->second.idx, ins->shape.dims);
    LinExpr got = linearize(idx, ins->shape.dims);
    if (want.equals(got)) return b->second.expr;
    MONONN_FAIL(kUnsupported) << ins->hlo_name << ": on-chip value requested at index [" << got.str(vars_)
                              << "], available at [" << want.str(vars_) << "]";
  }
  std::string k = key(ins, idx);
  for (auto it = scopes_.rbegin(); it != scopes_.rend(); ++it) {
    auto f = it->find(k);
    if (f != it->end()) return f->second;
  }
  std::string v = emit(ins, idx);
  scopes_.back()[k] = v;
  return v;
}

std::string Emitter::load(const Instr* root, const Index& idx) {
  LinExpr lin = physical_offset(prog_, root, idx, &vars_);
  auto sk = prog_.split_k.find(root);
  if (sk != prog_.split_k.end()) {
    // split-K GEMM result: S fp32 partial sums, added in a fixed order, then rounded to the f16 value
    // the HLO defines
    std::string p = ptrs_.input(root, DType::kF32);
    const int64_t E = root->shape.num_elements();
    // every partial sum is a definition of its own, so that all of them can be requested before the first add
    std::string sum;
    for (int i = 0; i < sk->second; ++i) {
      std::string ref = p + "[" + lin.plus_const(i * E).str(vars_) + "]";
      if (lin.opaques().empty() && guarded_ == 0) simple_loads_.emplace_back(ref, "float");
      sum += (i ? " + " : "") + def(DType::kF32, ref);
    }
    return def(root->shape.dtype, "(" + std::string(hlo::dtype_ctype(root->shape.dtype)) + ")(" + sum + ")");
  }
  std::string ref = ptrs_.input(root) + "[" + lin.str(vars_) + "]";
  if (lin.opaques().empty() && guarded_ == 0) simple_loads_.emplace_back(ref, hlo::dtype_ctype(root->shape.dtype));
  return def(root->shape.dtype, ref);
}

std::string Emitter::serial_reduce(const Instr* ins, const Index& idx) {
  MONONN_CHECK(ins->operands.size() == 2 && ins->dimensions.size() == 1, kUnsupported)
      << ins->hlo_name << ": only single-operand reductions over one dimension are supported";
  const Instr* x = ins->operands[0];
  int d = static_cast<int>(ins->dimensions[0]);
  int64_t R = x->shape.dims[d];
  std::string t = hlo::dtype_ctype(ins->shape.dtype);
  std::string init = value(ins->operands[1], {});
  std::string acc = fresh("acc");
  std::string rk = fresh("rk");
  out_.line(t + " " + acc + " = " + init + ";");
  int var = vars_.add(rk, R);
  out_.open("for (int " + rk + " = 0; " + rk + " < " + std::to_string(R) + "; ++" + rk + ")");
  ++guarded_;
  push_scope();
  Index xi;
  for (int i = 0, j = 0; i < x->shape.rank(); ++i) {
    if (i == d) xi.push_back(LinExpr::variable(var, R));
    else xi.push_back(idx[j++]);
  }
  std::string v = value(x, xi);
  out_.line(acc + " = (" + t + ")" + reducer_expr(ins, acc, v) + ";");
  pop_scope();
  --guarded_;
  out_.close();
  return acc;
}

std::vector<std::string> Emitter::inline_scalar_computation(const hlo::Computation* c, const std::vector<std::string>& args) {
  MONONN_CHECK(c->params.size() == args.size(), kUnsupported) << "computation " << c->hlo_name << " takes " << c->params.size() << " parameters, " << args.size() << " given";
  for (auto* p : c->params) MONONN_CHECK(p->shape.rank() == 0, kUnsupported) << c->hlo_name << ": reducer parameters must be scalars";
  push_scope();
  for (size_t i = 0; i < args.size(); ++i) bind(c->params[i], {}, args[i]);
  std::vector<std::string> out;
  if (c->root->opcode == "tuple") {
    for (auto* o : c->root->operands) out.push_back(value(o, {}));
  } else {
    out.push_back(value(c->root, {}));
  }
  for (auto* p : c->params) unbind(p);
  pop_scope();
  return out;
}

// (value, index) reductions and their like (ir_parser_fused.cc:1169-1213, tuple functors of
// reduction_functor_generator.cc:246-283): the elements are combined in ascending order by the thread that owns
// the output element.
std::vector<std::string> Emitter::serial_reduce_variadic(const Instr* ins, const Index& idx) {
  const size_t n = ins->operands.size() / 2;
  MONONN_CHECK(n >= 1 && ins->operands.size() == 2 * n && ins->dimensions.size() == 1 && ins->shape.is_tuple() && ins->shape.tuple.size() == n, kUnsupported)
      << ins->hlo_name << ": a variadic reduce takes N operands, N init values and yields an N-tuple over one reduced dimension";
  const std::string k = "variadic:" + key(ins, idx);
  for (auto it = scopes_.rbegin(); it != scopes_.rend(); ++it) {
    auto f = it->find(k);
    if (f == it->end()) continue;
    std::vector<std::string> cached;
    std::istringstream is(f->second);
    std::string name;
    while (is >> name) cached.push_back(name);
    return cached;
  }
  const Instr* x0 = ins->operands[0];
  const int d = static_cast<int>(ins->dimensions[0]);
  const int64_t R = x0->shape.dims[d];
  std::vector<std::string> acc, types;
  for (size_t i = 0; i < n; ++i) {
    MONONN_CHECK(ins->operands[i]->shape.dims == x0->shape.dims, kUnsupported) << ins->hlo_name << ": operands of different shapes";
    types.push_back(hlo::dtype_ctype(ins->shape.tuple[i].dtype));
    acc.push_back(fresh("acc"));
    out_.line(types[i] + " " + acc[i] + " = " + value(ins->operands[n + i], {}) + ";");
  }
  std::string rk = fresh("rk");
  int var = vars_.add(rk, R);
  out_.open("for (int " + rk + " = 0; " + rk + " < " + std::to_string(R) + "; ++" + rk + ")");
  ++guarded_;
  push_scope();
  Index xi;
  for (int i = 0, j = 0; i < x0->shape.rank(); ++i) {
    if (i == d) xi.push_back(LinExpr::variable(var, R));
    else xi.push_back(idx[j++]);
  }
  std::vector<std::string> args = acc;
  for (size_t i = 0; i < n; ++i) args.push_back(value(ins->operands[i], xi));
  std::vector<std::string> res = inline_scalar_computation(ins->called, args);
  MONONN_CHECK(res.size() == n, kUnsupported) << ins->hlo_name << ": the reducer yields " << res.size() << " values for " << n << " operands";
  // all results are taken before any accumulator changes (a reducer may pass an accumulator through to another slot)
  std::vector<std::string> tmp;
  for (size_t i = 0; i < n; ++i) {
    tmp.push_back(fresh("nx"));
    out_.line("const " + types[i] + " " + tmp[i] + " = (" + types[i] + ")" + res[i] + ";");
  }
  for (size_t i = 0; i < n; ++i) out_.line(acc[i] + " = " + tmp[i] + ";");
  pop_scope();
  --guarded_;
  out_.close();
  std::string joined;
  for (auto& a : acc) joined += a + " ";
  scopes_.back()[k] = joined;
  return acc;
}

std::string Emitter::emit(const Instr* ins, const Index& idx) {
  const std::string& op = ins->opcode;
  const DType dt = ins->shape.dtype;
  const std::string T = hlo::dtype_ctype(dt);
  const bool entry = ins->parent->is_entry;

  if (op == "parameter") {
    if (entry) return load(ins, idx);
    auto c = caller_.find(ins->parent);
    MONONN_CHECK(c != caller_.end(), kInternal) << "fused computation " << ins->parent->hlo_name << " has no caller in this cluster";
    return value(c->second->operands[ins->parameter_number], idx);
  }
  if (op == "constant") {
    if (ins->is_scalar_constant()) return literal(ins);
    if (entry) return load(ins, idx);
    MONONN_CHECK(!ins->literal_elided, kUnsupported) << ins->hlo_name << ": elided constant inside a fused computation";
    // small literal table inside a fused computation -> device-global array named by content
    std::string flat;
    {
      std::string tok;
      std::vector<std::string> vals;
      for (char ch : ins->literal + ",") {
        if (ch == '{' || ch == '}' || ch == ',' || isspace(static_cast<unsigned char>(ch))) {
          if (!tok.empty()) vals.push_back(literal_of(dt, tok));
          tok.clear();
        } else {
          tok.push_back(ch);
        }
      }
      MONONN_CHECK(static_cast<int64_t>(vals.size()) == ins->shape.num_elements(), kParseError)
          << ins->hlo_name << ": literal has " << vals.size() << " elements, shape says " << ins->shape.num_elements();
      for (size_t i = 0; i < vals.size(); ++i) flat += (i ? ", " : "") + vals[i];
    }
    std::string name = "lit_" + std::to_string(std::hash<std::string>{}(T + flat));
    literal_tables_[name] = "__device__ const " + T + " " + name + "[] = {" + flat + "};";
    return def(dt, name + "[" + linearize(idx, ins->shape.dims).str(vars_) + "]");
  }
  if (op == "get-tuple-element" && ins->operands[0]->opcode == "reduce" && (!entry || is_member(ins->operands[0]))) {
    auto all = serial_reduce_variadic(ins->operands[0], idx);
    MONONN_CHECK(ins->tuple_index >= 0 && static_cast<size_t>(ins->tuple_index) < all.size(), kParseError) << ins->hlo_name << ": tuple index out of range";
    return all[ins->tuple_index];
  }
  if (entry && !is_member(ins)) {
    // value produced outside this cluster: follow pure renames, load at the storage root
    if (graph::is_alias_op(ins)) {
      const Instr* x = ins->operands[0];
      return value(x, reshape_index(idx, ins->shape.dims, x->shape.dims, vars_));
    }
    if (op == "get-tuple-element" && is_member(ins->operands[0])) return value(resolve_output(ins), idx);
    MONONN_CHECK(!ins->shape.is_tuple(), kUnsupported) << ins->hlo_name << ": tuple-shaped value read as an array";
    return load(ins, idx);
  }
  if (op == "fusion") {
    MONONN_CHECK(ins->called->root->opcode != "tuple", kUnsupported) << ins->hlo_name << ": multi-output fusion read without get-tuple-element";
    return value(ins->called->root, idx);
  }
  if (op == "get-tuple-element") return value(resolve_output(ins), idx);
  if (op == "copy") return value(ins->operands[0], idx);

  // ---- shape ops --------------------------------------------------------------------------
  if (op == "bitcast" || op == "reshape") {
    const Instr* x = ins->operands[0];
    MONONN_CHECK(x->shape.num_elements() == ins->shape.num_elements(), kUnsupported) << ins->hlo_name << ": element count changes";
    return value(x, reshape_index(idx, ins->shape.dims, x->shape.dims, vars_));
  }
  if (op == "broadcast") {
    const Instr* x = ins->operands[0];
    Index xi;
    for (int i = 0; i < x->shape.rank(); ++i) xi.push_back(idx[ins->dimensions[i]]);
    return value(x, xi);
  }
  if (op == "transpose") {
    const Instr* x = ins->operands[0];
    Index xi(idx.size());
    for (size_t i = 0; i < idx.size(); ++i) xi[ins->dimensions[i]] = idx[i];
    return value(x, xi);
  }
  if (op == "slice") {
    Index xi;
    for (size_t i = 0; i < idx.size(); ++i) xi.push_back(idx[i].plus_const(ins->slice_starts[i]));
    return value(ins->operands[0], xi);
  }
  if (op == "iota") return def(dt, "(" + T + ")(" + idx[ins->iota_dimension].str(vars_) + ")");
  if (op == "concatenate") {
    int d = static_cast<int>(ins->dimensions[0]);
    std::string e = idx[d].str(vars_);
    std::string v = fresh();
    out_.line(T + " " + v + ";");
    int64_t off = 0;
    for (size_t k = 0; k < ins->operands.size(); ++k) {
      const Instr* x = ins->operands[k];
      int64_t n = x->shape.dims[d];
      bool last = k + 1 == ins->operands.size();
      std::string head = (k == 0 ? "if (" : "else if (") + e + " < " + std::to_string(off + n) + ")";
      if (last) head = k == 0 ? "" : "else";
      out_.open(head);
      ++guarded_;
      push_scope();
      Index xi = idx;
      xi[d] = idx[d].plus_const(-off);
      out_.line(v + " = " + value(x, xi) + ";");
      pop_scope();
      --guarded_;
      out_.close();
      off += n;
    }
    return v;
  }
  if (op == "pad") {
    const Instr* x = ins->operands[0];
    std::string padv = value(ins->operands[1], {});
    std::string cond;
    Index xi;
    for (size_t i = 0; i < idx.size(); ++i) {
      int64_t lo = ins->pad_low[i], n = x->shape.dims[i];
      xi.push_back(idx[i].plus_const(-lo));
      if (lo == 0 && ins->pad_high[i] == 0) continue;
      std::string e = "(" + idx[i].str(vars_) + ")";
      cond += (cond.empty() ? "" : " && ") + e + " >= " + std::to_string(lo) + " && " + e + " < " + std::to_string(lo + n);
    }
    if (cond.empty()) return value(x, xi);
    std::string v = fresh();
    out_.line(T + " " + v + " = " + padv + ";");
    out_.open("if (" + cond + ")");
    ++guarded_;
    push_scope();
    out_.line(v + " = " + value(x, xi) + ";");
    pop_scope();
    --guarded_;
    out_.close();
    return v;
  }
  if (op == "gather") {
    // row gather: operand[indices[batch...], offset...] (index_tracer.cc:235-280)
    const Instr* table = ins->operands[0];
    const Instr* indices = ins->operands[1];
    bool row_gather = ins->collapsed_slice_dims == std::vector<int64_t>{0} && ins->start_index_map == std::vector<int64_t>{0} &&
                      ins->index_vector_dim == indices->shape.rank() && ins->slice_sizes.size() == static_cast<size_t>(table->shape.rank()) &&
                      ins->slice_sizes[0] == 1;
    for (int i = 1; row_gather && i < table->shape.rank(); ++i) row_gather = ins->slice_sizes[i] == table->shape.dims[i];
    MONONN_CHECK(row_gather, kUnsupported) << ins->hlo_name << ": only whole-row gathers along dimension 0 are supported";
    int r = indices->shape.rank();
    Index ii(idx.begin(), idx.begin() + r);
    std::string iv = value(indices, ii);
    int64_t rows = table->shape.dims[0];
    std::string clamped = fresh("g");
    out_.line("const int " + clamped + " = mononn_dev::clamp_index(" + iv + ", " + std::to_string(rows - 1) + ");");
    Index ti;
    ti.push_back(LinExpr::opaque(clamped, rows));
    for (size_t i = r; i < idx.size(); ++i) ti.push_back(idx[i]);
    return value(table, ti);
  }
  if (op == "dynamic-slice") {
    const Instr* x = ins->operands[0];
    Index xi;
    for (int i = 0; i < x->shape.rank(); ++i) {
      std::string s = value(ins->operands[1 + i], {});
      int64_t hi = x->shape.dims[i] - ins->dynamic_slice_sizes[i];
      std::string c = fresh("ds");
      out_.line("const int " + c + " = mononn_dev::clamp_index(" + s + ", " + std::to_string(hi) + ");");
      xi.push_back(idx[i].plus(LinExpr::opaque(c, hi + 1)));
    }
    return value(x, xi);
  }
  if (op == "dynamic-update-slice") {
    // the update where the index falls inside it (start indices clamped so that it fits), the operand elsewhere
    const Instr* x = ins->operands[0];
    const Instr* u = ins->operands[1];
    std::string cond;
    Index ui;
    for (int i = 0; i < x->shape.rank(); ++i) {
      const int64_t un = u->shape.dims[i], hi = x->shape.dims[i] - un;
      if (hi == 0) {
        ui.push_back(idx[i]);
        continue;
      }
      std::string s = value(ins->operands[2 + i], {});
      std::string c = fresh("us");
      out_.line("const int " + c + " = (" + idx[i].str(vars_) + ") - mononn_dev::clamp_index(" + s + ", " + std::to_string(hi) + ");");
      cond += (cond.empty() ? "" : " && ") + c + " >= 0 && " + c + " < " + std::to_string(un);
      ui.push_back(LinExpr::opaque(c, un));
    }
    if (cond.empty()) return value(u, ui);
    std::string v = fresh();
    out_.line(T + " " + v + ";");
    out_.open("if (" + cond + ")");
    ++guarded_;
    push_scope();
    out_.line(v + " = " + value(u, ui) + ";");
    pop_scope();
    --guarded_;
    out_.close();
    out_.open("else");
    ++guarded_;
    push_scope();
    out_.line(v + " = " + value(x, idx) + ";");
    pop_scope();
    --guarded_;
    out_.close();
    return v;
  }
  if (op == "reduce-window") {
    // acc = init; for every window position: acc = reducer(acc, inside the operand ? operand : init)
    // (index map of index_tracer.cc's reduce-window: input = output * stride + window offset - low padding)
    const Instr* x = ins->operands[0];
    const int r = x->shape.rank();
    std::string init = value(ins->operands[1], {});
    std::string acc = fresh("acc");
    out_.line(T + " " + acc + " = " + init + ";");
    std::vector<std::string> w(r);
    int opened = 0;
    for (int i = 0; i < r; ++i) {
      if (ins->window_size[i] == 1) continue;
      w[i] = fresh("w");
      out_.open("for (int " + w[i] + " = 0; " + w[i] + " < " + std::to_string(ins->window_size[i]) + "; ++" + w[i] + ")");
      ++guarded_;
      ++opened;
    }
    push_scope();
    std::string cond;
    Index xi;
    for (int i = 0; i < r; ++i) {
      const int64_t lo = ins->window_pad_low[i], hi = ins->window_pad_high[i], st = ins->window_stride[i], n = x->shape.dims[i];
      if (ins->window_size[i] == 1 && st == 1 && lo == 0 && hi == 0) {
        xi.push_back(idx[i]);
        continue;
      }
      std::string p = fresh("p");
      out_.line("const int " + p + " = (" + idx[i].str(vars_) + ") * " + std::to_string(st) + (w[i].empty() ? "" : " + " + w[i]) + " - " + std::to_string(lo) + ";");
      if (lo > 0 || hi > 0) cond += (cond.empty() ? "" : " && ") + p + " >= 0 && " + p + " < " + std::to_string(n);
      xi.push_back(LinExpr::opaque(p, n));
    }
    std::string v;
    if (cond.empty()) {
      v = value(x, xi);
    } else {
      v = fresh();
      out_.line(T + " " + v + " = " + init + ";");
      out_.open("if (" + cond + ")");
      ++guarded_;
      push_scope();
      out_.line(v + " = " + value(x, xi) + ";");
      pop_scope();
      --guarded_;
      out_.close();
    }
    out_.line(acc + " = (" + T + ")" + reducer_expr(ins, acc, v) + ";");
    pop_scope();
    guarded_ -= opened;
    for (int i = 0; i < opened; ++i) out_.close();
    return acc;
  }
  if (op == "reduce") {
    MONONN_CHECK(!ins->shape.is_tuple(), kUnsupported) << ins->hlo_name << ": tuple-valued reduce read without get-tuple-element";
    return serial_reduce(ins, idx);
  }

  // ---- element-wise -----------------------------------------------------------------------
  std::vector<std::string> a;
  for (auto* o : ins->operands) {
    MONONN_CHECK(o->shape.dims == ins->shape.dims || op == "select" || op == "clamp" || op == "compare" || op == "convert", kUnsupported)
        << ins->hlo_name << ": operand shape differs from result shape";
    Index oi = idx;
    if (o->shape.rank() == 0) oi.clear();   // scalar operands of clamp
    a.push_back(value(o, oi));
  }
  auto need = [&](size_t n) { MONONN_CHECK(a.size() == n, kParseError) << ins->hlo_name << ": " << op << " expects " << n << " operands"; };
  const DType st = ins->operands.empty() ? dt : ins->operands[0]->shape.dtype;
  const bool f32 = dt == DType::kF32, f16 = dt == DType::kF16, f64 = dt == DType::kF64;
  auto via_f32 = [&](const std::string& fn) {   // unary math evaluated in fp32
    if (f32) return def(dt, fn + "(" + a[0] + ")");
    if (f16 || dt == DType::kBF16) return def(dt, "(" + T + ")" + fn + "((float)" + a[0] + ")");
    MONONN_FAIL(kUnsupported) << ins->hlo_name << ": " << op << " on " << hlo::dtype_name(dt);
  };
  if (op == "add") { need(2); return def(dt, dt == DType::kPred ? "(" + a[0] + " || " + a[1] + ")" : "(" + T + ")(" + a[0] + " + " + a[1] + ")"); }
  if (op == "subtract") { need(2); return def(dt, "(" + T + ")(" + a[0] + " - " + a[1] + ")"); }
  if (op == "multiply") { need(2); return def(dt, dt == DType::kPred ? "(" + a[0] + " && " + a[1] + ")" : "(" + T + ")(" + a[0] + " * " + a[1] + ")"); }
  if (op == "divide") {
    need(2);
    if (f32 && fast_divide_) return def(dt, "(" + a[0] + " * __builtin_amdgcn_rcpf(" + a[1] + "))");
    return def(dt, "(" + T + ")(" + a[0] + " / " + a[1] + ")");
  }
  if (op == "maximum") { need(2); return def(dt, f32 ? "fmaxf(" + a[0] + ", " + a[1] + ")" : "(" + a[0] + " > " + a[1] + " ? " + a[0] + " : " + a[1] + ")"); }
  if (op == "minimum") { need(2); return def(dt, f32 ? "fminf(" + a[0] + ", " + a[1] + ")" : "(" + a[0] + " < " + a[1] + " ? " + a[0] + " : " + a[1] + ")"); }
  if (op == "power") { need(2); return def(dt, f64 ? "pow(" + a[0] + ", " + a[1] + ")" : "(" + T + ")powf((float)" + a[0] + ", (float)" + a[1] + ")"); }
  if (op == "and") { need(2); return def(dt, dt == DType::kPred ? "(" + a[0] + " && " + a[1] + ")" : "(" + T + ")(" + a[0] + " & " + a[1] + ")"); }
  if (op == "or") { need(2); return def(dt, dt == DType::kPred ? "(" + a[0] + " || " + a[1] + ")" : "(" + T + ")(" + a[0] + " | " + a[1] + ")"); }
  if (op == "not") { need(1); return def(dt, dt == DType::kPred ? "!" + a[0] : "(" + T + ")(~" + a[0] + ")"); }
  if (op == "negate") { need(1); return def(dt, "(" + T + ")(-" + a[0] + ")"); }
  if (op == "abs") { need(1); return def(dt, f32 ? "fabsf(" + a[0] + ")" : "(" + a[0] + " < (" + T + ")0 ? (" + T + ")(-" + a[0] + ") : " + a[0] + ")"); }
  if (op == "sign") { need(1); return def(dt, "mononn_dev::sign_of<" + T + ">(" + a[0] + ")"); }
  if (op == "exponential") { need(1); return f64 ? def(dt, "exp(" + a[0] + ")") : via_f32("__expf"); }
  if (op == "log") { need(1); return f64 ? def(dt, "log(" + a[0] + ")") : via_f32("__logf"); }
  if (op == "tanh") { need(1); return f64 ? def(dt, "tanh(" + a[0] + ")") : via_f32("mononn_dev::fast_tanh"); }
  if (op == "rsqrt") { need(1); return f64 ? def(dt, "(1.0 / sqrt(" + a[0] + "))") : via_f32("rsqrtf"); }
  if (op == "sqrt") { need(1); return f64 ? def(dt, "sqrt(" + a[0] + ")") : via_f32("sqrtf"); }
  if (op == "convert") {
    need(1);
    if (dt == st) return a[0];
    if (dt == DType::kPred) return def(dt, "(" + a[0] + " != (" + std::string(hlo::dtype_ctype(st)) + ")0)");
    return def(dt, "(" + T + ")" + a[0]);
  }
  if (op == "compare") {
    need(2);
    static const std::map<std::string, std::string> ops = {{"EQ", "=="}, {"NE", "!="}, {"LT", "<"}, {"LE", "<="}, {"GT", ">"}, {"GE", ">="}};
    auto it = ops.find(ins->comparison);
    MONONN_CHECK(it != ops.end(), kParseError) << ins->hlo_name << ": unknown comparison direction " << ins->comparison;
    return def(dt, "(" + a[0] + " " + it->second + " " + a[1] + ")");
  }
  if (op == "select") { need(3); return def(dt, "(" + a[0] + " ? " + a[1] + " : " + a[2] + ")"); }
  if (op == "clamp") {
    need(3);
    std::string lo = a[0], x = a[1], hi = a[2];
    return def(dt, "(" + x + " < " + lo + " ? " + lo + " : (" + x + " > " + hi + " ? " + hi + " : " + x + "))");
  }
  MONONN_FAIL(kUnsupported) << ins->hlo_name << ": opcode '" << op << "' cannot be emitted inside a fused cluster";
}

}  // namespace codegen
}  // namespace mononn
