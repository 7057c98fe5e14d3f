#include "codegen/cluster_codegen.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <functional>
#include <map>
#include <memory>
#include <set>
#include <regex>
#include <sstream>

#include "common/status.h"

namespace mononn {
namespace codegen {

using graph::Node;
using graph::NodeKind;
using graph::Program;
using hlo::DType;
using hlo::Instr;

namespace {

std::string S(int64_t v) { return std::to_string(v); }

struct RowInfo {
  bool has_reduce = false;
  bool row_program = false;
  int64_t rows = 0, row_len = 0;
};

std::vector<const Instr*> reduces_of(const std::vector<const Instr*>& members) {
  std::vector<const Instr*> out;
  for (auto* m : members) {
    if (m->opcode == "fusion") {
      for (auto& i : m->called->instrs)
        if (i->opcode == "reduce") out.push_back(i.get());
    } else if (m->opcode == "reduce") {
      out.push_back(m);
    }
  }
  return out;
}

RowInfo analyze_rows(const std::vector<const Instr*>& members) {
  RowInfo info;
  auto reds = reduces_of(members);
  info.has_reduce = !reds.empty();
  if (!info.has_reduce) return info;
  info.row_program = true;
  for (auto* r : reds) {
    const hlo::Shape& x = r->operands[0]->shape;
    // one operand and its init value, or N of each with a tuple-valued reducer ((value, index) reductions)
    bool arity = r->operands.size() == 2 || (r->operands.size() > 2 && r->operands.size() % 2 == 0 && r->shape.is_tuple() &&
                                              r->shape.tuple.size() == r->operands.size() / 2);
    bool ok = arity && r->dimensions.size() == 1 && x.rank() >= 1 && r->dimensions[0] == x.rank() - 1;
    if (!ok) {
      info.row_program = false;
      break;
    }
    int64_t len = x.dims.back(), rows = x.num_elements() / std::max<int64_t>(len, 1);
    if (info.row_len == 0) {
      info.row_len = len;
      info.rows = rows;
    } else if (info.row_len != len || info.rows != rows) {
      info.row_program = false;
      break;
    }
  }
  if (!info.row_program) info.rows = info.row_len = 0;
  return info;
}

std::string signature(const std::vector<PointerTable::Entry>& ptrs) {
  std::string s = "int unit";
  for (auto& e : ptrs) s += std::string(", ") + (e.is_output ? "" : "const ") + hlo::dtype_ctype(e.dtype) + "* " + e.name;
  return s + ", char* smem";
}

Index leading_index(int var, int64_t extent, const std::vector<int64_t>& dims, const VarTable& vars) {
  return delinearize(LinExpr::variable(var, extent), dims, vars);
}

// A result that no stage of the kernel reads back (a live-out for the host only) may stay in the writer's L2 until
// the kernel ends: it is written with plain stores, which the cache merges into whole lines, instead of the
// write-through stores that carry data to the other XCDs (2-byte stores into rows of odd length: 1.6x faster).
// Before buffers are assigned (dry runs of the passes) every result counts as read inside the kernel.
bool host_only_output(const Program& prog, const Instr* out) {
  auto it = prog.buffers.find(prog.storage_root(out));
  return it != prog.buffers.end() && it->second.kind == graph::Buffer::kLiveOut && it->second.last_use_stage == it->second.def_stage;
}
// Likewise a result whose readers all sit on the XCD that wrote what they read (regional synchronisation): the
// hand-over goes through that XCD's L2.
bool plain_stored_output(const Program& prog, const Instr* out) { return host_only_output(prog, out) || prog.regional_roots.count(prog.storage_root(out)) > 0; }
std::string st1_of(const Program& prog, const Instr* out) { return plain_stored_output(prog, out) ? "mononn_dev::st1_plain(" : "mononn_dev::st1("; }
std::string stN_of(const Program& prog, const Instr* out) { return plain_stored_output(prog, out) ? "mononn_dev::stN_plain<" : "mononn_dev::stN<"; }

void store(const Program& prog, CodeBuffer& cb, PointerTable& ptrs, const VarTable& vars, const Instr* out, const Index& idx, const std::string& v) {
  cb.line(st1_of(prog, out) + ptrs.output(out) + " + " + physical_offset(prog, out, idx, &vars).str(vars) + ", " + v + ");");
}

std::string align_prologue(const std::vector<PointerTable::Entry>& ptrs);

NodeFunction finish(const std::string& body, PointerTable& ptrs, const std::vector<std::string>& globals, int64_t units, int smem,
                    const std::string& pre = "") {
  NodeFunction f;
  f.pointers = ptrs.entries;
  f.num_units = units;
  f.smem_bytes = smem;
  f.globals = globals;
  f.text = pre + "__device__ __forceinline__ void @NAME@(" + signature(ptrs.entries) + ") {\n" + align_prologue(ptrs.entries) + body + "}\n";
  return f;
}

int pick_vector_width(int64_t len, int64_t lanes) {
  // largest of 8/4/2 elements per thread that divides the row and still keeps every lane busy
  for (int v : {8, 4, 2})
    if (len % v == 0 && len / v >= lanes) return v;
  return 1;
}

std::string align_prologue(const std::vector<PointerTable::Entry>& ptrs) {
  // every buffer handed to the kernel is at least 16-byte aligned (temp offsets are multiples of 256,
  // module globals are aligned(256), caller buffers are checked at launch); telling the compiler
  // lets it merge the per-element accesses of one thread into 64/128-bit loads and stores
  std::string out;
  for (auto& e : ptrs) {
    std::string T = std::string(e.is_output ? "" : "const ") + hlo::dtype_ctype(e.dtype) + "*";
    out += "  " + e.name + " = (" + T + ")__builtin_assume_aligned(" + e.name + ", 16);\n";
  }
  return out;
}

std::vector<std::string> tables_of(const Emitter& em) {
  std::vector<std::string> v;
  for (auto& kv : em.literal_tables()) v.push_back(kv.second);
  return v;
}

// Row programs are straight-line code in which a load is emitted where its value is first needed.  A load
// whose address depends on the row and column only (LayerNorm gamma / beta, a residual) and that is first
// needed after a workgroup reduction would be issued after that reduction's barrier, putting one more trip
// to memory on the critical path.  Such loads are moved up to the head of the program: definitions of the
// form `const T vN = <expression of inK[..], row, qK>;` go right behind the last `const int qK = ...;`.
std::string hoist_row_loads(const std::string& text, bool prologue = false) {
  std::vector<std::string> lines;
  {
    std::istringstream is(text);
    std::string l;
    while (std::getline(is, l)) lines.push_back(l);
  }
  static const std::regex q_def_row(R"(^\s*const int q\d+ = .*;$)");
  static const std::regex q_def_pro(R"(^\s*const int m\d+ = .*;$)");   // a GEMM prologue: rows m0, m1, .. come last
  const std::regex& q_def = prologue ? q_def_pro : q_def_row;
  static const std::regex v_def(R"(^\s*const [A-Za-z_][\w ]* v\d+ = (.*);$)");
  static const std::regex ident(R"((^|[^\w.])([A-Za-z_]\w*))");
  static const std::regex allowed(R"(^(in\d+|q\d+|m\d+|wk|g|r16|row|lane|tid|float|double|_Float16|int|long|unsigned|short|char|bool|int8_t|uint8_t|int16_t|uint16_t|int32_t|uint32_t|int64_t|uint64_t)$)");
  int anchor = -1;
  for (size_t i = 0; i < lines.size(); ++i)
    if (std::regex_match(lines[i], q_def)) anchor = static_cast<int>(i);
  if (anchor < 0) return text;
  // Only loads of the straight-line part move: one that sits under a condition (the branches of a concatenate, a pad,
  // a window's bounds test) is guarded by it, and its address is out of range exactly where the condition is false.
  auto indent_of = [](const std::string& l) { return l.find_first_not_of(' '); };
  const size_t base_indent = indent_of(lines[anchor]);
  std::vector<std::string> hoisted, rest;
  for (size_t i = static_cast<size_t>(anchor) + 1; i < lines.size(); ++i) {
    std::smatch m;
    bool hoist = false;
    if (indent_of(lines[i]) == base_indent && std::regex_match(lines[i], m, v_def)) {
      const std::string rhs = m[1].str();
      hoist = rhs.find('[') != std::string::npos;
      // in front of a GEMM registers are scarce (operand fragments are resident): only the partial sums of a split
      // GEMM, which come from another XCD's stores, are requested ahead; constants of the row program hit nearby caches
      if (prologue && lines[i].find("const float v") == std::string::npos) hoist = false;
      for (auto it = std::sregex_iterator(rhs.begin(), rhs.end(), ident); hoist && it != std::sregex_iterator(); ++it)
        hoist = std::regex_match((*it)[2].str(), allowed);
    }
    (hoist ? hoisted : rest).push_back(lines[i]);
  }
  std::string out;
  for (int i = 0; i <= anchor; ++i) out += lines[i] + "\n";
  for (auto& l : hoisted) out += l + "\n";
  // keeps the instruction scheduler from sinking a load to its first use (it would then wait for each
  // load in turn instead of having all of them in flight)
  if (!hoisted.empty()) out += std::string(prologue ? "" : "  ") + "  __builtin_amdgcn_sched_barrier(0);\n";
  for (auto& l : rest) out += l + "\n";
  return out;
}

NodeFunction gen_cluster(const Program& prog, const std::vector<const Instr*>& members, const std::vector<const Instr*>& outputs,
                         const LaunchShape& ls, const ClusterTuning& t) {
  MONONN_CHECK(!outputs.empty(), kUnsupported) << "cluster without outputs";
  RowInfo info = analyze_rows(members);
  CodeBuffer cb;
  VarTable vars;
  PointerTable ptrs;
  Emitter em(prog, members, cb, vars, ptrs);
  const int NW = ls.waves();

  if (info.row_program) {
    const int64_t ROWS = info.rows, R = info.row_len;
    const bool block_tier = t.locality_tier == 2;
    // G = 8, 4 or 2 rows per wave (reduce_implementation 1, 2, 3), 64 / G lanes per row, 16-byte runs per lane: rows of
    // whole runs that fit the registers.  Lane l works on row l % G of the wave's G rows.
    const int group_run = 16 / hlo::dtype_bytes(outputs[0]->shape.dtype);
    const int G = t.reduce_implementation == 1 ? 8 : t.reduce_implementation == 2 ? 4 : t.reduce_implementation == 3 ? 2 : 1;
    const int GL = 64 / G;   // lanes per row
    const bool row_groups = !block_tier && G > 1 && R % group_run == 0 && R / group_run >= GL && (R / group_run + GL - 1) / GL * group_run <= 160;
    const int stride = block_tier ? ls.block_size : row_groups ? GL : 64;
    int row = vars.add("row", ROWS);
    std::vector<const Instr*> row_outs, full_outs;
    for (auto* o : outputs) {
      int64_t n = o->shape.num_elements();
      if (n == ROWS * R && R > 1) full_outs.push_back(o);
      else if (n == ROWS) row_outs.push_back(o);
      else MONONN_FAIL(kUnsupported) << o->hlo_name << ": output with " << n << " elements does not fit a " << ROWS << " x " << R << " row space";
    }
    cb.line("const int lane = mononn_dev::lane_id();");
    cb.line(std::string("const int tid = ") + (block_tier ? "(int)threadIdx.x;" : row_groups ? "lane / " + S(G) + ";" : "lane;"));
    if (block_tier) {
      cb.line("const int row = unit;");
      cb.open("");
    } else if (row_groups) {
      cb.line("const int row = (unit * " + S(NW) + " + mononn_dev::wave_id()) * " + S(G) + " + (lane & " + S(G - 1) + ");");
      cb.open("if (row < " + S(ROWS) + ")");   // the lanes of a row agree
    } else {
      cb.line("const int row = unit * " + S(NW) + " + mononn_dev::wave_id();");
      cb.open("if (row < " + S(ROWS) + ")");
    }
    auto all_reduce = [&](const Instr* r, const std::string& acc) {
      std::string T = hlo::dtype_ctype(r->shape.dtype);
      if (block_tier) cb.line(acc + " = mononn_dev::block_all_reduce(" + acc + ", " + Emitter::reducer_functor(r) + ", reinterpret_cast<" + T + "*>(smem));");
      else if (row_groups) cb.line(acc + " = mononn_dev::lane_group_all_reduce<" + S(G) + ">(" + acc + ", " + Emitter::reducer_functor(r) + ");");
      else cb.line(acc + " = mononn_dev::wave_all_reduce(" + acc + ", " + Emitter::reducer_functor(r) + ");");
    };
    // Tuple-valued reductions: N accumulators, the reducer computation inlined for every element and, as a local
    // lambda, for the exchange between lanes and waves.  The lanes combine disjoint column sets in a butterfly, so
    // the reducer has to be associative and commutative (XLA's contract for reduce), as arg-max with the
    // first-index tie rule is.
    struct TupleAcc {
      std::vector<std::string> acc, types;
    };
    auto tuple_begin = [&](const Instr* r) {
      TupleAcc ta;
      const size_t n = r->operands.size() / 2;
      for (size_t i = 0; i < n; ++i) {
        ta.types.push_back(hlo::dtype_ctype(r->shape.tuple[i].dtype));
        ta.acc.push_back(em.fresh("red"));
        cb.line(ta.types[i] + " " + ta.acc[i] + " = " + em.value(r->operands[n + i], {}) + ";");
      }
      return ta;
    };
    // acc = reducer(acc, element) ; `guard` (may be empty) keeps the accumulators where it is false
    auto tuple_update = [&](const Instr* r, const TupleAcc& ta, const std::vector<std::string>& vals, const std::string& guard) {
      const size_t n = ta.acc.size();
      std::vector<std::string> args = ta.acc;
      args.insert(args.end(), vals.begin(), vals.end());
      std::vector<std::string> res = em.inline_scalar_computation(r->called, args);
      MONONN_CHECK(res.size() == n, kUnsupported) << r->hlo_name << ": the reducer yields " << res.size() << " values for " << n << " operands";
      std::vector<std::string> tmp;
      for (size_t i = 0; i < n; ++i) {
        tmp.push_back(em.fresh("nx"));
        cb.line("const " + ta.types[i] + " " + tmp[i] + " = (" + ta.types[i] + ")" + res[i] + ";");
      }
      for (size_t i = 0; i < n; ++i) cb.line(ta.acc[i] + " = " + (guard.empty() ? tmp[i] : guard + " ? " + tmp[i] + " : " + ta.acc[i]) + ";");
    };
    auto tuple_all_reduce = [&](const Instr* r, const TupleAcc& ta) {
      const size_t n = ta.acc.size();
      std::string comb = em.fresh("comb");
      std::string params;
      std::vector<std::string> a, b;
      for (size_t i = 0; i < n; ++i) {
        a.push_back("a" + S(i));
        b.push_back("b" + S(i));
        params += (i ? ", " : "") + ta.types[i] + "& a" + S(i);
      }
      for (size_t i = 0; i < n; ++i) params += ", const " + ta.types[i] + " b" + S(i);
      cb.open("auto " + comb + " = [](" + params + ")");
      {
        TupleAcc inner{a, ta.types};
        tuple_update(r, inner, b, "");
      }
      cb.close(";");
      auto call = [&](const std::function<std::string(size_t)>& other) {
        std::string args;
        for (size_t i = 0; i < n; ++i) args += (i ? ", " : "") + ta.acc[i];
        for (size_t i = 0; i < n; ++i) args += ", " + other(i);
        return comb + "(" + args + ");";
      };
      cb.line("#pragma unroll");
      cb.open("for (int off = 32; off >= " + S(row_groups ? G : 1) + "; off >>= 1)");
      cb.line(call([&](size_t i) { return "mononn_dev::lane_xor(" + ta.acc[i] + ", off)"; }));
      cb.close();
      if (!block_tier) return;
      // across the waves: every wave leaves its tuple in LDS (member i at byte offset i * NW * 8), then every thread
      // folds them in wave order
      auto slot = [&](size_t i, const std::string& w) { return "reinterpret_cast<" + ta.types[i] + "*>(smem + " + S(static_cast<int64_t>(i) * NW * 8) + ")[" + w + "]"; };
      cb.line("__syncthreads();");
      cb.open("if (lane == 0)");
      for (size_t i = 0; i < n; ++i) cb.line(slot(i, "mononn_dev::wave_id()") + " = " + ta.acc[i] + ";");
      cb.close();
      cb.line("__syncthreads();");
      for (size_t i = 0; i < n; ++i) cb.line(ta.acc[i] + " = " + slot(i, "0") + ";");
      cb.open("for (int w = 1; w < " + S(NW) + "; ++w)");
      cb.line(call([&](size_t i) { return slot(i, "w"); }));
      cb.close();
    };
    auto tuple_bind = [&](const Instr* r, const TupleAcc& ta) {
      for (auto* u : r->users) {
        MONONN_CHECK(u->opcode == "get-tuple-element" && u->tuple_index >= 0 && static_cast<size_t>(u->tuple_index) < ta.acc.size(), kUnsupported)
            << r->hlo_name << ": a tuple-valued reduce is read through get-tuple-element only";
        em.bind(u, leading_index(row, ROWS, u->shape.dims, vars), ta.acc[u->tuple_index]);
      }
    };
    size_t max_tuple = 1;
    for (auto* r : em.collect_reduces())
      if (r->shape.is_tuple()) max_tuple = std::max(max_tuple, r->shape.tuple.size());
    auto operand_index = [&](const Instr* x, const LinExpr& col) {
      std::vector<int64_t> lead(x->shape.dims.begin(), x->shape.dims.end() - 1);
      Index xi = leading_index(row, ROWS, lead, vars);
      xi.push_back(col);
      return xi;
    };
    auto emit_row_outputs = [&]() {
      if (row_outs.empty()) return;
      em.push_scope();
      std::vector<std::pair<const Instr*, std::string>> vals;
      for (auto* o : row_outs) vals.emplace_back(o, em.value(em.resolve_output(o), leading_index(row, ROWS, o->shape.dims, vars)));
      cb.open("if (tid == 0)");
      for (auto& kv : vals) store(prog, cb, ptrs, vars, kv.first, leading_index(row, ROWS, kv.first->shape.dims, vars), kv.second);
      cb.close();
      em.pop_scope();
    };

    // Register-resident form: a thread owns T chunks of V consecutive columns, the whole row program
    // is straight-line code, so a value loaded for the first reduction is still in a register when
    // the later phases need it (one trip to memory per row instead of one per phase).
    const int V = row_groups ? group_run : t.ilp_factor > 1 && R % t.ilp_factor == 0 ? t.ilp_factor : pick_vector_width(R, stride);
    const int64_t NQ = R / V;
    const int64_t T = (NQ + stride - 1) / stride;
    if (T * V <= 32 || row_groups) {
      std::vector<int> qvar(T);
      std::vector<bool> partial(T);
      for (int64_t k = 0; k < T; ++k) {
        partial[k] = (k + 1) * stride > NQ;
        std::string q = "q" + S(k);
        if (partial[k]) {
          cb.line("const bool act" + S(k) + " = tid + " + S(k * stride) + " < " + S(NQ) + ";");
          cb.line("const int " + q + " = act" + S(k) + " ? tid + " + S(k * stride) + " : " + S(NQ - 1) + ";");
        } else {
          cb.line("const int " + q + " = tid + " + S(k * stride) + ";");
        }
        qvar[k] = vars.add(q, NQ);
      }
      auto col_of = [&](int64_t k, int v) { return LinExpr::variable(qvar[k], NQ).scaled(V).plus_const(v); };
      for (auto* r : em.collect_reduces()) {
        if (r->shape.is_tuple()) {
          TupleAcc ta = tuple_begin(r);
          const size_t n = ta.acc.size();
          for (int64_t k = 0; k < T; ++k)
            for (int v = 0; v < V; ++v) {
              std::vector<std::string> vals;
              for (size_t i = 0; i < n; ++i) vals.push_back(em.value(r->operands[i], operand_index(r->operands[i], col_of(k, v))));
              tuple_update(r, ta, vals, partial[k] ? "act" + S(k) : "");
            }
          tuple_all_reduce(r, ta);
          tuple_bind(r, ta);
          continue;
        }
        std::string Tn = hlo::dtype_ctype(r->shape.dtype);
        std::string acc = em.fresh("red");
        cb.line(Tn + " " + acc + " = " + em.value(r->operands[1], {}) + ";");
        for (int64_t k = 0; k < T; ++k)
          for (int v = 0; v < V; ++v) {
            std::string val = em.value(r->operands[0], operand_index(r->operands[0], col_of(k, v)));
            std::string upd = "(" + Tn + ")" + Emitter::reducer_expr(r, acc, val);
            if (partial[k]) cb.line(acc + " = act" + S(k) + " ? " + upd + " : " + acc + ";");
            else cb.line(acc + " = " + upd + ";");
          }
        all_reduce(r, acc);
        em.bind(r, leading_index(row, ROWS, r->shape.dims, vars), acc);
      }
      emit_row_outputs();
      for (int64_t k = 0; k < T; ++k) {
        std::vector<std::string> lines;
        for (auto* o : full_outs) {
          std::vector<std::string> vals;
          std::vector<LinExpr> offs;
          for (int v = 0; v < V; ++v) {
            LinExpr lin = LinExpr::variable(row, ROWS).scaled(R).plus(col_of(k, v));
            Index oi = delinearize(lin, o->shape.dims, vars);
            vals.push_back(em.value(em.resolve_output(o), oi));
            offs.push_back(physical_offset(prog, o, oi, &vars));
          }
          // one packed store when the V elements are adjacent in memory and the pack is 4/8/16 bytes
          const int bytes = V * hlo::dtype_bytes(o->shape.dtype);
          bool adjacent = V > 1 && (bytes == 4 || bytes == 8 || bytes == 16);
          for (int v = 1; adjacent && v < V; ++v) adjacent = offs[v].equals(offs[0].plus_const(v));
          if (adjacent) {
            std::string T = hlo::dtype_ctype(o->shape.dtype);
            std::string arr = em.fresh("pk");
            std::string init;
            for (int v = 0; v < V; ++v) init += (v ? ", " : "") + vals[v];
            lines.push_back("const " + T + " " + arr + "[" + S(V) + "] = {" + init + "};");
            lines.push_back(stN_of(prog, o) + T + ", " + S(V) + ">(" + ptrs.output(o) + " + " + offs[0].str(vars) + ", " + arr + ");");
          } else {
            for (int v = 0; v < V; ++v) lines.push_back(st1_of(prog, o) + ptrs.output(o) + " + " + offs[v].str(vars) + ", " + vals[v] + ");");
          }
        }
        if (lines.empty()) continue;
        if (partial[k]) cb.open("if (act" + S(k) + ")");
        for (auto& l : lines) cb.line(l);
        if (partial[k]) cb.close();
      }
    } else {
      // long rows: loops over the columns, operands re-read per phase
      int col = vars.add("col", R);
      const std::string col_loop = "for (int col = tid; col < " + S(R) + "; col += " + S(stride) + ")";
      for (auto* r : em.collect_reduces()) {
        if (r->shape.is_tuple()) {
          TupleAcc ta = tuple_begin(r);
          cb.open(col_loop);
          em.push_scope();
          std::vector<std::string> vals;
          for (size_t i = 0; i < ta.acc.size(); ++i) vals.push_back(em.value(r->operands[i], operand_index(r->operands[i], LinExpr::variable(col, R))));
          tuple_update(r, ta, vals, "");
          em.pop_scope();
          cb.close();
          tuple_all_reduce(r, ta);
          tuple_bind(r, ta);
          continue;
        }
        std::string Tn = hlo::dtype_ctype(r->shape.dtype);
        std::string acc = em.fresh("red");
        cb.line(Tn + " " + acc + " = " + em.value(r->operands[1], {}) + ";");
        cb.open(col_loop);
        em.push_scope();
        std::string v = em.value(r->operands[0], operand_index(r->operands[0], LinExpr::variable(col, R)));
        cb.line(acc + " = (" + Tn + ")" + Emitter::reducer_expr(r, acc, v) + ";");
        em.pop_scope();
        cb.close();
        all_reduce(r, acc);
        em.bind(r, leading_index(row, ROWS, r->shape.dims, vars), acc);
      }
      emit_row_outputs();
      if (!full_outs.empty()) {
        cb.open(col_loop);
        em.push_scope();
        for (auto* o : full_outs) {
          LinExpr lin = LinExpr::variable(row, ROWS).scaled(R).plus(LinExpr::variable(col, R));
          Index oi = delinearize(lin, o->shape.dims, vars);
          store(prog, cb, ptrs, vars, o, oi, em.value(em.resolve_output(o), oi));
        }
        em.pop_scope();
        cb.close();
      }
    }
    cb.close();
    int64_t units = block_tier ? ROWS : row_groups ? (ROWS + G * NW - 1) / (G * NW) : (ROWS + NW - 1) / NW;
    return finish(T * V <= 32 || row_groups ? hoist_row_loads(cb.text()) : cb.text(), ptrs, tables_of(em), units, block_tier ? NW * 8 * static_cast<int>(max_tuple) : 0);
  }

  // element-wise loop(s); outputs of equal element count share one loop.  A thread owns V consecutive
  // elements (V = ilp_factor when it divides the element count) so its accesses can be merged.
  std::vector<std::pair<int64_t, std::vector<const Instr*>>> groups;
  for (auto* o : outputs) {
    int64_t n = o->shape.num_elements();
    bool placed = false;
    for (auto& g : groups)
      if (g.first == n) {
        g.second.push_back(o);
        placed = true;
      }
    if (!placed) groups.push_back({n, {o}});
  }
  int64_t unit_base = 0;
  for (size_t gi = 0; gi < groups.size(); ++gi) {
    const int64_t N = groups[gi].first;
    // A thread owns V consecutive elements (one 16-byte run of the first output unless the specification names a
    // width) and, where the stage is long enough to come round several times, U such runs a workgroup apart: all
    // U * V values are computed before the first store, so the loads of a unit are in flight together and the
    // stores, whose acknowledgements a later load would otherwise wait for, come last.
    const int auto_v = std::min<int>(8, 16 / hlo::dtype_bytes(groups[gi].second[0]->shape.dtype));
    int V = 1;
    if (t.ilp_factor > 1 && N % t.ilp_factor == 0 && t.ilp_factor <= 16) V = t.ilp_factor;
    else if (t.ilp_factor <= 1 && N % auto_v == 0) V = auto_v;
    const int64_t NQ = N / V;
    const int U = NQ >= 4 * static_cast<int64_t>(ls.block_size) * 256 ? 4 : 1;
    const int64_t units = (NQ + static_cast<int64_t>(ls.block_size) * U - 1) / (static_cast<int64_t>(ls.block_size) * U);
    std::string u = "unit";
    if (groups.size() > 1) {
      cb.open(std::string(gi ? "else " : "") + "if (unit < " + S(unit_base + units) + ")");
      u = "(unit - " + S(unit_base) + ")";
    } else {
      cb.open("");
    }
    em.push_scope();
    struct Pending {
      std::string guard;
      std::vector<std::string> lines;
    };
    std::vector<Pending> stores;
    for (int uu = 0; uu < U; ++uu) {
      const std::string qv = "q" + S(static_cast<int64_t>(gi)) + "_" + S(uu);
      const std::string act = "act" + S(static_cast<int64_t>(gi)) + "_" + S(uu);
      int var = vars.add(qv, NQ);
      const std::string raw = u + " * " + S(static_cast<int64_t>(ls.block_size) * U) + " + " + S(static_cast<int64_t>(uu) * ls.block_size) + " + (int)mononn_dev::thread_id()";
      const bool exact = NQ % (static_cast<int64_t>(ls.block_size) * U) == 0;
      if (exact) {
        cb.line("const int " + qv + " = " + raw + ";");
      } else {
        // past the end: values are computed for the last run (in range), nothing is stored
        cb.line("const bool " + act + " = " + raw + " < " + S(NQ) + ";");
        cb.line("const int " + qv + " = " + act + " ? " + raw + " : " + S(NQ - 1) + ";");
      }
      Pending pend;
      pend.guard = exact ? "" : act;
      for (auto* o : groups[gi].second) {
        std::vector<std::string> vals;
        std::vector<LinExpr> offs;
        for (int v = 0; v < V; ++v) {
          LinExpr lin = LinExpr::variable(var, NQ).scaled(V).plus_const(v);
          Index oi = delinearize(lin, o->shape.dims, vars);
          vals.push_back(em.value(em.resolve_output(o), oi));
          offs.push_back(physical_offset(prog, o, oi, &vars));
        }
        const int bytes = V * hlo::dtype_bytes(o->shape.dtype);
        bool adjacent = V > 1 && (bytes == 4 || bytes == 8 || bytes == 16);
        for (int v = 1; adjacent && v < V; ++v) adjacent = offs[v].equals(offs[0].plus_const(v));
        if (adjacent) {
          std::string T = hlo::dtype_ctype(o->shape.dtype);
          std::string arr = em.fresh("pk");
          std::string init;
          for (int v = 0; v < V; ++v) init += (v ? ", " : "") + vals[v];
          pend.lines.push_back("const " + T + " " + arr + "[" + S(V) + "] = {" + init + "};");
          pend.lines.push_back(stN_of(prog, o) + T + ", " + S(V) + ">(" + ptrs.output(o) + " + " + offs[0].str(vars) + ", " + arr + ");");
        } else {
          for (int v = 0; v < V; ++v) pend.lines.push_back(st1_of(prog, o) + ptrs.output(o) + " + " + offs[v].str(vars) + ", " + vals[v] + ");");
        }
      }
      stores.push_back(std::move(pend));
    }
    for (auto& pend : stores) {
      if (!pend.guard.empty()) cb.open("if (" + pend.guard + ")");
      for (auto& l : pend.lines) cb.line(l);
      if (!pend.guard.empty()) cb.close();
    }
    em.pop_scope();
    cb.close();
    unit_base += units;
  }
  return finish(cb.text(), ptrs, tables_of(em), unit_base, 0);
}

}  // namespace

bool WriteMap::element_offset(int64_t bidx, int64_t m, int64_t n, int64_t* out) const {
  std::vector<int64_t> v(num_vars, 0);
  auto set = [&](int var, int64_t value) {
    if (var >= 0 && static_cast<size_t>(var) < v.size()) v[var] = value;
  };
  set(vb, bidx);
  if (vm4 >= 0) {   // four consecutive rows per call
    set(vm4, m / 4);
    set(vr, m % 4);
    set(vnn, n);
  } else {
    set(vm, m);
    if (vn4 >= 0) {
      set(vn4, n / 4);
      set(vr, n % 4);
    } else {
      set(vnn, n);
    }
  }
  return offset.evaluate(v, out);
}

bool operand_offset_expr(const Program& prog, const Instr* operand, int64_t elements, LinExpr* out) {
  const Instr* root = prog.storage_root(operand);
  if (root->shape.num_elements() != elements) return false;
  VarTable vars;
  const int ve = vars.add("e", elements);
  *out = physical_offset(prog, root, delinearize(LinExpr::variable(ve, elements), root->shape.dims, vars), &vars);
  return true;
}

std::vector<const Instr*> external_outputs(const Program& prog, const std::vector<const Instr*>& members) {
  std::set<const Instr*> mem(members.begin(), members.end());
  const Instr* root = prog.module->entry->root;
  std::function<bool(const Instr*)> used_outside = [&](const Instr* v) -> bool {
    if (v == root) return true;
    for (auto* u : v->users) {
      if (mem.count(u)) continue;
      if (graph::is_alias_op(u)) {
        if (used_outside(u)) return true;
        continue;
      }
      if (u->opcode == "tuple") {
        if (u == root) return true;
        MONONN_FAIL(kUnsupported) << u->hlo_name << ": tuple that is not the module root";
      }
      return true;
    }
    return false;
  };
  std::vector<const Instr*> out;
  for (auto& up : prog.module->entry->instrs) {
    const Instr* v = up.get();
    bool defined = (mem.count(v) && !v->shape.is_tuple()) || (v->opcode == "get-tuple-element" && mem.count(v->operands[0]));
    if (defined && used_outside(v)) out.push_back(v);
  }
  return out;
}

void classify_cluster(const Program& prog, Node& node) {
  (void)prog;
  RowInfo info = analyze_rows(node.members);
  node.has_reduce = info.has_reduce;
  node.row_program = info.row_program;
  node.rows = info.rows;
  node.row_len = info.row_len;
}

NodeFunction generate_cluster(const Program& prog, const Node& node, const LaunchShape& ls, const ClusterTuning& t) {
  return gen_cluster(prog, node.members, node.outputs, ls, t);
}

bool can_merge_clusters(const Program& prog, const std::vector<const Instr*>& producer, const std::vector<const Instr*>& consumer,
                        const std::vector<const Instr*>& merged) {
  (void)producer;
  (void)consumer;
  RowInfo info = analyze_rows(merged);
  if (info.has_reduce && !info.row_program) return false;
  try {
    auto outs = external_outputs(prog, merged);
    if (outs.empty()) return false;
    if (!info.has_reduce) {
      for (auto* o : outs)
        if (o->shape.num_elements() != outs[0]->shape.num_elements()) return false;
    }
    gen_cluster(prog, merged, outs, LaunchShape{}, ClusterTuning{});
    return true;
  } catch (const Error& e) {
    if (e.code() == kUnsupported) return false;
    throw;
  }
}

// ------------------------------------------------------------------------------------------
// GEMM
// ------------------------------------------------------------------------------------------
bool gemm_uses_mfma(const graph::GemmDesc& g) {
  if (g.f32) return !g.is_conv && g.a_k_contig;   // f32 tiles take any k extent and either right-operand layout
  if (g.is_conv && !g.conv_fragment_loads()) return false;
  // either operand k-contiguous, or a plain matrix with k as its slow dimension (gathered per lane); the right one
  // also packed.  An m-contiguous left operand comes as plain memory only: no fragment order, no convolution map.
  if (!g.a_k_contig && (g.a_packed || g.is_conv)) return false;
  // a k extent that is not a multiple of 32 is zero-filled in the last step, from plain row-major operands only
  return g.K % 32 == 0 || (!g.is_conv && !g.b_packed && !g.a_packed && g.split_k <= 1);
}

// the LDS-staged tile copies k-contiguous or fragment-order operands
static bool gemm_lds_capable(const graph::GemmDesc& g) { return !g.f32 && gemm_uses_mfma(g) && g.a_k_contig && (g.b_k_contig || g.b_packed) && g.K % 32 == 0; }

GemmTuning default_gemm_tuning(const graph::GemmDesc& g, const LaunchShape& ls, int num_cus, bool allow_lds_tile) {
  GemmTuning t;
  int waves = ls.waves();
  // Large problems: every wave owns a 64x64 (else 32x32) block of the result over the whole k range, no exchange
  // through LDS, as long as that still leaves a tile per compute unit (BERT-large at batch 16: 128x128 tiles run
  // 2.1x faster than the small-problem default below).  Larger blocks per wave (64x128, 128x128) fetch fewer operand
  // fragments per MFMA and are up to 1.5x faster on such a GEMM alone (its tiles are bound by what the L1
  // delivers), but inside whole models they made the kernels slower more often than faster (BERT-large 9.9 ->
  // 11.6 ms: stages whose code did not change, attention and LayerNorm, slow down with them), so they are
  // neither the default nor tuner candidates (they win the isolated stage clocks and lose in the whole kernel);
  // a specification may still name them (up to 64 accumulator fragments per wave).
  // Large problems (any MFMA-capable GEMM with k a multiple of 32): operand tiles go through LDS once per workgroup.
  // Among the tile shapes the one that needs the least time by a simple model: rounds of tiles over the compute
  // units x tile area / throughput of a compute unit that is busy with such a tile, relative to 256 x 256 (measured
  // on [6144, 1024] x [1024, 4096] with both operands in fragment order: 1.0 PFLOP/s-equivalent for 256 x 256,
  // which fills the chip only 1.5 times there; 0.87 for 192 x 256, which fills it twice).
  if (allow_lds_tile && gemm_lds_capable(g) && g.K >= 128 && waves == 4 && ls.waves_per_simd == 1 && g.split_k <= 1) {
    struct Cand { int bm, bn, bk; double eff; };
    double best = 0;
    const int cus = std::max(num_cus, 1);
    for (const Cand& c : {Cand{256, 256, 32, 1.0}, Cand{192, 256, 32, 0.86}, Cand{256, 192, 32, 0.82}, Cand{256, 128, 64, 0.78}, Cand{128, 256, 64, 0.77},
                          Cand{192, 128, 64, 0.74}, Cand{128, 128, 64, 0.65}}) {
      if (g.M < c.bm || g.N < c.bn) continue;
      const int64_t units = ((g.M + c.bm - 1) / c.bm) * ((g.N + c.bn - 1) / c.bn) * g.batch;
      if (units < cus) continue;   // every compute unit gets a tile, or the small-problem paths below take over
      const int64_t rounds = (units + cus - 1) / cus;
      // per tile: its multiply-adds at the tile's efficiency plus a fixed cost (first operands on their way, epilogue,
      // waves of a workgroup out of step) worth about ten million multiply-adds
      const double cost = static_cast<double>(rounds) * (static_cast<double>(c.bm) * c.bn * g.K / c.eff + 1.0e7);
      if (best == 0 || cost < best) {
        best = cost;
        t.bm = c.bm;
        t.bn = c.bn;
        t.bk = c.bk;
      }
    }
    if (best > 0) {
      t.wm = 2;
      t.wn = 2;
      t.wk = 1;
      t.stages = 2;
      return t;
    }
  }
  for (int per_wave : {64, 32}) {
    if (!allow_lds_tile) break;             // a row program in front: the waves split k so that a wave's fragments of its rows fit its registers
    if (g.f32 && per_wave > 32) continue;   // 16 fragments of a 64 x 64 block leave no room for a chunk in flight
    int wm = 1, wn = waves;
    while (wn > wm) {
      wn /= 2;
      wm *= 2;
    }
    const int bm = per_wave * wm, bn = per_wave * wn;
    const int64_t units = ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * g.batch;
    if (units >= static_cast<int64_t>(std::max(num_cus, 1)) && g.M >= bm && g.N >= bn) {
      t.wm = wm;
      t.wn = wn;
      t.wk = 1;
      t.bm = bm;
      t.bn = bn;
      return t;
    }
  }
  int wk = 1;
  while (!g.f32 && wk * 2 <= waves && g.K / 32 >= wk * 2 * 2 && g.K >= 256 * wk) wk *= 2;
  // with a row program in front a wave holds the fragments of its rows over its whole k range: as many waves along k
  // as divide the k steps
  if (!allow_lds_tile && !g.f32)
    while (wk * 2 <= waves && (g.K / 32) % (wk * 2) == 0) wk *= 2;
  t.wk = wk;
  int rest = waves / wk;
  t.wm = 1;
  t.wn = rest;
  while (t.wn > 1 && t.wn * 32 > g.N && t.wn % 2 == 0) {
    t.wn /= 2;
    t.wm *= 2;
  }
  t.bm = 32 * t.wm;
  t.bn = 32 * t.wn;
  return t;
}

void validate_gemm_tuning(const graph::GemmDesc& g, const LaunchShape& ls, const GemmTuning& t, bool has_prologue) {
  if (g.f32) {
    MONONN_CHECK(!has_prologue && t.wk == 1 && t.stages < 2 && t.split_k <= 1, kSpecError)
        << "an f32 GEMM tile takes no row-program prologue, no k split (over waves or workgroups) and no LDS staging";
    MONONN_CHECK((t.bm / std::max(t.wm, 1) / 16) * (t.bn / std::max(t.wn, 1) / 16) <= 16, kSpecError) << "f32 GEMM tile " << t.bm << "x" << t.bn << ": more than 16 fragments per wave";
  }
  if (has_prologue) {
    const int tm = t.bm / std::max(t.wm, 1) / 16, tn = t.bn / std::max(t.wn, 1) / 16;
    const int64_t ksteps = g.K / 32;
    // mirrors mononn_dev::gemm_chunk_steps: with the weights requested ahead of the tile a wave keeps up to 56 fragments
    const bool wide = t.preload_b && g.b_packed && t.wk >= 1 && ksteps / t.wk * (tm + tn) <= ls.whole_range_fragments();
    MONONN_CHECK(t.wk >= 1 && ksteps % t.wk == 0 && tm + tn > 0 && (wide || ksteps / t.wk <= (tm * tn > 32 ? ls.chunk_fragments() / 2 : ls.chunk_fragments()) / (tm + tn)), kSpecError)
        << "GEMM with a row-program prologue: a wave's whole k range (" << ksteps / std::max(t.wk, 1) << " steps) must fit one register chunk";
  }
  MONONN_CHECK(t.split_k >= 1 && (t.split_k == 1 || g.K % (32 * t.split_k) == 0), kSpecError)
      << "split_k " << t.split_k << " does not divide the k steps of the GEMM";
  MONONN_CHECK(t.wm >= 1 && t.wn >= 1 && t.wk >= 1 && t.wm * t.wn * t.wk == ls.waves(), kSpecError)
      << "GEMM wave arrangement " << t.wm << "x" << t.wn << "x" << t.wk << " does not use " << ls.waves() << " waves";
  MONONN_CHECK(t.bm % (16 * t.wm) == 0 && t.bn % (16 * t.wn) == 0 && t.bm > 0 && t.bn > 0, kSpecError)
      << "GEMM tile " << t.bm << "x" << t.bn << " is not a multiple of 16 per wave";
  if (t.stages >= 2) {
    MONONN_CHECK(g.a_k_contig && (g.b_k_contig || g.b_packed), kSpecError) << "an LDS-staged GEMM tile takes a k-contiguous left operand and a k-contiguous or packed right operand";
    MONONN_CHECK(!has_prologue && t.wk == 1 && g.K % 32 == 0, kSpecError) << "an LDS-staged GEMM tile takes no row-program prologue, no k split over waves and a k extent that is a multiple of 32";
    MONONN_CHECK(t.stages == 2 && t.bk >= 32 && t.bk % 32 == 0 && t.bk <= 128, kSpecError)
        << "LDS-staged GEMM tile: " << t.stages << " stages of " << t.bk << " k: two LDS buffers of 32, 64, 96 or 128 k";
    const int kstp = t.bk / 16, ablk = t.bm / 32 * kstp, bblk = t.bn / 32 * kstp;   // 1 KiB blocks of 32 rows x 16 k
    MONONN_CHECK(t.bm % (32 * t.wm) == 0 && t.bn % (32 * t.wn) == 0, kSpecError) << "LDS-staged GEMM tile " << t.bm << "x" << t.bn << " is not a multiple of 32 per wave";
    MONONN_CHECK(ablk % ls.waves() == 0 && bblk % ls.waves() == 0, kSpecError)
        << "LDS-staged GEMM tile " << t.bm << "x" << t.bn << "x" << t.bk << ": the " << ls.waves() << " waves cannot share the copy of a k tile evenly";
    MONONN_CHECK((ablk + bblk) / ls.waves() <= 16, kSpecError) << "LDS-staged GEMM tile " << t.bm << "x" << t.bn << "x" << t.bk << ": more than 16 staged pieces per lane and k tile";
  }
  int frags = (t.bm / t.wm / 16) * (t.bn / t.wn / 16);
  const int max_frags = ls.waves_per_simd >= 2 ? 32 : 64;   // 4 accumulator registers each, out of 512 / waves per SIMD
  MONONN_CHECK(frags <= max_frags, kSpecError) << "GEMM tile " << t.bm << "x" << t.bn << " needs " << frags << " accumulator fragments per wave (max " << max_frags << ")";
}

namespace {

// Epilogue of an MFMA / fallback GEMM as a functor: the GEMM result (fp32 accumulator, scaled, rounded
// to the f16 value the HLO defines) is bound to a register and every fused element-wise cluster is
// emitted on top of it.  Pointers the epilogue needs are appended to `ptrs`; the functor's members
// are all entries from `first_epi` on.
struct Epilogue {
  std::string struct_text;   // struct @NAME@_epi { ... };
  bool along_m = false;      // the four values of a call are four consecutive rows of one column (else columns of one row)
  int vector_stores = 0;     // outputs written with one 8-byte store per call
  std::string init_line;     // @NAME@_epi epi{...};
  std::vector<std::string> globals;
  std::vector<WriteMap> writes;   // where each output's element (bidx, m, n) goes (not for split-K partial sums)
};

// along_m: the MFMA is issued with the operands swapped, so that a lane holds four consecutive rows m of one
// column n; outputs that are stored with m as the fast dimension (a transposed result) then take one packed
// store instead of four scattered ones.
// fold / fold_bm: the left operand's LayerNorm is folded (graph::LayerNormFold); the accumulator then holds
// x . (gamma o W) and becomes the GEMM value as r[m] * (acc - mean[m] * colsum_gamma[n]) + colsum_beta[n], with mean and
// r of the workgroup's fold_bm rows read from LDS (`ln_stats`, written by the statistics functor in front of the MFMAs).
Epilogue build_epilogue(const Program& prog, const Instr* gi, const std::vector<const Instr*>& cluster_members,
                        const std::vector<const Instr*>& outputs, const graph::GemmDesc& g, bool mfma, PointerTable& ptrs,
                        size_t first_epi, bool along_m = false, const graph::LayerNormFold* fold = nullptr, int fold_bm = 0) {
  if (g.split_k > 1) {
    // fp32 partial sums [split][batch][M][N]; the consumers add them up and apply the rounding
    MONONN_CHECK(mfma && g.N % 4 == 0 && cluster_members.empty() && outputs.size() == 1 && outputs[0] == gi && !g.has_addend, kSpecError)
        << gi->hlo_name << ": split_k needs the MFMA path, N % 4 == 0 and no fused epilogue";
    std::string po = ptrs.output(gi, DType::kF32);
    std::ostringstream al;
    al.precision(9);
    al << g.alpha;
    std::string a = al.str();
    if (a.find_first_of(".e") == std::string::npos) a += ".0";
    Epilogue e;
    // where element (bidx, m, n0) of one partial sum lives: row-major, or in fragment order when the consumer
    // takes the rows as MFMA fragments (a row program fused in front of the next GEMM)
    std::string where = "(long)bidx * " + S(g.M * g.N) + " + m * " + S(g.N) + " + n0";
    if (prog.physical_tile.count(gi)) {
      VarTable tv;
      int vbi = tv.add("bidx", g.batch), vmi = tv.add("m", g.M), vni = tv.add("n4", g.N / 4);
      Index gidx = delinearize(LinExpr::variable(vbi, g.batch), std::vector<int64_t>(gi->shape.dims.begin(), gi->shape.dims.end() - 2), tv);
      gidx.push_back(LinExpr::variable(vmi, g.M));
      gidx.push_back(LinExpr::variable(vni, g.N / 4).scaled(4));
      where = physical_offset(prog, gi, gidx, &tv).str(tv);
    }
    e.struct_text = "struct @NAME@_epi {\n  float* out;\n  int ksplit;\n"
                    "  struct Pre {};\n"
                    "  __device__ __forceinline__ void preload(int, int, int, Pre&) const {}\n"
                    "  __device__ __forceinline__ void operator()(int bidx, int m, int n0, const float (&acc)[4], const Pre&) const {\n"
                    "    const int n4 = n0 >> 2;\n    (void)n4;\n"
                    "    const float v[4] = {acc[0] * " + a + "f, acc[1] * " + a + "f, acc[2] * " + a + "f, acc[3] * " + a + "f};\n"
                    "    mononn_dev::stN<float, 4>(out + (long)ksplit * " + S(g.batch * g.M * g.N) + " + " + where + ", v);\n"
                    "  }\n};\n";
    e.init_line = "@NAME@_epi epi{" + po + ", ksplit};";
    return e;
  }
  MONONN_CHECK(!along_m || (mfma && g.M % 4 == 0 && !g.is_conv), kUnsupported) << gi->hlo_name << ": rows cannot be taken four at a time";
  const bool vec4 = mfma && (along_m || g.N % 4 == 0);
  // N off the lane's run of 4 columns (an LM head over 50257 tokens): the rows start at addresses that are only
  // 2-byte aligned.  A single f16 result that only the host reads is still written four columns at a time, through
  // a copy without an alignment promise, wherever the whole run lies inside the row (decided further down).
  bool ragged4 = false;
  std::string ragged4_offset, ragged4_type = "_Float16";
  std::vector<std::pair<std::string, std::string>> fold_loads;   // (expression, type) of the folded LayerNorm's column sums
  CodeBuffer cb;   // epilogue body
  VarTable vars;
  Emitter em(prog, cluster_members, cb, vars, ptrs);
  const hlo::Shape& D = gi->shape;
  std::vector<int64_t> batch_dims(D.dims.begin(), D.dims.end() - 2);
  int vb = vars.add("bidx", g.batch);
  int vm = -1, vm4 = -1, vn4 = -1, vr = -1, vnn = -1;
  if (along_m) {
    vm4 = vars.add("m4", g.M / 4);
    vr = vars.add("r", 4);
    vnn = vars.add("nn", g.N);
  } else {
    vm = vars.add("m", g.M);
    if (vec4) {
      vn4 = vars.add("n4", g.N / 4);
      vr = vars.add("r", 4);
    } else {
      vnn = vars.add("nn", g.N);
    }
  }
  auto gemm_index = [&](bool with_r) {
    Index idx;
    if (g.is_conv) {
      // the GEMM row m enumerates the output pixels (n, p, q) in row-major order
      idx = delinearize(LinExpr::variable(vm, g.M), std::vector<int64_t>(D.dims.begin(), D.dims.end() - 1), vars);
    } else if (along_m) {
      idx = delinearize(LinExpr::variable(vb, g.batch), batch_dims, vars);
      LinExpr m = LinExpr::variable(vm4, g.M / 4).scaled(4);
      if (with_r) m = m.plus(LinExpr::variable(vr, 4));
      idx.push_back(m);
      idx.push_back(LinExpr::variable(vnn, g.N));
      return idx;
    } else {
      idx = delinearize(LinExpr::variable(vb, g.batch), batch_dims, vars);
      idx.push_back(LinExpr::variable(vm, g.M));
    }
    if (vec4) {
      LinExpr n = LinExpr::variable(vn4, g.N / 4).scaled(4);
      if (with_r) n = n.plus(LinExpr::variable(vr, 4));
      idx.push_back(n);
    } else {
      idx.push_back(LinExpr::variable(vnn, g.N));
    }
    return idx;
  };
  // output index candidates derived from the GEMM coordinates: identity, or through one transpose
  auto candidates = [&](const Instr* o, bool with_r) {
    std::vector<Index> c;
    LinExpr lin = linearize(gemm_index(with_r), D.dims);
    c.push_back(delinearize(lin, o->shape.dims, vars));
    for (auto* m : cluster_members) {
      if (m->opcode != "fusion") continue;
      for (auto& up : m->called->instrs) {
        const Instr* tr = up.get();
        if (tr->opcode != "transpose" || tr->shape.num_elements() != D.num_elements()) continue;
        Index in = delinearize(lin, tr->operands[0]->shape.dims, vars);
        Index outi(in.size());
        for (size_t i = 0; i < in.size(); ++i) outi[i] = in[tr->dimensions[i]];
        c.push_back(delinearize(linearize(outi, tr->shape.dims), o->shape.dims, vars));
      }
    }
    return c;
  };

  const double alpha = g.alpha;
  std::ostringstream alpha_s;
  alpha_s.precision(9);
  alpha_s << alpha;
  std::string alpha_lit = alpha_s.str();
  if (alpha_lit.find_first_of(".e") == std::string::npos) alpha_lit += ".0";
  alpha_lit += "f";

  if (along_m) cb.line("const int m4 = m0 >> 2;");
  else if (vec4) cb.line("const int n4 = n0 >> 2;");
  // per-output staging arrays for the vector store
  struct Out {
    const Instr* o;
    Index idx;        // chosen index (with r)
    Index idx_base;   // same with r = 0
    bool vector_store;
    std::string stage;
  };
  std::vector<Out> outs;
  int n_vector_stores = 0;
  for (auto* o : outputs) {
    MONONN_CHECK(o->shape.num_elements() == D.num_elements(), kUnsupported)
        << o->hlo_name << ": epilogue output has a different element count than the GEMM result";
    outs.push_back({o, {}, {}, false, ""});
  }
  if (vec4) {
    for (size_t i = 0; i < outs.size(); ++i) {
      outs[i].stage = "st" + S(static_cast<int64_t>(i));
      cb.line(std::string(hlo::dtype_ctype(outs[i].o->shape.dtype)) + " " + outs[i].stage + "[4];");
    }
    cb.line("#pragma unroll");
    cb.open("for (int r = 0; r < 4; ++r)");
  } else {
    cb.open("");
  }
  em.push_scope();
  {
    Index gidx = gemm_index(true);
    std::string accv = vec4 ? "acc[r]" : "acc";
    if (fold) {
      MONONN_CHECK(mfma && vec4 && alpha == 1.0 && !g.has_addend && fold_bm > 0, kInternal) << gi->hlo_name << ": folded LayerNorm outside its preconditions";
      const std::string pc1 = ptrs.input(fold->colsum_gamma), pc2 = ptrs.input(fold->colsum_beta);
      const std::string row = along_m ? "((m0 + r) % " + S(fold_bm) + ")" : "(m % " + S(fold_bm) + ")";
      const std::string col = along_m ? "nn" : "n4 * 4 + r";
      // the two column sums are requested with the other operands of the epilogue, ahead of the main loop
      fold_loads = {{pc1 + "[" + col + "]", "float"}, {pc2 + "[" + col + "]", "float"}};
      cb.line("const float ln_acc = ln_stats[" + row + " * 2 + 1] * (" + accv + " - ln_stats[" + row + " * 2] * " + fold_loads[0].first + ") + " + fold_loads[1].first + ";");
      accv = "ln_acc";
    }
    std::string expr = alpha == 1.0 ? accv : "(" + accv + " * " + alpha_lit + ")";
    if (g.has_addend) {
      std::ostringstream beta_s;
      beta_s.precision(9);
      beta_s << g.beta;
      std::string beta_lit = beta_s.str();
      if (beta_lit.find_first_of(".e") == std::string::npos) beta_lit += ".0";
      std::string c = em.value(gi->operands[2], gidx);
      expr = "(" + expr + " + " + beta_lit + "f * (float)" + c + ")";
    }
    std::string gv = em.fresh("g");
    const std::string gt = hlo::dtype_ctype(gi->shape.dtype);   // the GEMM's value as the HLO defines it: rounded to its result type
    cb.line("const " + gt + " " + gv + " = (" + gt + ")" + expr + ";");
    em.bind(gi, gidx, gv);
    for (auto& out : outs) {
      if (out.o == gi) {
        out.idx = gidx;
        out.idx_base = gemm_index(false);
      } else {
        // pick the first candidate index under which every read of the GEMM value is aligned
        auto cands = candidates(out.o, true);
        auto bases = candidates(out.o, false);
        bool found = false;
        std::string last_err;
        for (size_t c = 0; c < cands.size() && !found; ++c) {
          CodeBuffer scratch;
          VarTable vcopy = vars;
          PointerTable pcopy = ptrs;
          Emitter probe(prog, cluster_members, scratch, vcopy, pcopy);
          probe.bind(gi, gidx, gv);
          try {
            probe.value(probe.resolve_output(out.o), cands[c]);
            out.idx = cands[c];
            out.idx_base = bases[c];
            found = true;
          } catch (const Error& e) {
            if (e.code() != kUnsupported) throw;
            last_err = e.what();
          }
        }
        MONONN_CHECK(found, kUnsupported) << out.o->hlo_name << ": not an element-wise function of the GEMM result (" << last_err << ")";
      }
      std::string v = em.value(em.resolve_output(out.o), out.idx);
      if (vec4) {
        LinExpr full = physical_offset(prog, out.o, out.idx, &vars);
        LinExpr base = physical_offset(prog, out.o, out.idx_base, &vars);
        out.vector_store = full.equals(base.plus(LinExpr::variable(vr, 4))) && hlo::is_half_float(out.o->shape.dtype);
        if (out.vector_store) ++n_vector_stores;
        if (out.vector_store) cb.line(out.stage + "[r] = " + v + ";");
        else store(prog, cb, ptrs, vars, out.o, out.idx, v);
      } else {
        if (mfma && !along_m && !g.is_conv && outs.size() == 1 && hlo::is_half_float(out.o->shape.dtype) && host_only_output(prog, out.o) && g.N >= 4) {
          ragged4_type = hlo::dtype_ctype(out.o->shape.dtype);
          Index at0 = out.idx;
          // the same element with column 0: the offset must be that plus the column
          Index probe_idx = delinearize(linearize([&] {
            Index z = delinearize(LinExpr::variable(vb, g.batch), batch_dims, vars);
            z.push_back(LinExpr::variable(vm, g.M));
            z.push_back(LinExpr::constant(0));
            return z;
          }(), D.dims), out.o->shape.dims, vars);
          if (out.o == gi) probe_idx = [&] {
            Index z = delinearize(LinExpr::variable(vb, g.batch), batch_dims, vars);
            z.push_back(LinExpr::variable(vm, g.M));
            z.push_back(LinExpr::constant(0));
            return z;
          }();
          LinExpr full = physical_offset(prog, out.o, out.idx, &vars);
          LinExpr base = physical_offset(prog, out.o, probe_idx, &vars);
          if (full.equals(base.plus(LinExpr::variable(vnn, g.N)))) {
            ragged4 = true;
            ragged4_offset = ptrs.output(out.o) + " + " + base.str(vars);   // (registers the pointer as a member of the functor)
          }
        }
        if (ragged4) cb.line("return " + v + ";");
        else store(prog, cb, ptrs, vars, out.o, out.idx, v);
      }
    }
  }
  em.pop_scope();
  cb.close();
  std::vector<WriteMap> writes;
  for (auto& out : outs) {
    WriteMap w;
    w.root = prog.storage_root(out.o);
    w.offset = physical_offset(prog, out.o, out.idx, &vars);
    w.vb = vb, w.vm = vm, w.vm4 = vm4, w.vn4 = vn4, w.vr = vr, w.vnn = vnn;
    w.num_vars = vars.size();
    w.batch = g.batch, w.M = g.M, w.N = g.N;
    writes.push_back(w);
  }
  if (vec4) {
    for (auto& out : outs)
      if (out.vector_store) {
        std::string lin = physical_offset(prog, out.o, out.idx_base, &vars).str(vars);
        cb.line(stN_of(prog, out.o) + hlo::dtype_ctype(out.o->shape.dtype) + ", 4>(" + ptrs.output(out.o) + " + " + lin + ", " + out.stage + ");");
      }
  }

  // ---- assemble: epilogue functor + stage function -------------------------------------------
  std::string pre = "struct @NAME@_epi {\n";
  for (size_t i = first_epi; i < ptrs.entries.size(); ++i) {
    auto& e = ptrs.entries[i];
    pre += std::string("  ") + (e.is_output ? "" : "const ") + hlo::dtype_ctype(e.dtype) + "* " + e.name + ";\n";
  }
  if (fold) pre += "  const float* ln_stats = nullptr;   // LDS: (mean, rsqrt(var + eps)) of the workgroup's rows\n";
  // Operands of the epilogue (bias, residual) whose address depends on (bidx, m, n) only are loaded into
  // registers ahead of the GEMM main loop, so their latency overlaps it; the body then reads the registers.
  std::vector<std::pair<std::string, std::string>> preloads;
  std::string body_text = cb.text();
  if (mfma) {
    pre += "  struct Pre {\n";
    if (vec4) {
      for (auto& l : em.simple_loads()) {
        bool seen = false;
        for (auto& q : preloads) seen = seen || q.first == l.first;
        if (!seen) preloads.push_back(l);
      }
      for (auto& l : fold_loads) preloads.push_back(l);
      for (size_t i = 0; i < preloads.size(); ++i) pre += "    " + preloads[i].second + " v" + S(i) + "[4];\n";
    }
    pre += "  };\n";
    pre += along_m ? "  __device__ __forceinline__ void preload(int bidx, int m0, int nn, Pre& pre) const {\n"
                   : "  __device__ __forceinline__ void preload(int bidx, int m, int n0, Pre& pre) const {\n";
    if (!preloads.empty()) {
      pre += along_m ? "    const int m4 = m0 >> 2;\n" : "    const int n4 = n0 >> 2;\n";
      pre += "    #pragma unroll\n    for (int r = 0; r < 4; ++r) {\n";
      for (size_t i = 0; i < preloads.size(); ++i) pre += "      pre.v" + S(i) + "[r] = " + preloads[i].first + ";\n";
      pre += "    }\n";
    }
    pre += "  }\n";
    for (size_t i = 0; i < preloads.size(); ++i) {
      const std::string& ref = preloads[i].first;
      const std::string with = "pre.v" + S(i) + "[r]";
      for (size_t pos = body_text.find(ref); pos != std::string::npos; pos = body_text.find(ref, pos + with.size())) body_text.replace(pos, ref.size(), with);
    }
  }
  if (along_m) pre += "  __device__ __forceinline__ void operator()(int bidx, int m0, int nn, const float (&acc)[4], const Pre& pre) const {\n";
  else if (vec4) pre += "  __device__ __forceinline__ void operator()(int bidx, int m, int n0, const float (&acc)[4], const Pre& pre) const {\n";
  else if (mfma) {
    pre += "  __device__ __forceinline__ void operator()(int bidx, int m, int n0, const float (&accv)[4], const Pre&) const {\n";
    if (ragged4) {
      pre += "    " + ragged4_type + "* row = " + ragged4_offset + ";\n";
      pre += "    if (n0 + 3 < " + S(g.N) + ") {\n";
      pre += "      const " + ragged4_type + " st[4] = {one(bidx, m, n0, accv[0]), one(bidx, m, n0 + 1, accv[1]), one(bidx, m, n0 + 2, accv[2]), one(bidx, m, n0 + 3, accv[3])};\n";
      pre += "      mononn_dev::stN_plain_unaligned<" + ragged4_type + ", 4>(row + n0, st);\n";
      pre += "    } else {\n";
      pre += "      for (int r = 0; r < 4; ++r) { const int nn = n0 + r; if (nn < " + S(g.N) + ") mononn_dev::st1_plain(row + nn, one(bidx, m, nn, accv[r])); }\n";
      pre += "    }\n  }\n";
      pre += "  __device__ __forceinline__ " + ragged4_type + " one(int bidx, int m, int nn, float acc) const {\n";
    } else {
      pre += "    for (int r = 0; r < 4; ++r) { const int nn = n0 + r; if (nn < " + S(g.N) + ") { const float acc = accv[r]; one(bidx, m, nn, acc); } }\n  }\n";
      pre += "  __device__ __forceinline__ void one(int bidx, int m, int nn, float acc) const {\n";
    }
  } else {
    pre += "  __device__ __forceinline__ void operator()(int bidx, int m, int nn, float acc) const {\n";
  }
  {
    std::istringstream is(body_text);
    std::string l;
    while (std::getline(is, l)) pre += "  " + l + "\n";
  }
  pre += "  }\n};\n";

  Epilogue out_e;
  out_e.struct_text = pre;
  out_e.along_m = along_m;
  out_e.vector_stores = n_vector_stores;
  std::string init = "@NAME@_epi epi{";
  for (size_t i = first_epi; i < ptrs.entries.size(); ++i) init += (i > first_epi ? ", " : "") + ptrs.entries[i].name;
  init += "};";
  out_e.init_line = init;
  out_e.writes = writes;
  for (auto& kv : em.literal_tables()) out_e.globals.push_back(kv.second);
  return out_e;
}

// Row program (LayerNorm) on the A fragments of gemm_tile.  Lane (r16, g) of the wave with k slot wk
// holds, for row fragment i and k step s, the 8 elements of row m_base + 16 i + r16 at columns
// 32 (s WK + wk) + 8 g + e.  The program is generated as straight-line code over those CH * 8 values
// per row fragment; a reduction ends with two butterfly steps over the 4 lanes of a row and one LDS
// exchange between the WK waves.  The results replace the fragments in place.
struct Prologue {
  std::string struct_text;   // struct @NAME@_pro { ... };
  std::string init_line;
  std::vector<std::string> globals;
  int smem = 0;
  const Instr* primary = nullptr;   // the [M,K] input whose rows arrive as MFMA fragments
};

}  // namespace

// primary input of a row program fused in front of a GEMM: an [M,K] f16 value that the cluster reads from outside
// and that is stored as such (not as the partial sums of a split GEMM); its rows arrive as MFMA fragments
const Instr* prologue_primary(const Program& prog, const std::vector<const Instr*>& row_members, int64_t M, int64_t K) {
  std::set<const Instr*> mem(row_members.begin(), row_members.end());
  for (auto* m : row_members)
    for (auto* o : m->operands) {
      const Instr* r = prog.storage_root(o);
      if (mem.count(r) || (r->opcode == "get-tuple-element" && mem.count(r->operands[0]))) continue;
      if (prog.split_k.count(r)) continue;
      if (r->shape.dtype == DType::kF16 && r->shape.dims == std::vector<int64_t>({M, K})) return r;
    }
  return nullptr;
}

namespace {

// ---- LayerNorm recogniser -------------------------------------------------------------------------------------------
// A row program in front of a GEMM is generated element by element from whatever the HLO says.  For the one program
// that matters there (LayerNorm: y = (x - mean(x)) * rsqrt(var(x) + eps) * gamma + beta over the last dimension) a
// hand-laid-out form is an order of magnitude cheaper, so the program's expression is rebuilt symbolically from the
// member fusions and compared with that formula (operand order of + and * free).  Anything else keeps the generic form.
struct Sym {
  enum Kind { kX, kCol, kConst, kRowSum, kOp };
  enum Class { kScalar, kRow, kColumn, kFull };
  Kind kind = kOp;
  Class cls = kScalar;
  std::string op;              // kOp: add subtract multiply divide rsqrt
  double c = 0;                // kConst
  const Instr* col = nullptr;  // kCol: a [K] vector read from outside the program
  std::vector<std::shared_ptr<Sym>> kids;
};
using SymP = std::shared_ptr<Sym>;

struct LayerNormMatch {
  const Instr* gamma = nullptr;
  const Instr* beta = nullptr;
  double eps = 0;
};

struct SymBuilder {
  const Program& prog;
  std::set<const Instr*> members;
  const Instr* primary;
  int64_t K;
  bool failed = false;

  SymP fail() {
    failed = true;
    return nullptr;
  }
  static SymP make(Sym::Kind k, Sym::Class c) {
    auto s = std::make_shared<Sym>();
    s->kind = k;
    s->cls = c;
    return s;
  }
  // value of an instruction of the entry computation
  SymP entry(const Instr* ins) {
    if (failed) return nullptr;
    if (members.count(ins)) {
      if (ins->opcode != "fusion" || ins->shape.is_tuple()) return fail();
      std::map<const Instr*, SymP> env;
      for (size_t i = 0; i < ins->operands.size(); ++i) {
        SymP v = entry(ins->operands[i]);
        if (!v) return fail();
        env[ins->called->params[i]] = v;
      }
      return inner(ins->called->root, env);
    }
    if (prog.storage_root(ins) == primary) return make(Sym::kX, Sym::kFull);
    if (ins->opcode == "constant") {
      if (ins->is_scalar_constant()) {
        auto s = make(Sym::kConst, Sym::kScalar);
        s->c = std::strtod(ins->literal.c_str(), nullptr);
        return s;
      }
      if (ins->shape.rank() == 1 && ins->shape.dims[0] == K) {
        auto s = make(Sym::kCol, Sym::kColumn);
        s->col = ins;
        return s;
      }
    }
    return fail();
  }
  SymP inner(const Instr* ins, std::map<const Instr*, SymP>& env) {
    if (failed) return nullptr;
    auto it = env.find(ins);
    if (it != env.end()) return it->second;
    const std::string& op = ins->opcode;
    SymP r;
    if (op == "parameter") return fail();   // every parameter is bound above
    if (op == "constant") {
      if (!ins->is_scalar_constant()) return fail();
      r = make(Sym::kConst, Sym::kScalar);
      r->c = std::strtod(ins->literal.c_str(), nullptr);
    } else if (op == "convert" || op == "bitcast" || op == "reshape" || op == "copy") {
      r = inner(ins->operands[0], env);
    } else if (op == "broadcast") {
      SymP k = inner(ins->operands[0], env);
      if (!k) return fail();
      const int rank_in = ins->operands[0]->shape.rank();
      if (rank_in == 0) r = k;
      else if (rank_in == 1 && ins->shape.rank() == 1 && k->cls != Sym::kFull) r = k;   // a splat written as [M] -> [M]
      else if (rank_in == 1 && ins->shape.rank() == 2 && ins->dimensions.size() == 1 &&
               ((k->cls == Sym::kRow && ins->dimensions[0] == 0) || (k->cls == Sym::kColumn && ins->dimensions[0] == 1) || k->cls == Sym::kScalar))
        r = k;
      else return fail();
    } else if (op == "reduce") {
      if (ins->operands.size() != 2 || ins->dimensions.size() != 1 || ins->operands[0]->shape.rank() != 2 || ins->dimensions[0] != 1) return fail();
      if (!ins->called || ins->called->root->opcode != "add") return fail();
      SymP init = inner(ins->operands[1], env);
      SymP x = inner(ins->operands[0], env);
      if (!init || !x || init->kind != Sym::kConst || init->c != 0.0) return fail();
      r = make(Sym::kRowSum, Sym::kRow);
      r->kids = {x};
    } else if (op == "add" || op == "subtract" || op == "multiply" || op == "divide") {
      SymP a = inner(ins->operands[0], env), b = inner(ins->operands[1], env);
      if (!a || !b) return fail();
      r = make(Sym::kOp, Sym::kScalar);
      r->op = op;
      r->kids = {a, b};
      if (a->cls == b->cls) r->cls = a->cls;
      else if (a->cls == Sym::kScalar) r->cls = b->cls;
      else if (b->cls == Sym::kScalar) r->cls = a->cls;
      else r->cls = Sym::kFull;
    } else if (op == "rsqrt") {
      SymP a = inner(ins->operands[0], env);
      if (!a) return fail();
      r = make(Sym::kOp, a->cls);
      r->op = op;
      r->kids = {a};
    } else {
      return fail();
    }
    if (r) env[ins] = r;
    return r;
  }
};

bool sym_equal(const SymP& a, const SymP& b) {
  if (a->kind != b->kind) return false;
  switch (a->kind) {
    case Sym::kX: return true;
    case Sym::kCol: return a->col == b->col;
    case Sym::kConst: return a->c == b->c;
    case Sym::kRowSum: return sym_equal(a->kids[0], b->kids[0]);
    case Sym::kOp:
      if (a->op != b->op || a->kids.size() != b->kids.size()) return false;
      if (a->kids.size() == 1) return sym_equal(a->kids[0], b->kids[0]);
      if (sym_equal(a->kids[0], b->kids[0]) && sym_equal(a->kids[1], b->kids[1])) return true;
      return (a->op == "add" || a->op == "multiply") && sym_equal(a->kids[0], b->kids[1]) && sym_equal(a->kids[1], b->kids[0]);
  }
  return false;
}

// s = op(p, q) with p satisfying `first` (either operand order when the operation commutes); p and q are returned
bool sym_split(const SymP& s, const char* op, const std::function<bool(const SymP&)>& first, SymP* p, SymP* q) {
  if (s->kind != Sym::kOp || s->op != op || s->kids.size() != 2) return false;
  const bool commutes = s->op == "add" || s->op == "multiply";
  for (int order = 0; order < (commutes ? 2 : 1); ++order) {
    const SymP& a = s->kids[order];
    const SymP& b = s->kids[1 - order];
    if (first(a)) {
      *p = a;
      *q = b;
      return true;
    }
  }
  return false;
}

// sum / K written as a product with 1/K or a quotient by K
bool sym_is_mean_of(const SymP& s, int64_t K, SymP* summed) {
  SymP c, rest;
  auto is_const = [](const SymP& v) { return v->kind == Sym::kConst; };
  if (sym_split(s, "multiply", is_const, &c, &rest) && std::fabs(c->c * static_cast<double>(K) - 1.0) < 1e-5 && rest->kind == Sym::kRowSum) {
    *summed = rest->kids[0];
    return true;
  }
  if (s->kind == Sym::kOp && s->op == "divide" && s->kids[1]->kind == Sym::kConst && s->kids[1]->c == static_cast<double>(K) && s->kids[0]->kind == Sym::kRowSum) {
    *summed = s->kids[0]->kids[0];
    return true;
  }
  return false;
}

bool match_layer_norm(const Program& prog, const std::vector<const Instr*>& row_members, const Instr* primary, const Instr* H, int64_t K, LayerNormMatch* out) {
  SymBuilder b{prog, std::set<const Instr*>(row_members.begin(), row_members.end()), primary, K};
  SymP y = b.entry(H);
  if (!y || b.failed) return false;
  auto is_col = [](const SymP& v) { return v->kind == Sym::kCol; };
  auto is_row = [](const SymP& v) { return v->cls == Sym::kRow; };
  auto is_const = [](const SymP& v) { return v->kind == Sym::kConst; };
  SymP beta, t, gamma, u, r, d;
  if (!sym_split(y, "add", is_col, &beta, &t)) return false;
  if (!sym_split(t, "multiply", is_col, &gamma, &u)) return false;
  if (!sym_split(u, "multiply", is_row, &r, &d)) return false;
  // d = x - mean(x)
  auto is_centred = [&](const SymP& v) {
    SymP summed;
    return v->kind == Sym::kOp && v->op == "subtract" && v->kids[0]->kind == Sym::kX && sym_is_mean_of(v->kids[1], K, &summed) && summed->kind == Sym::kX;
  };
  if (!is_centred(d)) return false;
  // r = rsqrt(mean(d * d) + eps)
  if (r->kind != Sym::kOp || r->op != "rsqrt") return false;
  SymP eps, var, sq;
  if (!sym_split(r->kids[0], "add", is_const, &eps, &var)) return false;
  if (!sym_is_mean_of(var, K, &sq)) return false;
  if (sq->kind != Sym::kOp || sq->op != "multiply" || !is_centred(sq->kids[0]) || !sym_equal(sq->kids[0], sq->kids[1]) || !sym_equal(sq->kids[0], d)) return false;
  if (!(eps->c > 0)) return false;
  out->gamma = gamma->col;
  out->beta = beta->col;
  out->eps = eps->c;
  return out->gamma->shape.dtype == DType::kF16 && out->beta->shape.dtype == DType::kF16;
}

}  // namespace

bool match_prologue_layer_norm(const Program& prog, const std::vector<const Instr*>& row_members, const Instr* H, int64_t M, int64_t K,
                               const Instr** gamma, const Instr** beta, double* eps) {
  const Instr* primary = prologue_primary(prog, row_members, M, K);
  if (!primary) return false;
  LayerNormMatch ln;
  if (!match_layer_norm(prog, row_members, primary, H, K, &ln)) return false;
  *gamma = ln.gamma;
  *beta = ln.beta;
  *eps = ln.eps;
  return true;
}

namespace {

Prologue build_prologue(const Program& prog, const std::vector<const Instr*>& row_members, const Instr* gi, const graph::GemmDesc& g,
                        const GemmTuning& t, const LaunchShape& ls, bool stores, PointerTable& ptrs, const graph::LayerNormFold* fold = nullptr,
                        int fold_stats_offset = 0, int fold_exchange_offset = 0) {
  (void)ls;
  RowInfo info = analyze_rows(row_members);
  MONONN_CHECK(info.row_program && info.rows == g.M && info.row_len == g.K && g.batch == 1, kUnsupported)
      << "GEMM prologue: the cluster is not a row program over the rows of the left operand";
  auto outs = external_outputs(prog, row_members);
  MONONN_CHECK(outs.size() == 1 && prog.storage_root(gi->operands[0]) == outs[0] && outs[0]->shape.dtype == DType::kF16 &&
                   outs[0]->shape.dims == std::vector<int64_t>({g.M, g.K}),
               kUnsupported)
      << "GEMM prologue: the row program must produce exactly the f16 [M,K] left operand";
  const Instr* H = outs[0];
  const int TM = t.bm / t.wm / 16, WK = t.wk, CH = static_cast<int>(g.K / 32 / WK);   // the wave's whole k range (one chunk)
  const Instr* primary = prologue_primary(prog, row_members, g.M, g.K);
  MONONN_CHECK(primary != nullptr, kUnsupported) << "GEMM prologue: no [M,K] f16 input to take the place of the left operand";
  Prologue out;
  out.primary = primary;
  const size_t first = ptrs.entries.size();
  CodeBuffer cb;
  VarTable vars;
  Emitter em(prog, row_members, cb, vars, ptrs);
  std::vector<int> vm(TM);
  for (int i = 0; i < TM; ++i) vm[i] = vars.add("m" + S(i), g.M);
  int vwk = vars.add("wk", WK);
  int vg = vars.add("g", 4);
  auto col_of = [&](int s, int e) {
    return LinExpr::variable(vwk, WK).scaled(32).plus(LinExpr::variable(vg, 4).scaled(8)).plus_const(static_cast<int64_t>(s) * WK * 32 + e);
  };
  auto primary_index = [&](int i, int s, int e) {
    Index idx;
    idx.push_back(LinExpr::variable(vm[i], g.M));
    idx.push_back(col_of(s, e));
    return idx;
  };
  auto operand_index = [&](const Instr* x, int i, int s, int e) {
    // rows of the operand = leading dims; all leading dims together are the row
    std::vector<int64_t> lead(x->shape.dims.begin(), x->shape.dims.end() - 1);
    Index idx = delinearize(LinExpr::variable(vm[i], g.M), lead, vars);
    idx.push_back(col_of(s, e));
    return idx;
  };
  cb.line("const int lane = mononn_dev::lane_id();");
  cb.line("const int r16 = lane & 15, g = lane >> 4;");
  for (int i = 0; i < TM; ++i) {
    cb.line("const bool mv" + S(i) + " = m_base + " + S(i * 16) + " + r16 < " + S(g.M) + ";");
    cb.line("const int m" + S(i) + " = mv" + S(i) + " ? m_base + " + S(i * 16) + " + r16 : " + S(g.M - 1) + ";");
  }
  auto bind_elem = [&](int i, int s, int e) { em.bind(primary, primary_index(i, s, e), "a[" + S(s) + "][" + S(i) + "][" + S(e) + "]"); };
  auto finish_struct = [&](const std::string& body, int smem_bytes) {
    out.smem = smem_bytes;
    for (auto& kv : em.literal_tables()) out.globals.push_back(kv.second);
    std::string st = std::string("struct @NAME@_pro {\n  static constexpr bool enabled = true;\n  static constexpr bool after_mfma = ") + (fold ? "true" : "false") + ";\n";
    for (size_t i = first; i < ptrs.entries.size(); ++i) {
      auto& e = ptrs.entries[i];
      st += std::string("  ") + (e.is_output ? "" : "const ") + hlo::dtype_ctype(e.dtype) + "* " + e.name + ";\n";
    }
    st += "  __device__ __forceinline__ void operator()(half8_t (&a)[" + S(CH) + "][" + S(TM) + "], int m_base, int wk, int mn_wave, bool store, int store_slot, char* smem) const {\n";
    std::istringstream is(body);
    std::string l;
    while (std::getline(is, l)) st += "  " + l + "\n";
    st += "  }\n};\n";
    out.struct_text = st;
    std::string init = "@NAME@_pro pro{";
    for (size_t i = first; i < ptrs.entries.size(); ++i) init += (i > first ? ", " : "") + ptrs.entries[i].name;
    init += "};";
    out.init_line = init;
  };
  // LayerNorm, laid out by hand: gamma / beta of the lane's columns requested first (16 bytes per k step each), the
  // sums of x and x * x in one pass over the fragments, one exchange across the 4 lanes of a row and (WK > 1) one
  // through LDS for both sums, then ((x - mean) * r) * gamma + beta as two fused multiply-adds per element.  The variance is
  // E[x^2] - mean^2 in fp32 (one exchange instead of two); the generic form computes the centred sum of squares.
  LayerNormMatch ln;
  if (fold) {
    // Folded LayerNorm: the fragments go into the MFMAs as they are.  This functor only computes the statistics of the
    // wave's rows (nothing after it waits for them before the epilogue, so they overlap the MFMAs), leaves them in LDS
    // for the epilogue, and - in the one GEMM that also owes the normalised rows to later stages - stores them, each
    // column tile taking the k steps s with s % tiles == its own number so that no workgroup carries all of it.
    char num[64];
    const int64_t tiles_n = (g.N + t.bn - 1) / t.bn;
    const int64_t ksteps = g.K / 32;
    const int64_t owners = std::min<int64_t>(tiles_n, ksteps);
    std::string pg, pb;
    if (stores) {
      pg = ptrs.input(fold->gamma);
      pb = ptrs.input(fold->beta);
      for (int s = 0; s < CH; ++s) {
        const std::string col = "(wk * 32 + g * 8 + " + S(static_cast<int64_t>(s) * WK * 32) + ")";
        cb.line("const bool own" + S(s) + " = store_slot >= 0 && (" + S(s * WK) + " + wk) % " + S(owners) + " == store_slot;");
        cb.line("half8_t gam" + S(s) + " = {}, bet" + S(s) + " = {};");
        cb.open("if (own" + S(s) + ")");
        cb.line("gam" + S(s) + " = *reinterpret_cast<const half8_t*>(" + pg + " + " + col + ");");
        cb.line("bet" + S(s) + " = *reinterpret_cast<const half8_t*>(" + pb + " + " + col + ");");
        cb.close();
      }
    }
    for (int i = 0; i < TM; ++i) {
      cb.line("float s1_" + S(i) + " = 0.f, s2_" + S(i) + " = 0.f;");
      for (int s = 0; s < CH; ++s)
        for (int p2 = 0; p2 < 4; ++p2) {
          const std::string h = "__builtin_shufflevector(a[" + S(s) + "][" + S(i) + "], a[" + S(s) + "][" + S(i) + "], " + S(2 * p2) + ", " + S(2 * p2 + 1) + ")";
          cb.line("s1_" + S(i) + " = __builtin_amdgcn_fdot2(" + h + ", half2_t{(_Float16)1, (_Float16)1}, s1_" + S(i) + ", false);");
          cb.line("s2_" + S(i) + " = __builtin_amdgcn_fdot2(" + h + ", " + h + ", s2_" + S(i) + ", false);");
        }
      for (int off : {16, 32}) {
        cb.line("s1_" + S(i) + " += __shfl_xor(s1_" + S(i) + ", " + S(off) + ", 64);");
        cb.line("s2_" + S(i) + " += __shfl_xor(s2_" + S(i) + ", " + S(off) + ", 64);");
      }
    }
    int smem_ln = 0;
    if (WK > 1) {
      cb.line("float* rb = reinterpret_cast<float*>(smem + " + S(fold_exchange_offset) + ") + mn_wave * " + S(TM * WK * 32) + ";");
      smem_ln = fold_exchange_offset + t.wm * t.wn * TM * WK * 32 * 4;
      cb.open("if (g == 0)");
      for (int i = 0; i < TM; ++i) {
        cb.line("rb[" + S(i * WK * 32) + " + wk * 32 + r16 * 2] = s1_" + S(i) + ";");
        cb.line("rb[" + S(i * WK * 32) + " + wk * 32 + r16 * 2 + 1] = s2_" + S(i) + ";");
      }
      cb.close();
      cb.line("__syncthreads();");
      for (int i = 0; i < TM; ++i) {
        cb.line("s1_" + S(i) + " = rb[" + S(i * WK * 32) + " + r16 * 2];");
        cb.line("s2_" + S(i) + " = rb[" + S(i * WK * 32) + " + r16 * 2 + 1];");
        for (int w = 1; w < WK; ++w) {
          cb.line("s1_" + S(i) + " += rb[" + S(i * WK * 32 + w * 32) + " + r16 * 2];");
          cb.line("s2_" + S(i) + " += rb[" + S(i * WK * 32 + w * 32) + " + r16 * 2 + 1];");
        }
      }
    } else {
      cb.line("__syncthreads();   // the previous unit's epilogue may still be reading the statistics");
    }
    MONONN_CHECK(fold_stats_offset >= smem_ln, kInternal) << "statistics of a folded LayerNorm overlap the exchange buffer";
    std::snprintf(num, sizeof num, "%.9g", 1.0 / static_cast<double>(g.K));
    const std::string inv_k = std::string(num) + "f";
    std::snprintf(num, sizeof num, "%.9g", fold->eps);
    std::string eps_lit = num;
    if (eps_lit.find_first_of(".e") == std::string::npos) eps_lit += ".0";
    eps_lit += "f";
    cb.line("float* ln_stats = reinterpret_cast<float*>(smem + " + S(fold_stats_offset) + ");");
    for (int i = 0; i < TM; ++i) {
      cb.line("const float mean" + S(i) + " = s1_" + S(i) + " * " + inv_k + ";");
      cb.line("const float rs" + S(i) + " = rsqrtf(fmaxf(s2_" + S(i) + " * " + inv_k + " - mean" + S(i) + " * mean" + S(i) + ", 0.f) + " + eps_lit + ");");
      cb.open("if (g == 0 && wk == 0)");
      cb.line("ln_stats[(m_base % " + S(t.bm) + " + " + S(i * 16) + " + r16) * 2] = mean" + S(i) + ";");
      cb.line("ln_stats[(m_base % " + S(t.bm) + " + " + S(i * 16) + " + r16) * 2 + 1] = rs" + S(i) + ";");
      cb.close();
    }
    cb.line("__syncthreads();");
    if (stores) {
      for (int i = 0; i < TM; ++i) {
        cb.line("const float nmr" + S(i) + " = -mean" + S(i) + " * rs" + S(i) + ";");
        for (int s = 0; s < CH; ++s) {
          LinExpr off = physical_offset(prog, H, primary_index(i, s, 0), &vars);
          cb.open("if (own" + S(s) + " && mv" + S(i) + ")");
          std::string arr = em.fresh("hn");
          cb.line("_Float16 " + arr + "[8];");
          cb.line("#pragma unroll");
          cb.open("for (int e = 0; e < 8; ++e)");
          cb.line(arr + "[e] = (_Float16)fmaf(fmaf((float)a[" + S(s) + "][" + S(i) + "][e], rs" + S(i) + ", nmr" + S(i) + "), (float)gam" + S(s) + "[e], (float)bet" + S(s) + "[e]);");
          cb.close();
          cb.line("mononn_dev::stN<_Float16, 8>(" + ptrs.output(H) + " + " + off.str(vars) + ", " + arr + ");");
          cb.close();
        }
      }
    }
    finish_struct(cb.text(), std::max(smem_ln, fold_stats_offset + t.bm * 8));
    return out;
  }
  if (match_layer_norm(prog, row_members, primary, H, g.K, &ln)) {
    const std::string pg = ptrs.input(ln.gamma), pb = ptrs.input(ln.beta);
    char num[64];
    for (int s = 0; s < CH; ++s) {
      const std::string col = "(wk * 32 + g * 8 + " + S(static_cast<int64_t>(s) * WK * 32) + ")";
      cb.line("const half8_t gam" + S(s) + " = *reinterpret_cast<const half8_t*>(" + pg + " + " + col + ");");
      cb.line("const half8_t bet" + S(s) + " = *reinterpret_cast<const half8_t*>(" + pb + " + " + col + ");");
    }
    for (int i = 0; i < TM; ++i) {
      // two elements per instruction and sum: v_dot2_f32_f16 (products and sums in fp32)
      cb.line("float s1_" + S(i) + " = 0.f, s2_" + S(i) + " = 0.f;");
      for (int s = 0; s < CH; ++s)
        for (int p2 = 0; p2 < 4; ++p2) {
          const std::string h = "__builtin_shufflevector(a[" + S(s) + "][" + S(i) + "], a[" + S(s) + "][" + S(i) + "], " + S(2 * p2) + ", " + S(2 * p2 + 1) + ")";
          cb.line("s1_" + S(i) + " = __builtin_amdgcn_fdot2(" + h + ", half2_t{(_Float16)1, (_Float16)1}, s1_" + S(i) + ", false);");
          cb.line("s2_" + S(i) + " = __builtin_amdgcn_fdot2(" + h + ", " + h + ", s2_" + S(i) + ", false);");
        }
      for (int off : {16, 32}) {
        cb.line("s1_" + S(i) + " += __shfl_xor(s1_" + S(i) + ", " + S(off) + ", 64);");
        cb.line("s2_" + S(i) + " += __shfl_xor(s2_" + S(i) + ", " + S(off) + ", 64);");
      }
    }
    int smem_ln = 0;
    if (WK > 1) {
      // [mn wave][row fragment][wk][16 rows][2 sums]
      cb.line("float* rb = reinterpret_cast<float*>(smem) + mn_wave * " + S(TM * WK * 32) + ";");
      smem_ln = t.wm * t.wn * TM * WK * 32 * 4;
      cb.open("if (g == 0)");
      for (int i = 0; i < TM; ++i) {
        cb.line("rb[" + S(i * WK * 32) + " + wk * 32 + r16 * 2] = s1_" + S(i) + ";");
        cb.line("rb[" + S(i * WK * 32) + " + wk * 32 + r16 * 2 + 1] = s2_" + S(i) + ";");
      }
      cb.close();
      cb.line("__syncthreads();");
      for (int i = 0; i < TM; ++i) {
        cb.line("s1_" + S(i) + " = rb[" + S(i * WK * 32) + " + r16 * 2];");
        cb.line("s2_" + S(i) + " = rb[" + S(i * WK * 32) + " + r16 * 2 + 1];");
        for (int w = 1; w < WK; ++w) {
          cb.line("s1_" + S(i) + " += rb[" + S(i * WK * 32 + w * 32) + " + r16 * 2];");
          cb.line("s2_" + S(i) + " += rb[" + S(i * WK * 32 + w * 32) + " + r16 * 2 + 1];");
        }
      }
    }
    std::snprintf(num, sizeof num, "%.9g", 1.0 / static_cast<double>(g.K));
    const std::string inv_k = std::string(num) + "f";
    std::snprintf(num, sizeof num, "%.9g", ln.eps);
    std::string eps_lit = num;
    if (eps_lit.find_first_of(".e") == std::string::npos) eps_lit += ".0";
    eps_lit += "f";
    for (int i = 0; i < TM; ++i) {
      cb.line("const float mean" + S(i) + " = s1_" + S(i) + " * " + inv_k + ";");
      cb.line("const float rs" + S(i) + " = rsqrtf(fmaxf(s2_" + S(i) + " * " + inv_k + " - mean" + S(i) + " * mean" + S(i) + ", 0.f) + " + eps_lit + ");");
      cb.line("const float nmr" + S(i) + " = -mean" + S(i) + " * rs" + S(i) + ";   // (x - mean) * r as one fused multiply-add");
      for (int s = 0; s < CH; ++s) {
        std::string arr = em.fresh("hn");
        cb.line("_Float16 " + arr + "[8];");
        cb.line("#pragma unroll");
        cb.open("for (int e = 0; e < 8; ++e)");
        cb.line(arr + "[e] = (_Float16)fmaf(fmaf((float)a[" + S(s) + "][" + S(i) + "][e], rs" + S(i) + ", nmr" + S(i) + "), (float)gam" + S(s) + "[e], (float)bet" + S(s) + "[e]);");
        cb.close();
        cb.line("a[" + S(s) + "][" + S(i) + "] = half8_t{" + arr + "[0], " + arr + "[1], " + arr + "[2], " + arr + "[3], " + arr + "[4], " + arr + "[5], " + arr + "[6], " + arr + "[7]};");
        if (stores) {
          LinExpr off = physical_offset(prog, H, primary_index(i, s, 0), &vars);
          cb.line("if (store && mv" + S(i) + ") mononn_dev::stN<_Float16, 8>(" + ptrs.output(H) + " + " + off.str(vars) + ", " + arr + ");");
        }
      }
    }
    finish_struct(cb.text(), smem_ln);
    return out;
  }
  auto reduces = em.collect_reduces();
  std::vector<std::vector<std::string>> reduce_accs_;   // [reduce][row fragment]
  int smem = 0;
  for (size_t ri = 0; ri < reduces.size(); ++ri) {
    const Instr* red = reduces[ri];
    std::string Tn = hlo::dtype_ctype(red->shape.dtype);
    MONONN_CHECK(hlo::dtype_bytes(red->shape.dtype) <= 8, kUnsupported) << "reduction type too wide";
    std::vector<std::string> accs;
    for (int i = 0; i < TM; ++i) {
      // earlier reductions of this row fragment are available to the operand of this one
      for (size_t pj = 0; pj < ri; ++pj)
        em.bind(reduces[pj], delinearize(LinExpr::variable(vm[i], g.M), reduces[pj]->shape.dims, vars), reduce_accs_[pj][i]);
      std::string acc = em.fresh("red");
      accs.push_back(acc);
      cb.line(Tn + " " + acc + " = " + em.value(red->operands[1], {}) + ";");
      for (int s = 0; s < CH; ++s)
        for (int e = 0; e < 8; ++e) {
          bind_elem(i, s, e);
          std::string val = em.value(red->operands[0], operand_index(red->operands[0], i, s, e));
          cb.line(acc + " = (" + Tn + ")" + Emitter::reducer_expr(red, acc, val) + ";");
        }
      for (int off : {16, 32}) {
        std::string other = "__shfl_xor(" + acc + ", " + S(off) + ", 64)";
        cb.line(acc + " = (" + Tn + ")" + Emitter::reducer_expr(red, acc, other) + ";");
      }
    }
    if (WK > 1) {
      // [mn wave][row fragment][wk][16 rows]
      std::string buf = em.fresh("rb");
      cb.line(Tn + "* " + buf + " = reinterpret_cast<" + Tn + "*>(smem + " + S(smem) + ") + mn_wave * " + S(TM * WK * 16) + ";");
      smem += t.wm * t.wn * TM * WK * 16 * 8;
      for (int i = 0; i < TM; ++i) cb.line("if (g == 0) " + buf + "[" + S(i * WK * 16) + " + wk * 16 + r16] = " + accs[i] + ";");
      cb.line("__syncthreads();");
      for (int i = 0; i < TM; ++i) {
        cb.line(accs[i] + " = " + buf + "[" + S(i * WK * 16) + " + r16];");
        for (int w = 1; w < WK; ++w)
          cb.line(accs[i] + " = (" + Tn + ")" + Emitter::reducer_expr(red, accs[i], buf + "[" + S(i * WK * 16 + w * 16) + " + r16]") + ";");
      }
    }
    reduce_accs_.push_back(accs);   // bound per row fragment where the results are consumed
  }
  // results replace the fragments
  for (int i = 0; i < TM; ++i) {
    for (size_t ri = 0; ri < reduces.size(); ++ri) {
      Index ridx;
      const Instr* red = reduces[ri];
      ridx = delinearize(LinExpr::variable(vm[i], g.M), red->shape.dims, vars);
      em.bind(red, ridx, reduce_accs_[ri][i]);
    }
    for (int s = 0; s < CH; ++s) {
      std::vector<std::string> vals;
      for (int e = 0; e < 8; ++e) {
        bind_elem(i, s, e);
        vals.push_back(em.value(em.resolve_output(H), primary_index(i, s, e)));
      }
      std::string arr = em.fresh("hn");
      std::string init;
      for (int e = 0; e < 8; ++e) init += (e ? ", " : "") + vals[e];
      cb.line("const _Float16 " + arr + "[8] = {" + init + "};");
      cb.line("a[" + S(s) + "][" + S(i) + "] = half8_t{" + arr + "[0], " + arr + "[1], " + arr + "[2], " + arr + "[3], " + arr + "[4], " + arr + "[5], " + arr + "[6], " + arr + "[7]};");
      if (stores) {
        LinExpr off = physical_offset(prog, H, primary_index(i, s, 0), &vars);
        cb.line("if (store && mv" + S(i) + ") mononn_dev::stN<_Float16, 8>(" + ptrs.output(H) + " + " + off.str(vars) + ", " + arr + ");");
      }
    }
  }
  em.unbind(primary);
  out.smem = smem;
  for (auto& kv : em.literal_tables()) out.globals.push_back(kv.second);
  std::string st = "struct @NAME@_pro {\n  static constexpr bool enabled = true;\n  static constexpr bool after_mfma = false;\n";
  for (size_t i = first; i < ptrs.entries.size(); ++i) {
    auto& e = ptrs.entries[i];
    st += std::string("  ") + (e.is_output ? "" : "const ") + hlo::dtype_ctype(e.dtype) + "* " + e.name + ";\n";
  }
  st += "  __device__ __forceinline__ void operator()(half8_t (&a)[" + S(CH) + "][" + S(TM) + "], int m_base, int wk, int mn_wave, bool store, int store_slot, char* smem) const {\n";
  {
    // every operand of the row program is requested before the first of them is used: one trip to memory
    std::istringstream is(hoist_row_loads(cb.text(), true));
    std::string l;
    while (std::getline(is, l)) st += "  " + l + "\n";
  }
  st += "  }\n};\n";
  out.struct_text = st;
  std::string init = "@NAME@_pro pro{";
  for (size_t i = first; i < ptrs.entries.size(); ++i) init += (i > first ? ", " : "") + ptrs.entries[i].name;
  init += "};";
  out.init_line = init;
  return out;
}

NodeFunction gen_gemm(const Program& prog, const std::vector<const Instr*>& members, const std::vector<const Instr*>& outputs,
                      const graph::GemmDesc& g, const LaunchShape& ls, const GemmTuning& t,
                      const std::vector<const Instr*>& prologue = {}, bool prologue_stores = false, const graph::LayerNormFold* fold = nullptr) {
  const Instr* gi = members[0];
  if (fold && !fold->on()) fold = nullptr;
  // LDS of a folded LayerNorm: the statistics of the workgroup's rows live behind the slabs of the k-slice reduction
  // and behind the exchange of the sums, which itself sits behind the slabs: a wave that is first into the next unit
  // writes its sums while slower waves still read the slabs of this one
  int fold_stats_offset = 0, fold_exchange_offset = 0;
  if (fold) {
    const int tm16 = t.bm / t.wm / 16, tn16 = t.bn / t.wn / 16;
    const int red = t.wk > 1 ? ls.waves() * tm16 * tn16 * 64 * 16 : 0;
    const int rb = t.wk > 1 ? t.wm * t.wn * tm16 * t.wk * 32 * 4 : 0;
    fold_exchange_offset = (red + 15) / 16 * 16;
    fold_stats_offset = (fold_exchange_offset + rb + 15) / 16 * 16;
  }
  const bool mfma = gemm_uses_mfma(g);
  bool has_pro = !prologue.empty();
  MONONN_CHECK(!has_pro || mfma, kUnsupported) << gi->hlo_name << ": a row-program prologue needs the MFMA path";
  // A folded LayerNorm on the LDS-staged tile: no row program runs at all, the tile itself adds up the row sums of
  // the fragments it multiplies (mononn_dev::gemm_tile_lds, LN_STATS); the statistics live behind the operand
  // buffers and the rows of the epilogue.  Where later stages read the normalised rows (prologue_stores), the column
  // tiles of a row block store a share of them each, from the statistics and a second look at the operand rows.
  const bool lds_fold = fold && has_pro && t.stages >= 2;
  const Instr* lds_fold_primary = nullptr;
  if (lds_fold) {
    MONONN_CHECK(g.split_k <= 1 && !g.bf16 && !g.is_conv, kSpecError) << gi->hlo_name << ": a folded LayerNorm needs the whole k range in one f16 GEMM";
    lds_fold_primary = prologue_primary(prog, prologue, g.M, g.K);
    MONONN_CHECK(lds_fold_primary != nullptr, kUnsupported) << gi->hlo_name << ": no [M,K] f16 input to take the place of the left operand";
    has_pro = false;
    const int rows_bytes = ls.waves() * 32 * (t.bn / t.wn + 4) * 4;
    fold_stats_offset = (std::max(2 * (t.bm + t.bn) * t.bk * 2, rows_bytes) + 15) / 16 * 16;
  }
  if (mfma) validate_gemm_tuning(g, ls, t, has_pro);
  PointerTable ptrs;
  // the two operands come first in the pointer list; with a prologue the left operand is the row
  // program's input, whose rows are normalised on the way into the MFMAs
  Prologue pro;
  std::string pa, pb;
  std::vector<const Instr*> epi_outputs = outputs;
  if (has_pro) {
    // find the primary input first (the pointer order must start with the operand the GEMM loads)
    PointerTable probe_ptrs;
    Prologue probe = build_prologue(prog, prologue, gi, g, t, ls, false, probe_ptrs, fold, fold_stats_offset, fold_exchange_offset);
    pa = ptrs.input(probe.primary);
    pb = ptrs.input(prog.storage_root(gi->operands[1]));
    pro = build_prologue(prog, prologue, gi, g, t, ls, prologue_stores, ptrs, fold, fold_stats_offset, fold_exchange_offset);
    auto pouts = external_outputs(prog, prologue);
    epi_outputs.clear();
    for (auto* o : outputs)
      if (std::find(pouts.begin(), pouts.end(), o) == pouts.end()) epi_outputs.push_back(o);
  } else {
    pa = ptrs.input(lds_fold ? lds_fold_primary : prog.storage_root(gi->operands[0]));
    pb = ptrs.input(prog.storage_root(gi->operands[1]));
    if (lds_fold) {
      auto pouts = external_outputs(prog, prologue);
      epi_outputs.clear();
      for (auto* o : outputs)
        if (std::find(pouts.begin(), pouts.end(), o) == pouts.end()) epi_outputs.push_back(o);
    }
  }
  // rows of a LayerNorm folded into an LDS-staged tile, for the stages that read them: ((x - mean) * r) * gamma + beta
  // as two fused multiply-adds per element, like the folded direct tile stores them
  std::string rows_struct, rows_init;
  if (lds_fold && prologue_stores) {
    auto pouts = external_outputs(prog, prologue);
    MONONN_CHECK(pouts.size() == 1 && pouts[0]->shape.dtype == DType::kF16 && pouts[0]->shape.dims == std::vector<int64_t>({g.M, g.K}), kUnsupported)
        << gi->hlo_name << ": the folded LayerNorm must produce exactly the f16 [M,K] rows";
    const Instr* H = pouts[0];
    VarTable rv;
    const int vm = rv.add("m", g.M), vr = rv.add("run", g.K / 8);
    Index idx;
    idx.push_back(LinExpr::variable(vm, g.M));
    idx.push_back(LinExpr::variable(vr, g.K / 8).scaled(8));
    const LinExpr off = physical_offset(prog, H, idx, &rv);
    const std::string pg = ptrs.input(fold->gamma), pbt = ptrs.input(fold->beta), ph = ptrs.output(H);
    rows_struct = "struct @NAME@_rows {\n  static constexpr bool enabled = true;\n  const _Float16* gamma;\n  const _Float16* beta;\n  _Float16* out;\n"
                  "  __device__ __forceinline__ void operator()(int m, int k, half8_t x, float mean, float rs) const {\n"
                  "    const int run = k >> 3;\n"
                  "    const half8_t gam = *reinterpret_cast<const half8_t*>(gamma + k), bet = *reinterpret_cast<const half8_t*>(beta + k);\n"
                  "    const float nmr = -mean * rs;\n"
                  "    _Float16 hn[8];\n"
                  "#pragma unroll\n"
                  "    for (int e = 0; e < 8; ++e) hn[e] = (_Float16)fmaf(fmaf((float)x[e], rs, nmr), (float)gam[e], (float)bet[e]);\n"
                  "    mononn_dev::stN<_Float16, 8>(out + " + off.str(rv) + ", hn);\n"
                  "  }\n};\n";
    rows_init = "@NAME@_rows rows{" + pg + ", " + pbt + ", " + ph + "};";
  }
  const size_t first_epi = ptrs.entries.size();   // 1 when both operands are the same buffer
  if (g.bf16) {
    // the tiles move operands as 16-byte pieces whatever the 2-byte type; only the MFMA differs (last template argument)
    MONONN_CHECK(!has_pro && !fold, kUnsupported) << gi->hlo_name << ": bf16 GEMMs take no row-program prologue";
    if (mfma) {
      pa = "reinterpret_cast<const half_t*>(" + pa + ")";
      pb = "reinterpret_cast<const half_t*>(" + pb + ")";
    }
  }
  std::vector<const Instr*> cluster_members(members.begin() + 1, members.end());
  Epilogue epi;
  {
    // both orientations of the accumulator tile are generated; rows-per-lane wins when it packs more stores
    PointerTable p_n = ptrs;
    epi = build_epilogue(prog, gi, cluster_members, epi_outputs, g, mfma, p_n, first_epi, false, fold, t.bm);
    bool use_m = false;
    if (mfma && g.split_k <= 1 && !g.is_conv && g.M % 4 == 0) {
      try {
        PointerTable p_m = ptrs;
        Epilogue e_m = build_epilogue(prog, gi, cluster_members, epi_outputs, g, mfma, p_m, first_epi, true, fold, t.bm);
        if (e_m.vector_stores > epi.vector_stores) {
          epi = std::move(e_m);
          ptrs = std::move(p_m);
          use_m = true;
        }
      } catch (const Error& e) {
        if (e.code() != kUnsupported) throw;
      }
    }
    if (!use_m) ptrs = std::move(p_n);
  }
  CodeBuffer fb;
  std::string conv_struct, preload_body;
  bool preload = false, rows_lds = false;
  int preload_regs = 0;
  if (g.split_k <= 1) fb.line(epi.init_line);
  if (fold) fb.line("epi.ln_stats = reinterpret_cast<const float*>(smem + " + S(fold_stats_offset) + ");");
  if (has_pro) fb.line(pro.init_line);
  if (!rows_struct.empty()) fb.line(rows_init);
  int64_t units = 0;
  int smem = 0;
  if (mfma) {
    // Unit order: the workgroups that read the same columns of B (same tile_n, all tile_m) differ by
    // multiples of 8 in their unit index; with units dealt round-robin over the 8 XCDs they land on
    // one XCD and share its L2.  tile_n = 8 * (q / tiles_m) + u % 8, tile_m = q % tiles_m, q = u / 8.
    const int64_t tiles_m = (g.M + t.bm - 1) / t.bm, tiles_n = (g.N + t.bn - 1) / t.bn;
    const int S_ = std::max(1, g.split_k);
    const int64_t KS = g.K / S_;   // k extent of one split
    const int64_t per_batch = tiles_n * tiles_m * S_;
    units = g.batch * per_batch;
    // Regional synchronisation: unit 8 q + x belongs to XCD x, which takes its slice of the columns or its k slice
    const Partition& part = t.part;
    if (part.on()) {
      MONONN_CHECK(g.batch == 1 && !g.is_conv && t.stages < 2 && part.parts <= 8, kInternal) << gi->hlo_name << ": GEMM cannot be dealt to the XCDs";
      MONONN_CHECK(part.kind == Partition::kSplitK ? S_ == part.parts : (part.kind == Partition::kColumns && S_ == 1 && tiles_n % part.parts == 0 && g.N % t.bn == 0), kInternal)
          << gi->hlo_name << ": partition does not fit the tile grid";
      units = 8 * (part.kind == Partition::kSplitK ? tiles_n * tiles_m : tiles_n / part.parts * tiles_m);
      fb.line("const int bidx = 0;");
      fb.line("const int xcd = unit & 7;   // of " + S(part.parts) + " that take part");
      fb.line(std::string("const int ksplit = ") + (part.kind == Partition::kSplitK ? "xcd" : "0") + ";");
      fb.line("const int rem = unit >> 3;");
    } else {
    fb.line("const int bidx = unit / " + S(per_batch) + ";");
    fb.line("const int rem0 = unit % " + S(per_batch) + ";");
    fb.line("const int ksplit = rem0 % " + S(S_) + ";");
    fb.line("const int rem = rem0 / " + S(S_) + ";");
    }
    if (g.split_k > 1) fb.line(epi.init_line);
    // LDS-staged tiles (large problems): the 8 XCDs each take a rectangle of the tile grid, rm x rn tiles, walked
    // row by row, so that the tiles an XCD works on at one time share few operand panels: every panel an XCD
    // touches comes over the fabric once per XCD, and with a strip of single columns (below) the left operand
    // would cross it once per XCD for every tile column.  The split of the grid into gm x gn rectangles is the
    // one with the fewest panel bytes per XCD.
    int gm = 0, gn = 0;
    if (t.stages >= 2 && S_ == 1) {
      int64_t best = -1;
      for (int a : {1, 2, 4, 8}) {
        const int b = 8 / a;
        if (tiles_m % a || tiles_n % b) continue;
        const int64_t cost = tiles_m / a * t.bm + tiles_n / b * t.bn;
        if (best < 0 || cost < best) best = cost, gm = a, gn = b;
      }
    }
    if (part.kind == Partition::kColumns) {
      fb.line("const int tile_n = xcd * " + S(tiles_n / part.parts) + " + rem / " + S(tiles_m) + ";");
      fb.line("const int tile_m = rem % " + S(tiles_m) + ";");
    } else if (gm > 0) {
      const int64_t rn = tiles_n / gn, rm = tiles_m / gm;
      fb.line("const int xcd = rem & 7, q = rem >> 3;   // " + S(rm) + " x " + S(rn) + " tiles per XCD");
      fb.line("const int tile_n = (xcd / " + S(gm) + ") * " + S(rn) + " + q % " + S(rn) + ";");
      fb.line("const int tile_m = (xcd % " + S(gm) + ") * " + S(rm) + " + q / " + S(rn) + ";");
    } else if (tiles_n % 8 == 0 && S_ == 1) {
      fb.line("const int tile_n = (rem >> 3) / " + S(tiles_m) + " * 8 + (rem & 7);");
      fb.line("const int tile_m = (rem >> 3) % " + S(tiles_m) + ";");
    } else {
      fb.line("const int tile_n = rem / " + S(tiles_m) + ";");
      fb.line("const int tile_m = rem % " + S(tiles_m) + ";");
    }
    std::ostringstream call;
    if (g.is_conv) {
      MONONN_CHECK(!has_pro && S_ == 1, kUnsupported) << gi->hlo_name << ": a convolution takes neither a row-program prologue nor split-K";
      const hlo::ConvConfig& c = g.conv;
      std::ostringstream am;
      am << "struct @NAME@_amap {\n  static constexpr bool kRowMajor = false;\n"
         << "  __device__ __forceinline__ const half_t* operator()(const half_t* in, int m, int k, int) const {\n"
         << "    const int n = m / " << c.P * c.Q << ", pq = m % " << c.P * c.Q << ", p = pq / " << c.Q << ", q = pq % " << c.Q << ";\n"
         << "    const int r = k / " << c.S * c.C << ", sc = k % " << c.S * c.C << ";\n"
         << "    return in + (((long)n * " << c.H << " + p * " << c.stride_h << " + r) * " << c.W << " + q * " << c.stride_w << ") * " << c.C << " + sc;\n"
         << "  }\n};\n";
      conv_struct = am.str();
      if (t.stages >= 2)
        call << "mononn_dev::gemm_tile_lds<" << t.bm << ", " << t.bn << ", " << t.wm << ", " << t.wn << ", " << KS << ", " << g.K << ", false, false, false, "
             << t.bk << ", @NAME@_epi, @NAME@_amap" << (g.bf16 ? ", true" : "") << ">(" << pa << ", " << pb << ", " << g.M << ", " << g.N << ", " << g.K << ", " << g.K
             << ", bidx, tile_m, tile_n, epi, smem, @NAME@_amap());";
      else
        call << "mononn_dev::gemm_tile<" << t.bm << ", " << t.bn << ", " << t.wm << ", " << t.wn << ", " << t.wk << ", " << KS << ", false, " << g.K
             << ", @NAME@_epi, mononn_dev::NoPrologue, @NAME@_amap" << (g.bf16 ? ", false, mononn_dev::NoPreB, false, false, false, true" : "") << ">(" << pa << ", " << pb << ", " << g.M << ", " << g.N << ", " << g.K << ", " << g.K
             << ", bidx, tile_m, tile_n, epi, smem, mononn_dev::NoPrologue(), @NAME@_amap());";
    } else {
      std::ostringstream b_expr;
      const bool b_along_n = !g.b_k_contig && !g.b_packed;
      b_expr << pb << " + (long)bidx * " << g.b_batch_stride << " + ksplit * " << (g.b_packed ? KS / 32 * 512 : b_along_n ? KS * g.N : KS);
      preload = t.preload_b && g.b_packed && t.stages < 2;
      if (g.f32)
        call << "mononn_dev::gemm_tile_f32<" << t.bm << ", " << t.bn << ", " << t.wm << ", " << t.wn << ", " << g.K << ", " << (b_along_n ? "true" : "false") << ", "
             << (epi.along_m ? "true" : "false") << ", @NAME@_epi>(" << pa << " + (long)bidx * " << g.a_batch_stride << ", " << pb << " + (long)bidx * " << g.b_batch_stride
             << ", " << g.M << ", " << g.N << ", " << g.K << ", " << (b_along_n ? g.N : g.K) << ", bidx, tile_m, tile_n, epi";
      else if (t.stages >= 2) {
        // results stored row-major go through LDS a fragment row at a time, so that the epilogue's stores and operand
        // loads cover whole rows of the wave's tile (results in fragment order are written in 8-byte pieces of
        // different 16-byte runs either way)
        // (a result in fragment order is already written as runs of 256 contiguous bytes per instruction; dealt out in
        // that order through LDS it came out slower)
        rows_lds = !epi.along_m && !epi_outputs.empty();
        for (auto* o : epi_outputs) rows_lds = rows_lds && !prog.physical_tile.count(prog.storage_root(o)) && !prog.physical_perm.count(prog.storage_root(o));
        call << "mononn_dev::gemm_tile_lds<" << t.bm << ", " << t.bn << ", " << t.wm << ", " << t.wn << ", " << KS << ", " << g.K << ", "
             << (g.a_packed ? "true" : "false") << ", " << (g.b_packed ? "true" : "false") << ", " << (epi.along_m ? "true" : "false") << ", " << t.bk
             << ", @NAME@_epi"
             << (g.bf16 || rows_lds || lds_fold ? std::string(", mononn_dev::RowMajorA, ") + (g.bf16 ? "true" : "false") + (rows_lds || lds_fold ? (rows_lds ? ", true" : ", false") : "") + (lds_fold ? ", true" : "") +
                                                      (!rows_struct.empty() ? ", @NAME@_rows" : "")
                                                : std::string())
             << ">(" << pa << " + (long)bidx * " << g.a_batch_stride << " + ksplit * " << (g.a_packed ? KS / 32 * 512 : KS) << ", "
             << b_expr.str() << ", " << g.M << ", " << g.N << ", " << g.K << ", " << g.K << ", bidx, tile_m, tile_n, epi, smem";
        if (lds_fold) {
          char eps[48];
          std::snprintf(eps, sizeof eps, "%.9gf", fold->eps);
          std::string e = eps;
          if (e.find_first_of(".e") == std::string::npos) e.insert(e.size() - 1, ".0");
          call << ", mononn_dev::RowMajorA(), " << e << ", reinterpret_cast<float*>(smem + " << fold_stats_offset << ")";
          if (!rows_struct.empty()) call << ", rows, " << tiles_n;
        }
      } else
        call << "mononn_dev::gemm_tile<" << t.bm << ", " << t.bn << ", " << t.wm << ", " << t.wn << ", " << t.wk << ", " << KS << ", "
             << (g.b_packed ? "true" : "false") << ", " << g.K << ", @NAME@_epi, " << (has_pro ? "@NAME@_pro" : "mononn_dev::NoPrologue")
             << ", mononn_dev::RowMajorA, " << (preload ? "true, @NAME@_preb" : "false, mononn_dev::NoPreB") << ", " << (g.a_packed ? "true" : "false") << ", "
             << (epi.along_m ? "true" : "false") << ", " << (b_along_n ? "true" : "false") << (g.bf16 || !g.a_k_contig ? (g.bf16 ? ", true" : ", false") : "")
             << (!g.a_k_contig ? ", true" : "") << ">("
             << pa << " + (long)bidx * " << g.a_batch_stride << " + ksplit * " << (g.a_packed ? KS / 32 * 512 : g.a_k_contig ? KS : KS * g.M) << ", " << b_expr.str() << ", " << g.M
             << ", " << g.N << ", " << (g.a_k_contig ? g.K : g.M) << ", " << (b_along_n ? g.N : g.K) << ", bidx, tile_m, tile_n, epi, smem, " << (has_pro ? "pro" : "mononn_dev::NoPrologue()")
             << ", mononn_dev::RowMajorA()" << (preload ? ", &pre_b" : "");
      call << ");";
      if (preload) {
        // the companion repeats the unit decoding as far as the right operand needs it
        const int TM = t.bm / t.wm / 16, TN = t.bn / t.wn / 16;
        const int my_steps = static_cast<int>((KS / 32 + t.wk - 1) / t.wk);
        const int chunk = TM * TN > 32 ? ls.chunk_fragments() / 2 : ls.chunk_fragments();
        const int ch_max = chunk / (TM + TN) > 0 ? chunk / (TM + TN) : 1;   // mirrors mononn_dev::gemm_chunk_steps
        preload_regs = (my_steps * (TM + TN) <= ls.whole_range_fragments() ? my_steps : std::min(my_steps, ch_max)) * TN;
        CodeBuffer pf;
        if (part.on()) {
          pf.line("const int bidx = 0;");
          pf.line("const int xcd = unit & 7;");
          pf.line(std::string("const int ksplit = ") + (part.kind == Partition::kSplitK ? "xcd" : "0") + ";");
          pf.line("const int rem = unit >> 3;");
        } else {
        pf.line("const int bidx = unit / " + S(per_batch) + ";");
        pf.line("const int rem0 = unit % " + S(per_batch) + ";");
        pf.line("const int ksplit = rem0 % " + S(S_) + ";");
        pf.line("const int rem = rem0 / " + S(S_) + ";");
        }
        if (part.kind == Partition::kColumns) pf.line("const int tile_n = xcd * " + S(tiles_n / part.parts) + " + rem / " + S(tiles_m) + ";");
        else if (tiles_n % 8 == 0 && S_ == 1) pf.line("const int tile_n = (rem >> 3) / " + S(tiles_m) + " * 8 + (rem & 7);");
        else pf.line("const int tile_n = rem / " + S(tiles_m) + ";");
        std::ostringstream pc;
        pc << "mononn_dev::gemm_b_preload<" << t.bm << ", " << t.bn << ", " << t.wm << ", " << t.wn << ", " << t.wk << ", " << KS << ", " << g.K << ">("
           << b_expr.str() << ", " << g.N << ", tile_n, pre_b);";
        pf.line(pc.str());
        preload_body = pf.text();
      }
    }
    fb.line(call.str());
    if (t.wk > 1) smem = ls.waves() * (t.bm / t.wm / 16) * (t.bn / t.wn / 16) * 64 * 16;
    if (t.stages >= 2) smem = std::max(2 * (t.bm + t.bn) * t.bk * 2, rows_lds ? ls.waves() * 32 * (t.bn / t.wn + 4) * 4 : 0);
    if (lds_fold) smem = fold_stats_offset + t.bm * 8;
    smem = std::max(smem, pro.smem);
  } else {
    const int64_t total = g.batch * g.M * g.N;
    units = (total + ls.block_size - 1) / ls.block_size;
    fb.line("const long e = (long)unit * " + S(ls.block_size) + " + threadIdx.x;");
    fb.open("if (e < " + S(total) + "L)");
    fb.line("const int bidx = (int)(e / " + S(g.M * g.N) + ");");
    fb.line("const int m = (int)((e / " + S(g.N) + ") % " + S(g.M) + ");");
    fb.line("const int n = (int)(e % " + S(g.N) + ");");
    std::ostringstream call;
    if (g.is_conv) {
      const hlo::ConvConfig& c = g.conv;
      call << "mononn_dev::conv_naive_element(" << pa << ", " << pb << ", " << c.H << ", " << c.W << ", " << c.C << ", " << c.R << ", " << c.S << ", "
           << c.P << ", " << c.Q << ", " << c.stride_h << ", " << c.stride_w << ", " << c.pad_h << ", " << c.pad_w << ", m, n, epi);";
    } else {
      call << "mononn_dev::gemm_naive_element(" << pa << " + (long)bidx * " << g.a_batch_stride << ", " << pb << " + (long)bidx * "
           << g.b_batch_stride << ", " << g.K << ", " << (g.a_k_contig ? g.K : 1) << ", " << (g.a_k_contig ? 1 : g.M) << ", "
           << (g.b_k_contig ? 1 : g.N) << ", " << (g.b_k_contig ? g.K : 1) << ", bidx, m, n, epi);";
    }
    fb.line(call.str());
    fb.close();
  }
  std::vector<std::string> globals = epi.globals;
  for (auto& gl : pro.globals) globals.push_back(gl);
  NodeFunction f = finish(fb.text(), ptrs, globals, units, smem, pro.struct_text + rows_struct + epi.struct_text + conv_struct);
  f.write_maps = epi.writes;
  if (preload) {
    const std::string tail = ", char* smem) {";
    size_t at = f.text.find(tail);
    MONONN_CHECK(at != std::string::npos, kInternal) << "node function signature not found";
    f.text.replace(at, tail.size(), ", char* smem, const @NAME@_preb& pre_b) {");
    f.text = "typedef mononn_dev::PreB<" + S(preload_regs) + "> @NAME@_preb;\n" + f.text;
    std::string sig = signature(ptrs.entries);
    sig = sig.substr(0, sig.rfind(", char* smem"));
    f.preload_text = "__device__ __forceinline__ void @NAME@_pre(" + sig + ", @NAME@_preb& pre_b) {\n" + preload_body + "}\n";
  }
  return f;
}

// Output projection inside the attention node: the context of batch element bidx = (b, h), rows m, columns n must be
// exactly element (b * M + m, h * N2 + n) of the projection's left operand, moved there by the epilogue clusters
// without any arithmetic.  Proven on the code generator itself: the second GEMM's value is bound to a register at
// (bidx, m, n) and the left operand is requested at the expected place; it must come back as that register.
void check_out_proj_mapping(const Program& prog, const Instr* g2, const graph::GemmDesc& d2, const std::vector<const Instr*>& epi_members,
                            const Instr* g3, const graph::GemmDesc& d3, int heads) {
  MONONN_CHECK(heads >= 1 && d2.batch % heads == 0 && d3.K == heads * d2.N && d3.M == d2.batch / heads * d2.M, kUnsupported)
      << g3->hlo_name << ": not a projection of merged heads";
  MONONN_CHECK(d2.N % 32 == 0 && d3.N % 16 == 0 && d3.a_k_contig && d3.batch == 1, kUnsupported) << g3->hlo_name << ": projection extents do not fit MFMA steps";
  const Instr* c = nullptr;   // entry-level value whose storage the projection reads
  for (auto* o : external_outputs(prog, [&] {
         std::vector<const Instr*> tail{g2};
         tail.insert(tail.end(), epi_members.begin(), epi_members.end());
         return tail;
       }()))
    if (prog.storage_root(g3->operands[0]) == o) c = o;
  MONONN_CHECK(c != nullptr && c != g2, kUnsupported) << g3->hlo_name << ": left operand is not the merged context";
  CodeBuffer scratch;
  VarTable vars;
  PointerTable ptrs;
  Emitter em(prog, epi_members, scratch, vars, ptrs);
  int vb = vars.add("bidx", d2.batch), vm = vars.add("m", d2.M), vn = vars.add("n", d2.N);
  const hlo::Shape& D2 = g2->shape;
  Index gidx = delinearize(LinExpr::variable(vb, d2.batch), std::vector<int64_t>(D2.dims.begin(), D2.dims.end() - 2), vars);
  gidx.push_back(LinExpr::variable(vm, d2.M));
  gidx.push_back(LinExpr::variable(vn, d2.N));
  em.bind(g2, gidx, "GV");
  Index bh = delinearize(LinExpr::variable(vb, d2.batch), {d2.batch / heads, static_cast<int64_t>(heads)}, vars);
  LinExpr lin = linearize({bh[0], LinExpr::variable(vm, d2.M), bh[1], LinExpr::variable(vn, d2.N)}, {d2.batch / heads, d2.M, static_cast<int64_t>(heads), d2.N});
  std::string v = em.value(em.resolve_output(c), delinearize(lin, c->shape.dims, vars));
  MONONN_CHECK(v == "GV", kUnsupported) << g3->hlo_name << ": the clusters between the attention and the projection do more than move data";
}

// The row program between the two contractions of an attention node is straight-line code per query row block.  What
// does not depend on the query row - a padding mask read per key column and everything computed from it alone - is
// moved to the line `marker`, which sits with the operand loads in front of the first MFMA (and, with several row
// blocks per wave, in front of their loop): definitions `const T vN = <expression>;` at the indentation of the
// straight-line part whose identifiers are parameters, the lane's coordinates of the key column (g, kw; not r16 or
// lane, which also say which row the lane holds), the batch index, pure functions and earlier moved values.
std::string hoist_row_invariant_values(const std::string& text, const std::string& marker) {
  std::vector<std::string> lines;
  {
    std::istringstream is(text);
    std::string l;
    while (std::getline(is, l)) lines.push_back(l);
  }
  size_t at = lines.size();
  for (size_t i = 0; i < lines.size(); ++i)
    if (lines[i].find(marker) != std::string::npos) at = i;
  if (at == lines.size()) return text;
  static const std::regex v_def(R"(^(\s*)const ([A-Za-z_]\w*) (v\d+) = (.*);$)");
  static const std::regex ident(R"((^|[^\w.])([A-Za-z_]\w*))");
  static const std::regex allowed(
      R"(^(in\d+|bidx|g|kw|colc|colv|float|double|_Float16|int|long|unsigned|short|char|bool|int8_t|uint8_t|int16_t|uint16_t|int32_t|uint32_t|int64_t|uint64_t|fmaxf|fminf|fabsf|__expf|__logf|tanhf|sqrtf|rsqrtf|__builtin_amdgcn_rcpf|__builtin_inff)$)");
  // the straight-line part: the indentation of the first value definition behind the marker
  size_t body_indent = std::string::npos;
  std::set<std::string> moved_names;
  std::vector<std::string> moved, rest;
  const std::string pad(lines[at].find_first_not_of(' ') == std::string::npos ? 0 : lines[at].find_first_not_of(' '), ' ');
  for (size_t i = at + 1; i < lines.size(); ++i) {
    std::smatch m;
    bool move = false;
    if (std::regex_match(lines[i], m, v_def)) {
      if (body_indent == std::string::npos) body_indent = m[1].length();
      if (static_cast<size_t>(m[1].length()) == body_indent) {
        move = true;
        const std::string rhs = m[4].str();
        for (auto it = std::sregex_iterator(rhs.begin(), rhs.end(), ident); move && it != std::sregex_iterator(); ++it) {
          const std::string id = (*it)[2].str();
          move = std::regex_match(id, allowed) || moved_names.count(id) || (id.size() > 1 && id.back() == 'f' && std::isdigit(static_cast<unsigned char>(id[0])));
        }
        if (move) {
          moved_names.insert(m[3].str());
          moved.push_back(pad + "const " + m[2].str() + " " + m[3].str() + " = " + rhs + ";");
        }
      }
    }
    if (!move) rest.push_back(lines[i]);
  }
  std::string out;
  for (size_t i = 0; i < at; ++i) out += lines[i] + "\n";
  for (auto& l : moved) out += l + "\n";
  for (auto& l : rest) out += l + "\n";
  return out;
}

// GEMM -> row program -> GEMM with everything between the two contractions on chip.
//
// A workgroup owns RW blocks of 16 rows m of one batch element; the KW waves of a block split the
// N1 columns of the first GEMM (the keys) between them.  S = A1 . B1^T is accumulated with the B1
// fragment as first MFMA operand, which leaves lane (r16, g) with S[m = r16][n = n_w + 16 j + 4 g + r]:
// the wave's part of a row lives in the 4 lanes r16, r16+16, r16+32, r16+48.  The row program
// (soft-max) is generated as straight-line code over those values; a reduction finishes with two
// butterfly steps across the 4 lanes and, for KW > 1, one exchange through LDS.  The result P feeds
// the second contraction directly: its k index inside one 32-wide MFMA step is enumerated as
// k(g, i) = 16 (i / 4) + 4 g + i % 4, i < 8, for both operands (a permutation of the summation order
// leaves the sum unchanged), which is exactly the order the lane already holds P in.  The right
// operand of the second GEMM is read through the same enumeration: two 8-byte loads per fragment
// from its k-contiguous layout.  The KW partial products meet in LDS; wave kw finishes the column
// tiles t with t % KW == kw and runs the epilogue on them.
NodeFunction gen_attention(const Program& prog, const Instr* g1, const graph::GemmDesc& d1, const std::vector<const Instr*>& row_members,
                           const Instr* g2, const graph::GemmDesc& d2, const std::vector<const Instr*>& epi_members,
                           const std::vector<const Instr*>& outputs, const LaunchShape& ls, int key_waves,
                           const Instr* g3 = nullptr, const graph::GemmDesc* d3p = nullptr, int heads = 0, bool preload_w = false, int row_blocks = 1,
                           Partition part = Partition()) {
  const int NW = ls.waves();
  const int64_t M1 = d1.M, N1 = d1.N, K1 = d1.K, N2 = d2.N;
  MONONN_CHECK(d1.a_k_contig && d1.b_k_contig && d2.a_k_contig, kUnsupported) << "attention fusion needs k-contiguous operands";
  MONONN_CHECK(!d1.f32 && !d2.f32 && d1.bf16 == d2.bf16, kUnsupported) << "attention fusion needs both contractions in the same 2-byte type";
  // scores and probabilities are held between the two contractions in the type the HLO gives them: f16, or bf16 with
  // the bf16 form of the MFMA on the same bits (operands move as 16-byte pieces either way)
  const bool bf = d1.bf16;
  const std::string ET = bf ? "__bf16" : "_Float16";
  const std::string MFMA = std::string("mononn_dev::mfma_16x16x32<") + (bf ? "true" : "false") + ">(";
  MONONN_CHECK(!bf || !g3, kUnsupported) << "the projection inside the attention node is built for f16";
  MONONN_CHECK(K1 % 32 == 0 && N2 % 16 == 0, kUnsupported) << "attention fusion: head size must be an MFMA multiple";
  // A key count off the MFMA step (ViT: 197): every wave's slice is rounded up to whole steps of 32 keys; the keys
  // past the end are read from the last valid key (finite values, in range), take no part in the row reductions
  // and get probability zero.  Plain k-contiguous K and V only (fragment-order operands have whole blocks).
  const bool ragged = N1 % 32 != 0;
  MONONN_CHECK(!ragged || (!d1.b_tiled && !d2.b_tiled && !g3), kUnsupported) << "attention fusion: a key count off the MFMA step needs plain k-contiguous keys and values";
  int KW = 1;
  if (ragged) {
    while (KW * 2 <= NW && (N1 + KW * 2 - 1) / (KW * 2) >= 32) KW *= 2;
  } else {
    while (KW * 2 <= NW && N1 % (32 * KW * 2) == 0 && N1 / (KW * 2) >= 32) KW *= 2;
  }
  if (key_waves > 0) {
    // tuning knob: fewer key slices per row block mean fewer exchanges through LDS but fewer, longer units
    MONONN_CHECK(NW % key_waves == 0 && (ragged || N1 % (32 * key_waves) == 0), kSpecError)
        << "attention: " << key_waves << " key waves do not divide " << NW << " waves / " << N1 << " keys";
    KW = key_waves;
  }
  const int RW = NW / KW;
  // Row blocks a wave takes one after the other with the keys and values it loaded once (many rows per batch element:
  // the operand traffic of a unit is the whole K and V of the head, whatever the number of rows it serves).
  const int RB = std::max(1, row_blocks);
  MONONN_CHECK(RB <= 32 && (RB == 1 || !g3), kSpecError) << "attention: " << RB << " row blocks per wave (at most 32, and one with the projection inside)";
  const int64_t NKW = ragged ? ((N1 + KW - 1) / KW + 31) / 32 * 32 : N1 / KW;   // keys per wave
  MONONN_CHECK(!ragged || (KW - 1) * NKW < N1, kUnsupported) << "attention fusion: " << KW << " key waves leave a wave without keys";
  const int KS1 = static_cast<int>(K1 / 32), NT1 = static_cast<int>(NKW / 16), KS2 = static_cast<int>(NKW / 32), NT2 = static_cast<int>(N2 / 16);
  RowInfo info = analyze_rows(row_members);
  MONONN_CHECK(info.row_program && info.rows == d1.batch * M1 && info.row_len == N1, kUnsupported)
      << "attention fusion: the cluster between the GEMMs is not a row program over the first GEMM's rows";
  auto row_outs = external_outputs(prog, row_members);
  MONONN_CHECK(row_outs.size() == 1 && row_outs[0]->shape.num_elements() == d1.batch * M1 * N1 && row_outs[0]->shape.dtype == (bf ? DType::kBF16 : DType::kF16), kUnsupported)
      << "attention fusion: the row program must produce exactly one matrix of the operands' type";
  const Instr* P = row_outs[0];

  PointerTable ptrs;
  std::string pq = ptrs.input(prog.storage_root(g1->operands[0]));
  std::string pk = ptrs.input(prog.storage_root(g1->operands[1]));
  std::string pv = ptrs.input(prog.storage_root(g2->operands[1]));
  if (bf) {
    pq = "reinterpret_cast<const _Float16*>(" + pq + ")";
    pk = "reinterpret_cast<const _Float16*>(" + pk + ")";
    pv = "reinterpret_cast<const _Float16*>(" + pv + ")";
  }
  const size_t first_epi = ptrs.entries.size();

  CodeBuffer cb;
  VarTable vars;
  Emitter em(prog, row_members, cb, vars, ptrs);
  em.set_fast_divide(true);
  const hlo::Shape& D1 = g1->shape;
  std::vector<int64_t> batch_dims(D1.dims.begin(), D1.dims.end() - 2);
  int vb = vars.add("bidx", d1.batch);
  int vm = vars.add("m", M1);
  int vg = vars.add("g", 4);
  int vkw = vars.add("kw", KW);
  auto elem_index = [&](int j, int r) {
    Index idx = delinearize(LinExpr::variable(vb, d1.batch), batch_dims, vars);
    idx.push_back(LinExpr::variable(vm, M1));
    // ragged key count: the column comes from a run-time value clamped to the last key (colc[j][r], set up below)
    if (ragged) idx.push_back(LinExpr::opaque("colc[" + S(j) + "][" + S(r) + "]", N1));
    else idx.push_back(LinExpr::variable(vkw, KW).scaled(NKW).plus(LinExpr::variable(vg, 4).scaled(4)).plus_const(j * 16 + r));
    return idx;
  };
  Index row_index = delinearize(LinExpr::variable(vb, d1.batch), batch_dims, vars);
  row_index.push_back(LinExpr::variable(vm, M1));

  std::ostringstream alpha_s;
  alpha_s.precision(9);
  alpha_s << d1.alpha;
  std::string alpha_lit = alpha_s.str();
  if (alpha_lit.find_first_of(".e") == std::string::npos) alpha_lit += ".0";

  // LDS: one slot of RW*KW*16 values per reduction, then the partial products
  auto reduces = em.collect_reduces();
  int smem = 0;
  std::vector<int> red_off;
  if (KW > 1) {
    for (size_t i = 0; i < reduces.size(); ++i) {
      red_off.push_back(smem);
      smem += RW * KW * 16 * 8;
    }
  }
  const int o_off = smem;
  if (KW > 1) smem += RW * KW * NT2 * 64 * 16;
  // absorbed projection: the context rows of a row block as f16 left-operand fragments [N2 / 32][64 lanes][8]
  const int cx_off = smem;
  if (g3) smem += RW * static_cast<int>(N2) * 16 * 2;
  // Several row blocks per wave over keys and values in fragment order: the workgroup copies the head's K and V into
  // LDS once (a straight copy: fragment order is the order the MFMAs read) and every wave takes its fragments from
  // there, row block after row block.  Holding them in registers across the rounds instead (what the other layouts
  // do) leaves the soft-max no registers at 384 keys per wave.
  const bool kv_lds = RB > 1 && d1.b_tiled && d2.b_tiled && !ragged && !g3 && (N1 * K1) % 8 == 0 && (N2 * N1) % 8 == 0;
  const int kv_off = (smem + 15) / 16 * 16;
  if (kv_lds) smem = kv_off + static_cast<int>((N1 * K1 + N2 * N1) * 2);

  cb.line("const int lane = mononn_dev::lane_id();");
  cb.line("const int r16 = lane & 15, g = lane >> 4;");
  cb.line("const int kw = mononn_dev::wave_id() % " + S(KW) + ", rw = mononn_dev::wave_id() / " + S(KW) + ";");
  const int64_t blocks = (M1 + 16 * RW * RB - 1) / (16 * RW * RB);
  int64_t num_units = d1.batch * blocks;
  if (part.on()) {
    // regional synchronisation: unit 8 q + x belongs to XCD x, which takes a run of batch elements (heads)
    MONONN_CHECK(part.kind == Partition::kHeads && !g3 && part.parts <= 8 && d1.batch % part.parts == 0, kInternal) << "attention node cannot be dealt to the XCDs";
    num_units = 8 * (d1.batch / part.parts) * blocks;
    cb.line("const int bidx = (unit & 7) * " + S(d1.batch / part.parts) + " + (unit >> 3) / " + S(blocks) + ";");
    cb.line("const int mt0 = ((unit >> 3) % " + S(blocks) + ") * " + S(RW * RB) + " + rw;");
  } else {
  cb.line("const int bidx = unit / " + S(blocks) + ";");
  // row block of this wave in round rb of the unit: mt0 + rb * RW
  cb.line("const int mt0 = (unit % " + S(blocks) + ") * " + S(RW * RB) + " + rw;");
  }
  auto row_block_head = [&](const std::string& mt_expr) {
    cb.line("const int mt = " + mt_expr + ";");
    cb.line("const bool m_valid = mt * 16 + r16 < " + S(M1) + ";");
    cb.line("const int m = m_valid ? mt * 16 + r16 : " + S(M1 - 1) + ";");
  };
  // Operands in fragment order (stored so by the stage that produced them) are one contiguous KiB per MFMA step;
  // row-major ones cost a lane's 16 rows x 16 bytes = 16 cache lines per quarter wave.
  MONONN_CHECK(!d1.a_packed || M1 % 16 == 0, kInternal) << "fragment-order queries need whole row blocks";
  // the query fragments of row block `mt_expr` (clamped into the matrix) into `dst`
  auto load_queries = [&](const std::string& dst, const std::string& mt_expr) {
    cb.open("");
    if (d1.a_packed) {
      cb.line("const int mt_q = " + mt_expr + " < " + S(M1 / 16) + " ? " + mt_expr + " : " + S(M1 / 16 - 1) + ";");
      cb.line("const _Float16* qp = " + pq + " + (((long)bidx * " + S(M1 / 16) + " + mt_q) * " + S(KS1 * 64) + " + lane) * 8;");
    } else {
      cb.line("const int m_q = (" + mt_expr + ") * 16 + r16 < " + S(M1) + " ? (" + mt_expr + ") * 16 + r16 : " + S(M1 - 1) + ";");
      cb.line("const _Float16* qp = " + pq + " + (long)bidx * " + S(d1.a_batch_stride) + " + m_q * " + S(K1) + " + g * 8;");
    }
    cb.line("#pragma unroll");
    cb.line("for (int ks = 0; ks < " + S(KS1) + "; ++ks) " + dst + "[ks] = *reinterpret_cast<const half8_t*>(qp + ks * " + S(d1.a_packed ? 512 : 32) + ");");
    cb.close();
  };
  if (RB == 1) row_block_head("mt0");
  if (d1.b_tiled) cb.line("const _Float16* kp = " + pk + " + (((long)bidx * " + S(N1 / 16) + " + kw * " + S(NKW / 16) + ") * " + S(KS1 * 64) + " + lane) * 8;");
  else if (ragged) cb.line("const _Float16* kp = " + pk + " + (long)bidx * " + S(d1.b_batch_stride) + " + g * 8;   // + key * " + S(K1));
  else cb.line("const _Float16* kp = " + pk + " + (long)bidx * " + S(d1.b_batch_stride) + " + (kw * " + S(NKW) + " + r16) * " + S(K1) + " + g * 8;");
  if (d2.b_tiled) cb.line("const _Float16* vp = " + pv + " + (((long)bidx * " + S(N2 / 16) + ") * " + S(N1 / 32) + " + kw * " + S(NKW / 32) + ") * 512 + lane * 8;");
  else if (ragged) cb.line("const _Float16* vp = " + pv + " + (long)bidx * " + S(d2.b_batch_stride) + " + r16 * " + S(N1) + ";   // row r16 of V^T; + t * 16 rows + key");
  else cb.line("const _Float16* vp = " + pv + " + (long)bidx * " + S(d2.b_batch_stride) + " + r16 * " + S(N1) + " + kw * " + S(NKW) + " + g * 4;");
  if (ragged) {
    // this lane's score columns: key kw * NKW + 16 j + 4 g + r; colc = the key it reads instead when that one is past the end
    cb.line("int colc[" + S(NT1) + "][4];");
    cb.line("bool colv[" + S(NT1) + "][4];");
    cb.line("#pragma unroll");
    cb.open("for (int j = 0; j < " + S(NT1) + "; ++j)");
    cb.line("#pragma unroll");
    cb.open("for (int r = 0; r < 4; ++r)");
    cb.line("const int col = kw * " + S(NKW) + " + j * 16 + g * 4 + r;");
    cb.line("colv[j][r] = col < " + S(N1) + ";");
    cb.line("colc[j][r] = colv[j][r] ? col : " + S(N1 - 1) + ";");
    cb.close();
    cb.close();
  }
  // ---- absorbed output projection: this head's K3 slice of the packed weights, all N3 columns split over the KW waves
  std::string pw, po, preload_body;
  int NT3 = 0, NJ = 0, KS3 = 0;
  if (g3) {
    const graph::GemmDesc& d3 = *d3p;
    MONONN_CHECK(!d2.has_addend && N2 % 32 == 0 && d3.N % 16 == 0 && d3.K == heads * N2 && d1.batch % heads == 0 && !d3.has_addend, kUnsupported)
        << g3->hlo_name << ": projection cannot run inside the attention node";
    pw = ptrs.input(prog.storage_root(g3->operands[1]));
    po = ptrs.output(g3, DType::kF32);
    NT3 = static_cast<int>(d3.N / 16);
    NJ = (NT3 + KW - 1) / KW;
    KS3 = static_cast<int>(N2 / 32);
    CodeBuffer wl;
    wl.line("#pragma unroll");
    wl.open("for (int jj = 0; jj < " + S(NJ) + "; ++jj)");
    wl.line("int nt = jj * " + S(KW) + " + kw;");
    wl.line("nt = nt < " + S(NT3) + " ? nt : " + S(NT3 - 1) + ";");
    wl.line("#pragma unroll");
    wl.line("for (int s = 0; s < " + S(KS3) + "; ++s) pre_w.v[jj * " + S(KS3) + " + s] = *reinterpret_cast<const half8_t*>(" + pw + " + (((long)nt * " +
            S(d3.K / 32) + " + head * " + S(KS3) + " + s) * 64 + lane) * 8);");
    wl.close();
    preload_body = wl.text();
    cb.line("const int head = bidx % " + S(heads) + ";");
    if (!preload_w) {
      cb.line("@NAME@_preb pre_w;");
      std::istringstream is(preload_body);
      std::string l;
      while (std::getline(is, l)) cb.line(l);
    }
  }
  // all operand loads up front: one exposed memory latency for the whole unit
  cb.line("half8_t qf[" + S(KS1) + "];");
  load_queries("qf", "mt0");
  std::string kfrag = "kf[j][ks]", vfrag = "vf[t][ks]";
  if (kv_lds) {
    const int64_t kc = N1 * K1 / 8, vc = N2 * N1 / 8;   // 16-byte pieces of the head's K and V
    const int block = NW * 64;
    const int per_thread = static_cast<int>((kc + vc + block - 1) / block);
    MONONN_CHECK(per_thread <= 64, kSpecError) << "attention: keys and values of a head do not go through the workgroup's registers in one pass";
    cb.line("half8_t* lk = reinterpret_cast<half8_t*>(smem + " + S(kv_off) + ");");
    cb.line("half8_t* lv = lk + " + S(kc) + ";");
    cb.open("");
    cb.line("const half8_t* gk = reinterpret_cast<const half8_t*>(" + pk + " + (long)bidx * " + S(N1 * K1) + ");");
    cb.line("const half8_t* gv = reinterpret_cast<const half8_t*>(" + pv + " + (long)bidx * " + S(N2 * N1) + ");");
    cb.line("const int tid = mononn_dev::wave_id() * 64 + lane;");
    cb.line("half8_t stg[" + S(per_thread) + "];");
    cb.line("#pragma unroll");
    cb.open("for (int c = 0; c < " + S(per_thread) + "; ++c)");
    cb.line("const int i = c * " + S(block) + " + tid;");
    cb.line("if (i < " + S(kc) + ") stg[c] = gk[i];");
    cb.line("else if (i < " + S(kc + vc) + ") stg[c] = gv[i - " + S(kc) + "];");
    cb.close();
    cb.line("__syncthreads();   // the previous unit's readers are done with its keys and values");
    cb.line("#pragma unroll");
    cb.open("for (int c = 0; c < " + S(per_thread) + "; ++c)");
    cb.line("const int i = c * " + S(block) + " + tid;");
    cb.line("if (i < " + S(kc + vc) + ") lk[i] = stg[c];");
    cb.close();
    cb.line("__syncthreads();");
    cb.close();
    kfrag = "lk[((kw * " + S(NKW / 16) + " + j) * " + S(KS1) + " + ks) * 64 + lane]";
    vfrag = "lv[(t * " + S(N1 / 32) + " + kw * " + S(NKW / 32) + " + ks) * 64 + lane]";
  } else {
  cb.line("half8_t kf[" + S(NT1) + "][" + S(KS1) + "];");
  cb.line("half8_t vf[" + S(NT2) + "][" + S(KS2) + "];");
  cb.line("#pragma unroll");
  cb.open("for (int j = 0; j < " + S(NT1) + "; ++j)");
  cb.line("#pragma unroll");
  if (d1.b_tiled) {
    cb.line("for (int ks = 0; ks < " + S(KS1) + "; ++ks) kf[j][ks] = *reinterpret_cast<const half8_t*>(kp + (j * " + S(KS1) + " + ks) * 512);");
  } else if (ragged) {
    cb.open("for (int ks = 0; ks < " + S(KS1) + "; ++ks)");
    cb.line("int key = kw * " + S(NKW) + " + j * 16 + r16;");
    cb.line("key = key < " + S(N1) + " ? key : " + S(N1 - 1) + ";");
    cb.line("kf[j][ks] = *reinterpret_cast<const half8_t*>(kp + key * " + S(K1) + " + ks * 32);");
    cb.close();
  } else {
    cb.line("for (int ks = 0; ks < " + S(KS1) + "; ++ks) kf[j][ks] = *reinterpret_cast<const half8_t*>(kp + j * " + S(16 * K1) + " + ks * 32);");
  }
  cb.close();
  cb.line("#pragma unroll");
  cb.open("for (int t = 0; t < " + S(NT2) + "; ++t)");
  cb.line("#pragma unroll");
  cb.open("for (int ks = 0; ks < " + S(KS2) + "; ++ks)");
  if (d2.b_tiled) {
    cb.line("vf[t][ks] = *reinterpret_cast<const half8_t*>(vp + (t * " + S(N1 / 32) + " + ks) * 512);");
  } else if (ragged) {
    // rows of an odd length start at odd element offsets: no alignment promise, and the keys past the end read the
    // row's last element (their probabilities are zero)
    cb.line("vf[t][ks] = mononn_dev::load_key_run(vp + t * " + S(16 * N1) + ", kw * " + S(NKW) + " + ks * 32 + g * 4, " + S(N1) + ");");
  } else {
    cb.line("const half4_t lo = *reinterpret_cast<const half4_t*>(vp + t * " + S(16 * N1) + " + ks * 32);");
    cb.line("const half4_t hi = *reinterpret_cast<const half4_t*>(vp + t * " + S(16 * N1) + " + ks * 32 + 16);");
    cb.line("vf[t][ks] = half8_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};");
  }
  cb.close();
  cb.close();
  }
  cb.line("// @ROW_INVARIANT@");
  if (RB > 1) {
    // one round per row block: the next block's queries are requested before this one's arithmetic
    cb.line("#pragma unroll 1");
    cb.open("for (int rb = 0; rb < " + S(RB) + "; ++rb)");
    row_block_head("mt0 + rb * " + S(RW));
    cb.line("half8_t qn[" + S(KS1) + "];");
    load_queries("qn", "(mt + " + S(RW) + ")");
  }
  cb.line("float4_t sacc[" + S(NT1) + "];");
  if (kv_lds) {
    // A wave alone on its SIMD has nobody to hide an LDS read behind: the fragments come in groups, the next group
    // requested before the MFMAs of the current one, with the scheduler kept from sinking the reads to their uses.
    int G = 1;
    for (int c : {4, 3, 2})
      if (NT1 % c == 0) { G = c; break; }
    const int per = G * KS1;
    cb.line("half8_t kb[2][" + S(per) + "];");
    cb.line("#pragma unroll");
    cb.line("for (int x = 0; x < " + S(per) + "; ++x) kb[0][x] = lk[((kw * " + S(NKW / 16) + " + x / " + S(KS1) + ") * " + S(KS1) + " + x % " + S(KS1) + ") * 64 + lane];");
    cb.line("#pragma unroll");
    cb.open("for (int jg = 0; jg < " + S(NT1 / G) + "; ++jg)");
    cb.open("if (jg + 1 < " + S(NT1 / G) + ")");
    cb.line("#pragma unroll");
    cb.line("for (int x = 0; x < " + S(per) + "; ++x) kb[(jg + 1) & 1][x] = lk[((kw * " + S(NKW / 16) + " + (jg + 1) * " + S(G) + " + x / " + S(KS1) + ") * " + S(KS1) + " + x % " + S(KS1) + ") * 64 + lane];");
    cb.close();
    cb.line("__builtin_amdgcn_sched_barrier(0);");
    cb.line("#pragma unroll");
    cb.open("for (int x = 0; x < " + S(per) + "; ++x)");
    cb.line("const int j = jg * " + S(G) + " + x / " + S(KS1) + ";");
    cb.line("if (x % " + S(KS1) + " == 0) sacc[j] = float4_t{0.f, 0.f, 0.f, 0.f};");
    cb.line("sacc[j] = " + MFMA + "kb[jg & 1][x], qf[x % " + S(KS1) + "], sacc[j]);");
    cb.close();
    cb.line("__builtin_amdgcn_sched_barrier(0);");
    cb.close();
  } else {
  cb.line("#pragma unroll");
  cb.open("for (int j = 0; j < " + S(NT1) + "; ++j)");
  cb.line("sacc[j] = float4_t{0.f, 0.f, 0.f, 0.f};");
  cb.line("#pragma unroll");
  cb.line("for (int ks = 0; ks < " + S(KS1) + "; ++ks) sacc[j] = " + MFMA + "" + kfrag + ", qf[ks], sacc[j]);");
  cb.close();
  }
  // the first GEMM's result as the HLO defines it: scaled, rounded to f16
  cb.line(ET + " sv[" + S(NT1) + "][4], pr[" + S(NT1) + "][4];");
  cb.line("#pragma unroll");
  cb.open("for (int j = 0; j < " + S(NT1) + "; ++j)");
  cb.line("#pragma unroll");
  cb.line(std::string("for (int r = 0; r < 4; ++r) sv[j][r] = (" + ET + ")(sacc[j][r]") + (d1.alpha == 1.0 ? "" : " * " + alpha_lit + "f") + ");");
  cb.close();
  // ---- row program on the register-resident rows ------------------------------------------------
  auto bind_elem = [&](int j, int r) { em.bind(g1, elem_index(j, r), "sv[" + S(j) + "][" + S(r) + "]"); };
  for (size_t ri = 0; ri < reduces.size(); ++ri) {
    const Instr* red = reduces[ri];
    std::string Tn = hlo::dtype_ctype(red->shape.dtype);
    MONONN_CHECK(hlo::dtype_bytes(red->shape.dtype) <= 8, kUnsupported) << "reduction type too wide";
    std::string acc = em.fresh("red");
    cb.line(Tn + " " + acc + " = " + em.value(red->operands[1], {}) + ";");
    for (int j = 0; j < NT1; ++j)
      for (int r = 0; r < 4; ++r) {
        bind_elem(j, r);
        std::string val = em.value(red->operands[0], elem_index(j, r));
        // a key past the end contributes the reduction's init value (its identity)
        if (ragged) val = "(colv[" + S(j) + "][" + S(r) + "] ? (" + Tn + ")(" + val + ") : (" + Tn + ")(" + em.value(red->operands[1], {}) + "))";
        cb.line(acc + " = (" + Tn + ")" + Emitter::reducer_expr(red, acc, val) + ";");
      }
    for (int off : {16, 32}) {
      std::string other = "__shfl_xor(" + acc + ", " + S(off) + ", 64)";
      cb.line(acc + " = (" + Tn + ")" + Emitter::reducer_expr(red, acc, other) + ";");
    }
    if (KW > 1) {
      std::string buf = em.fresh("rb");
      cb.line(Tn + "* " + buf + " = reinterpret_cast<" + Tn + "*>(smem + " + S(red_off[ri]) + ") + rw * " + S(KW * 16) + ";");
      cb.line("if (g == 0) " + buf + "[kw * 16 + r16] = " + acc + ";");
      cb.line("__syncthreads();");
      cb.line(acc + " = " + buf + "[r16];");
      for (int w = 1; w < KW; ++w) cb.line(acc + " = (" + Tn + ")" + Emitter::reducer_expr(red, acc, buf + "[" + S(w * 16) + " + r16]") + ";");
    }
    em.bind(red, row_index, acc);
  }
  for (int j = 0; j < NT1; ++j)
    for (int r = 0; r < 4; ++r) {
      bind_elem(j, r);
      if (ragged) cb.line("pr[" + S(j) + "][" + S(r) + "] = colv[" + S(j) + "][" + S(r) + "] ? (" + ET + ")(" + em.value(em.resolve_output(P), elem_index(j, r)) + ") : (" + ET + ")0;");
      else cb.line("pr[" + S(j) + "][" + S(r) + "] = " + em.value(em.resolve_output(P), elem_index(j, r)) + ";");
    }
  em.unbind(g1);
  // ---- second contraction ---------------------------------------------------------------------------
  // the probabilities of one k step as an MFMA operand (bf16: the same 16 bytes under the f16 vector type)
  const std::string pf_elems = "pr[2 * ks][0], pr[2 * ks][1], pr[2 * ks][2], pr[2 * ks][3], pr[2 * ks + 1][0], pr[2 * ks + 1][1], pr[2 * ks + 1][2], pr[2 * ks + 1][3]";
  const std::string pf_line = bf ? "const half8_t pf = __builtin_bit_cast(half8_t, bf16x8_t{" + pf_elems + "});" : "const half8_t pf = {" + pf_elems + "};";
  cb.line("float4_t oacc[" + S(NT2) + "];");
  cb.line("#pragma unroll");
  cb.line("for (int t = 0; t < " + S(NT2) + "; ++t) oacc[t] = float4_t{0.f, 0.f, 0.f, 0.f};");
  if (kv_lds) {
    const int G2 = KS2 % 2 == 0 ? 2 : 1;   // k steps per group
    const int per = G2 * NT2;
    cb.line("half8_t vb[2][" + S(per) + "];");
    cb.line("#pragma unroll");
    cb.line("for (int x = 0; x < " + S(per) + "; ++x) vb[0][x] = lv[((x % " + S(NT2) + ") * " + S(N1 / 32) + " + kw * " + S(NKW / 32) + " + x / " + S(NT2) + ") * 64 + lane];");
    cb.line("#pragma unroll");
    cb.open("for (int kg = 0; kg < " + S(KS2 / G2) + "; ++kg)");
    cb.open("if (kg + 1 < " + S(KS2 / G2) + ")");
    cb.line("#pragma unroll");
    cb.line("for (int x = 0; x < " + S(per) + "; ++x) vb[(kg + 1) & 1][x] = lv[((x % " + S(NT2) + ") * " + S(N1 / 32) + " + kw * " + S(NKW / 32) + " + (kg + 1) * " + S(G2) + " + x / " + S(NT2) + ") * 64 + lane];");
    cb.close();
    cb.line("__builtin_amdgcn_sched_barrier(0);");
    cb.line("#pragma unroll");
    cb.open("for (int y = 0; y < " + S(G2) + "; ++y)");
    cb.line("const int ks = kg * " + S(G2) + " + y;");
    cb.line(pf_line);
    cb.line("#pragma unroll");
    cb.line("for (int t = 0; t < " + S(NT2) + "; ++t) oacc[t] = " + MFMA + "vb[kg & 1][y * " + S(NT2) + " + t], pf, oacc[t]);");
    cb.close();
    cb.line("__builtin_amdgcn_sched_barrier(0);");
    cb.close();
  } else {
  cb.line("#pragma unroll");
  cb.open("for (int ks = 0; ks < " + S(KS2) + "; ++ks)");
  cb.line(pf_line);
  cb.line("#pragma unroll");
  cb.open("for (int t = 0; t < " + S(NT2) + "; ++t)");
  cb.line("oacc[t] = " + MFMA + "" + vfrag + ", pf, oacc[t]);");
  cb.close();
  cb.close();
  }

  std::vector<std::string> globals = tables_of(em);
  if (g3) {
    const graph::GemmDesc& d3 = *d3p;
    auto lit = [](double v) {
      std::ostringstream o;
      o.precision(9);
      o << v;
      std::string t = o.str();
      if (t.find_first_of(".e") == std::string::npos) t += ".0";
      return t + "f";
    };
    const std::string a2 = d2.alpha == 1.0 ? "" : " * " + lit(d2.alpha);
    // The context (second GEMM's result, rounded to f16 as the HLO defines it) goes to LDS in left-operand fragment
    // order: element d of row r16 belongs to step d / 32, lane (d % 32 / 8) * 16 + r16, slot d % 8; a lane holds
    // d = 16 t + 4 g + r, r < 4.
    cb.line("_Float16* cx = reinterpret_cast<_Float16*>(smem + " + S(cx_off) + ") + rw * " + S(N2 * 16) + ";");
    auto write_ctx = [&](const std::string& o) {
      cb.line("const half4_t ch = {(_Float16)(" + o + "[0]" + a2 + "), (_Float16)(" + o + "[1]" + a2 + "), (_Float16)(" + o + "[2]" + a2 + "), (_Float16)(" + o + "[3]" + a2 + ")};");
      cb.line("*reinterpret_cast<half4_t*>(cx + (((t >> 1) * 64 + ((t & 1) * 2 + (g >> 1)) * 16 + r16) * 8 + (g & 1) * 4)) = ch;");
    };
    if (KW > 1) {
      cb.line("float4_t* ob = reinterpret_cast<float4_t*>(smem + " + S(o_off) + ") + rw * " + S(KW * NT2 * 64) + ";");
      cb.line("#pragma unroll");
      cb.open("for (int t = 0; t < " + S(NT2) + "; ++t)");
      cb.line("if (t % " + S(KW) + " != kw) ob[(kw * " + S(NT2) + " + t) * 64 + lane] = oacc[t];");
      cb.close();
      cb.line("__syncthreads();");
      cb.line("#pragma unroll");
      cb.open("for (int t = 0; t < " + S(NT2) + "; ++t)");
      cb.line("if (t % " + S(KW) + " != kw) continue;");
      cb.line("float4_t o = oacc[t];");
      cb.line("#pragma unroll");
      cb.line("for (int w = 0; w < " + S(KW) + "; ++w) if (w != kw) o += ob[(w * " + S(NT2) + " + t) * 64 + lane];");
      write_ctx("o");
      cb.close();
    } else {
      cb.line("#pragma unroll");
      cb.open("for (int t = 0; t < " + S(NT2) + "; ++t)");
      write_ctx("oacc[t]");
      cb.close();
    }
    cb.line("__syncthreads();");
    cb.line("half8_t af[" + S(KS3) + "];");
    cb.line("#pragma unroll");
    cb.line("for (int s = 0; s < " + S(KS3) + "; ++s) af[s] = *reinterpret_cast<const half8_t*>(cx + (s * 64 + lane) * 8);");
    // one fp32 partial sum per head: [heads][M3][N3]; the consuming row program adds them up
    cb.line("float* prow = " + po + " + ((long)head * " + S(d3.M) + " + (bidx / " + S(heads) + ") * " + S(M1) + " + m) * " + S(d3.N) + " + g * 4;");
    cb.line("#pragma unroll");
    cb.open("for (int jj = 0; jj < " + S(NJ) + "; ++jj)");
    cb.line("float4_t pacc = {0.f, 0.f, 0.f, 0.f};");
    cb.line("#pragma unroll");
    cb.line("for (int s = 0; s < " + S(KS3) + "; ++s) pacc = " + MFMA + "pre_w.v[jj * " + S(KS3) + " + s], af[s], pacc);");
    cb.line("const int nt = jj * " + S(KW) + " + kw;");
    cb.open("if (m_valid && nt < " + S(NT3) + ")");
    const std::string a3 = d3.alpha == 1.0 ? "" : " * " + lit(d3.alpha);
    cb.line("const float pv4[4] = {pacc[0]" + a3 + ", pacc[1]" + a3 + ", pacc[2]" + a3 + ", pacc[3]" + a3 + "};");
    cb.line("mononn_dev::stN<float, 4>(prow + nt * 16, pv4);");
    cb.close();
    cb.close();
    cb.line("__syncthreads();   // LDS is reused by the next unit");
    NodeFunction f = finish(hoist_row_invariant_values(cb.text(), "@ROW_INVARIANT@"), ptrs, globals, d1.batch * blocks, smem,
                            "typedef mononn_dev::PreB<" + S(NJ * KS3) + "> @NAME@_preb;\n");
    if (preload_w) {
      const std::string tail = ", char* smem) {";
      size_t at = f.text.find(tail);
      MONONN_CHECK(at != std::string::npos, kInternal) << "node function signature not found";
      f.text.replace(at, tail.size(), ", char* smem, const @NAME@_preb& pre_w) {");
      std::string sig = signature(ptrs.entries);
      sig = sig.substr(0, sig.rfind(", char* smem"));
      CodeBuffer pf;
      pf.line("const int lane = mononn_dev::lane_id();");
      pf.line("const int kw = mononn_dev::wave_id() % " + S(KW) + ";");
      pf.line("const int head = (unit / " + S(blocks) + ") % " + S(heads) + ";");
      f.preload_text = "__device__ __forceinline__ void @NAME@_pre(" + sig + ", @NAME@_preb& pre_w) {\n" + pf.text() + preload_body + "}\n";
    }
    return f;
  }
  Epilogue epi = build_epilogue(prog, g2, epi_members, outputs, d2, true, ptrs, first_epi);
  for (auto& gl : epi.globals) globals.push_back(gl);
  cb.line(epi.init_line);
  if (KW > 1) {
    cb.line("float4_t* ob = reinterpret_cast<float4_t*>(smem + " + S(o_off) + ") + rw * " + S(KW * NT2 * 64) + ";");
    cb.line("#pragma unroll");
    cb.open("for (int t = 0; t < " + S(NT2) + "; ++t)");
    cb.line("if (t % " + S(KW) + " != kw) ob[(kw * " + S(NT2) + " + t) * 64 + lane] = oacc[t];");
    cb.close();
    cb.line("__syncthreads();");
    cb.line("#pragma unroll");
    cb.open("for (int t = 0; t < " + S(NT2) + "; ++t)");
    cb.line("if (t % " + S(KW) + " != kw) continue;");
    cb.line("float4_t o = oacc[t];");
    cb.line("#pragma unroll");
    cb.line("for (int w = 0; w < " + S(KW) + "; ++w) if (w != kw) o += ob[(w * " + S(NT2) + " + t) * 64 + lane];");
    cb.open("if (m_valid)");
    cb.line("const float v[4] = {o[0], o[1], o[2], o[3]};");
    cb.line("decltype(epi)::Pre pre;");
    cb.line("epi.preload(bidx, m, t * 16 + g * 4, pre);");
    cb.line("epi(bidx, m, t * 16 + g * 4, v, pre);");
    cb.close();
    cb.close();
    cb.line("__syncthreads();   // LDS is reused by the next unit");
  } else {
    cb.open("if (m_valid)");
    cb.line("#pragma unroll");
    cb.open("for (int t = 0; t < " + S(NT2) + "; ++t)");
    cb.line("const float v[4] = {oacc[t][0], oacc[t][1], oacc[t][2], oacc[t][3]};");
    cb.line("decltype(epi)::Pre pre;");
    cb.line("epi.preload(bidx, m, t * 16 + g * 4, pre);");
    cb.line("epi(bidx, m, t * 16 + g * 4, v, pre);");
    cb.close();
    cb.close();
  }
  if (RB > 1) {
    cb.line("#pragma unroll");
    cb.line("for (int ks = 0; ks < " + S(KS1) + "; ++ks) qf[ks] = qn[ks];");
    cb.close();
  }
  NodeFunction f = finish(hoist_row_invariant_values(cb.text(), "@ROW_INVARIANT@"), ptrs, globals, num_units, smem, epi.struct_text);
  f.write_maps = epi.writes;
  return f;
}

}  // namespace

NodeFunction generate_gemm(const Program& prog, const Node& node, const LaunchShape& ls, const GemmTuning& t) {
  return gen_gemm(prog, node.members, node.outputs, node.gemm, ls, t, node.prologue, node.prologue_stores, &node.ln_fold);
}

NodeFunction generate_attention(const Program& prog, const Node& node, const LaunchShape& ls, int key_waves, bool preload_weights, int row_blocks, Partition part) {
  std::vector<const Instr*> row(node.members.begin() + 1, node.members.begin() + node.gemm2_index);
  if (node.gemm3_index != 0) {
    std::vector<const Instr*> epi(node.members.begin() + node.gemm2_index + 1, node.members.begin() + node.gemm3_index);
    return gen_attention(prog, node.members[0], node.gemm, row, node.members[node.gemm2_index], node.gemm2, epi, node.outputs, ls, key_waves,
                         node.members[node.gemm3_index], &node.gemm3, node.heads, preload_weights);
  }
  std::vector<const Instr*> epi(node.members.begin() + node.gemm2_index + 1, node.members.end());
  return gen_attention(prog, node.members[0], node.gemm, row, node.members[node.gemm2_index], node.gemm2, epi, node.outputs, ls, key_waves, nullptr, nullptr, 0,
                       false, row_blocks, part);
}

bool can_fuse_out_proj(const Program& prog, const Instr* gemm2, const graph::GemmDesc& d2, const std::vector<const Instr*>& epilogue_members,
                       const Instr* gemm3, const graph::GemmDesc& d3, int heads) {
  try {
    check_out_proj_mapping(prog, gemm2, d2, epilogue_members, gemm3, d3, heads);
    return !d2.has_addend && !d3.has_addend;
  } catch (const Error& e) {
    if (getenv("MONONN_DEBUG_PASSES")) fprintf(stderr, "[attention out-projection fusion rejected] %s\n", e.what());
    if (e.code() == kUnsupported) return false;
    throw;
  }
}

int default_attention_key_waves(const graph::GemmDesc& d1, const LaunchShape& ls) {
  int KW = 1;
  while (KW * 2 <= ls.waves() && d1.N % (32 * KW * 2) == 0 && d1.N / (KW * 2) >= 32) KW *= 2;
  return KW;
}

bool can_fuse_prologue(const Program& prog, const std::vector<const Instr*>& row_members, const std::vector<const Instr*>& gemm_members,
                       const graph::GemmDesc& g) {
  try {
    graph::GemmDesc d = g;
    if (!d.a_k_contig || d.batch != 1 || d.K % 32 != 0) return false;
    d.b_k_contig = true;   // constant weights are packed / activations re-laid out before real generation
    LaunchShape ls;
    // the dry run takes the direct tile: the row program runs on the fragments a wave holds in registers (a folded
    // LayerNorm may later get an LDS-staged tile, which needs no row program at all)
    GemmTuning t = default_gemm_tuning(d, ls, 256, false);
    auto outs = external_outputs(prog, gemm_members);
    if (outs.empty()) return false;
    gen_gemm(prog, gemm_members, outs, d, ls, t, row_members, true);
    return true;
  } catch (const Error& e) {
    if (getenv("MONONN_DEBUG_PASSES")) fprintf(stderr, "[prologue fusion rejected] %s\n", e.what());
    if (e.code() == kUnsupported || e.code() == kSpecError) return false;
    throw;
  }
}

bool can_fuse_attention(const Program& prog, const Instr* gemm1, const graph::GemmDesc& d1, const std::vector<const Instr*>& row_members,
                        const Instr* gemm2, const graph::GemmDesc& d2, const std::vector<const Instr*>& epilogue_members) {
  try {
    std::vector<const Instr*> tail{gemm2};
    tail.insert(tail.end(), epilogue_members.begin(), epilogue_members.end());
    auto outs = external_outputs(prog, tail);
    if (outs.empty()) return false;
    graph::GemmDesc d2k = d2;
    d2k.b_k_contig = true;   // the layout pass stores the operand k-contiguous before real generation
    gen_attention(prog, gemm1, d1, row_members, gemm2, d2k, epilogue_members, outs, LaunchShape{}, 0);
    return true;
  } catch (const Error& e) {
    if (e.code() == kUnsupported) return false;
    throw;
  }
}

bool can_fuse_epilogue(const Program& prog, const std::vector<const Instr*>& gemm_members, const std::vector<const Instr*>& cluster_members) {
  if (!reduces_of(cluster_members).empty()) return false;
  std::vector<const Instr*> merged = gemm_members;
  merged.insert(merged.end(), cluster_members.begin(), cluster_members.end());
  try {
    auto outs = external_outputs(prog, merged);
    if (outs.empty()) return false;
    graph::GemmDesc g;   // only the shape matters for the dry run; layouts fall back to the naive path
    const Instr* gi = gemm_members[0];
    const hlo::Shape& D = gi->shape;
    g.M = D.dims[D.rank() - 2];
    g.N = D.dims[D.rank() - 1];
    g.K = gi->operands[0]->shape.dims[gi->gemm.lhs_contracting];
    g.batch = D.num_elements() / (g.M * g.N);
    g.a_k_contig = g.b_k_contig = true;
    g.a_batch_stride = g.M * g.K;
    g.b_batch_stride = g.N * g.K;
    g.alpha = gi->gemm.alpha_real;
    g.beta = gi->gemm.beta;
    g.has_addend = gi->operands.size() == 3 && g.beta != 0;
    LaunchShape ls;
    GemmTuning t;
    t.bm = t.bn = 32;
    t.wm = 1;
    t.wn = 1;
    t.wk = ls.waves();
    gen_gemm(prog, merged, outs, g, ls, t);
    return true;
  } catch (const Error& e) {
    if (e.code() == kUnsupported) return false;
    throw;
  }
}

}  // namespace codegen
}  // namespace mononn
