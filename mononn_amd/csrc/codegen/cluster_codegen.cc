#include "codegen/cluster_codegen.h"

#include <algorithm>
#include <set>
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
    bool ok = r->operands.size() == 2 && r->dimensions.size() == 1 && x.rank() >= 1 && r->dimensions[0] == x.rank() - 1;
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

void store(const Program& prog, CodeBuffer& cb, PointerTable& ptrs, const VarTable& vars, const Instr* out, const Index& idx, const std::string& v) {
  cb.line("mononn_dev::st1(" + ptrs.output(out) + " + " + physical_offset(prog, out, idx).str(vars) + ", " + v + ");");
}

std::string align_prologue(const std::vector<PointerTable::Entry>& ptrs);

NodeFunction finish(const std::string& body, PointerTable& ptrs, Emitter& em, int64_t units, int smem, const std::string& pre = "") {
  NodeFunction f;
  f.pointers = ptrs.entries;
  f.num_units = units;
  f.smem_bytes = smem;
  for (auto& kv : em.literal_tables()) f.globals.push_back(kv.second);
  f.text = pre + "__device__ __noinline__ void @NAME@(" + signature(ptrs.entries) + ") {\n" + align_prologue(ptrs.entries) + body + "}\n";
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
    const int stride = block_tier ? ls.block_size : 64;
    int row = vars.add("row", ROWS);
    std::vector<const Instr*> row_outs, full_outs;
    for (auto* o : outputs) {
      int64_t n = o->shape.num_elements();
      if (n == ROWS * R && R > 1) full_outs.push_back(o);
      else if (n == ROWS) row_outs.push_back(o);
      else MONONN_FAIL(kUnsupported) << o->hlo_name << ": output with " << n << " elements does not fit a " << ROWS << " x " << R << " row space";
    }
    cb.line("const int lane = mononn_dev::lane_id();");
    cb.line(std::string("const int tid = ") + (block_tier ? "(int)threadIdx.x;" : "lane;"));
    if (block_tier) {
      cb.line("const int row = unit;");
      cb.open("");
    } else {
      cb.line("const int row = unit * " + S(NW) + " + mononn_dev::wave_id();");
      cb.open("if (row < " + S(ROWS) + ")");
    }
    auto all_reduce = [&](const Instr* r, const std::string& acc) {
      std::string T = hlo::dtype_ctype(r->shape.dtype);
      if (block_tier) cb.line(acc + " = mononn_dev::block_all_reduce(" + acc + ", " + Emitter::reducer_functor(r) + ", reinterpret_cast<" + T + "*>(smem));");
      else cb.line(acc + " = mononn_dev::wave_all_reduce(" + acc + ", " + Emitter::reducer_functor(r) + ");");
    };
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
    const int V = t.ilp_factor > 1 && R % t.ilp_factor == 0 ? t.ilp_factor : pick_vector_width(R, stride);
    const int64_t NQ = R / V;
    const int64_t T = (NQ + stride - 1) / stride;
    if (T * V <= 32) {
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
            offs.push_back(physical_offset(prog, o, oi));
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
            lines.push_back("mononn_dev::stN<" + T + ", " + S(V) + ">(" + ptrs.output(o) + " + " + offs[0].str(vars) + ", " + arr + ");");
          } else {
            for (int v = 0; v < V; ++v) lines.push_back("mononn_dev::st1(" + ptrs.output(o) + " + " + offs[v].str(vars) + ", " + vals[v] + ");");
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
    int64_t units = block_tier ? ROWS : (ROWS + NW - 1) / NW;
    return finish(cb.text(), ptrs, em, units, block_tier ? NW * 8 : 0);
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
    const int V = (t.ilp_factor > 1 && N % t.ilp_factor == 0 && t.ilp_factor <= 16) ? t.ilp_factor : 1;
    const int64_t NQ = N / V;
    const int64_t units = (NQ + ls.block_size - 1) / ls.block_size;
    std::string u = "unit";
    if (groups.size() > 1) {
      cb.open(std::string(gi ? "else " : "") + "if (unit < " + S(unit_base + units) + ")");
      u = "(unit - " + S(unit_base) + ")";
    }
    std::string qv = "q" + S(gi);
    int var = vars.add(qv, NQ);
    cb.line("const int " + qv + " = " + u + " * " + S(ls.block_size) + " + (int)threadIdx.x;");
    cb.open("if (" + qv + " < " + S(NQ) + ")");
    em.push_scope();
    for (int v = 0; v < V; ++v)
      for (auto* o : groups[gi].second) {
        LinExpr lin = LinExpr::variable(var, NQ).scaled(V).plus_const(v);
        Index oi = delinearize(lin, o->shape.dims, vars);
        store(prog, cb, ptrs, vars, o, oi, em.value(em.resolve_output(o), oi));
      }
    em.pop_scope();
    cb.close();
    if (groups.size() > 1) cb.close();
    unit_base += units;
  }
  return finish(cb.text(), ptrs, em, unit_base, 0);
}

}  // namespace

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
bool gemm_uses_mfma(const graph::GemmDesc& g) { return g.a_k_contig && (g.b_k_contig || g.b_packed) && g.K % 32 == 0; }

GemmTuning default_gemm_tuning(const graph::GemmDesc& g, const LaunchShape& ls, int num_cus) {
  (void)num_cus;
  GemmTuning t;
  int waves = ls.waves();
  int wk = 1;
  while (wk * 2 <= waves && g.K / 32 >= wk * 2 * 2 && g.K >= 256 * wk) wk *= 2;
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

void validate_gemm_tuning(const graph::GemmDesc& g, const LaunchShape& ls, const GemmTuning& t) {
  (void)g;
  MONONN_CHECK(t.wm >= 1 && t.wn >= 1 && t.wk >= 1 && t.wm * t.wn * t.wk == ls.waves(), kSpecError)
      << "GEMM wave arrangement " << t.wm << "x" << t.wn << "x" << t.wk << " does not use " << ls.waves() << " waves";
  MONONN_CHECK(t.bm % (16 * t.wm) == 0 && t.bn % (16 * t.wn) == 0 && t.bm > 0 && t.bn > 0, kSpecError)
      << "GEMM tile " << t.bm << "x" << t.bn << " is not a multiple of 16 per wave";
  int frags = (t.bm / t.wm / 16) * (t.bn / t.wn / 16);
  MONONN_CHECK(frags <= 32, kSpecError) << "GEMM tile " << t.bm << "x" << t.bn << " needs " << frags << " accumulator fragments per wave (max 32)";
}

namespace {

struct EpilogueVars {
  int b, m, n4, r, nn;
};

NodeFunction gen_gemm(const Program& prog, const std::vector<const Instr*>& members, const std::vector<const Instr*>& outputs,
                      const graph::GemmDesc& g, const LaunchShape& ls, const GemmTuning& t) {
  const Instr* gi = members[0];
  const bool mfma = gemm_uses_mfma(g);
  const bool vec4 = mfma && g.N % 4 == 0;
  if (mfma) validate_gemm_tuning(g, ls, t);
  CodeBuffer cb;   // epilogue body
  VarTable vars;
  PointerTable ptrs;
  // the two operands come first in the pointer list
  std::string pa = ptrs.input(prog.storage_root(gi->operands[0]));
  std::string pb = ptrs.input(prog.storage_root(gi->operands[1]));
  const size_t first_epi = ptrs.entries.size();   // 1 when both operands are the same buffer
  std::vector<const Instr*> cluster_members(members.begin() + 1, members.end());
  Emitter em(prog, cluster_members, cb, vars, ptrs);

  const hlo::Shape& D = gi->shape;
  std::vector<int64_t> batch_dims(D.dims.begin(), D.dims.end() - 2);
  int vb = vars.add("bidx", g.batch);
  int vm = vars.add("m", g.M);
  int vn4 = -1, vr = -1, vnn = -1;
  if (vec4) {
    vn4 = vars.add("n4", g.N / 4);
    vr = vars.add("r", 4);
  } else {
    vnn = vars.add("nn", g.N);
  }
  auto gemm_index = [&](bool with_r) {
    Index idx = delinearize(LinExpr::variable(vb, g.batch), batch_dims, vars);
    idx.push_back(LinExpr::variable(vm, g.M));
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

  if (vec4) cb.line("const int n4 = n0 >> 2;");
  // per-output staging arrays for the vector store
  struct Out {
    const Instr* o;
    Index idx;        // chosen index (with r)
    Index idx_base;   // same with r = 0
    bool vector_store;
    std::string stage;
  };
  std::vector<Out> outs;
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
    cb.line("const _Float16 " + gv + " = (_Float16)" + expr + ";");
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
        LinExpr full = physical_offset(prog, out.o, out.idx);
        LinExpr base = physical_offset(prog, out.o, out.idx_base);
        out.vector_store = full.equals(base.plus(LinExpr::variable(vr, 4))) && out.o->shape.dtype == DType::kF16;
        if (out.vector_store) cb.line(out.stage + "[r] = " + v + ";");
        else store(prog, cb, ptrs, vars, out.o, out.idx, v);
      } else {
        store(prog, cb, ptrs, vars, out.o, out.idx, v);
      }
    }
  }
  em.pop_scope();
  cb.close();
  if (vec4) {
    for (auto& out : outs)
      if (out.vector_store) {
        std::string lin = physical_offset(prog, out.o, out.idx_base).str(vars);
        cb.line("mononn_dev::stN<_Float16, 4>(" + ptrs.output(out.o) + " + " + lin + ", " + out.stage + ");");
      }
  }

  // ---- assemble: epilogue functor + stage function -------------------------------------------
  std::string pre = "struct @NAME@_epi {\n";
  for (size_t i = first_epi; i < ptrs.entries.size(); ++i) {
    auto& e = ptrs.entries[i];
    pre += std::string("  ") + (e.is_output ? "" : "const ") + hlo::dtype_ctype(e.dtype) + "* " + e.name + ";\n";
  }
  if (mfma) {
    // touch the epilogue's operands ahead of the main loop
    pre += "  __device__ __forceinline__ void prefetch(int bidx, int m, int n0) const {\n";
    if (vec4 && !em.simple_loads().empty()) {
      pre += "    const int n4 = n0 >> 2;\n    #pragma unroll\n    for (int r = 0; r < 4; ++r) {\n";
      for (auto& l : em.simple_loads()) pre += "      mononn_dev::touch(" + l + ");\n";
      pre += "    }\n";
    }
    pre += "  }\n";
  }
  if (vec4) pre += "  __device__ __forceinline__ void operator()(int bidx, int m, int n0, const float (&acc)[4]) const {\n";
  else if (mfma) {
    pre += "  __device__ __forceinline__ void operator()(int bidx, int m, int n0, const float (&accv)[4]) const {\n";
    pre += "    for (int r = 0; r < 4; ++r) { const int nn = n0 + r; if (nn < " + S(g.N) + ") { const float acc = accv[r]; one(bidx, m, nn, acc); } }\n  }\n";
    pre += "  __device__ __forceinline__ void one(int bidx, int m, int nn, float acc) const {\n";
  } else {
    pre += "  __device__ __forceinline__ void operator()(int bidx, int m, int nn, float acc) const {\n";
  }
  {
    std::istringstream is(cb.text());
    std::string l;
    while (std::getline(is, l)) pre += "  " + l + "\n";
  }
  pre += "  }\n};\n";

  CodeBuffer fb;
  std::string init = "@NAME@_epi epi{";
  for (size_t i = first_epi; i < ptrs.entries.size(); ++i) init += (i > first_epi ? ", " : "") + ptrs.entries[i].name;
  init += "};";
  fb.line(init);
  int64_t units = 0;
  int smem = 0;
  if (mfma) {
    // Unit order: the workgroups that read the same columns of B (same tile_n, all tile_m) differ by
    // multiples of 8 in their unit index; with units dealt round-robin over the 8 XCDs they land on
    // one XCD and share its L2.  tile_n = 8 * (q / tiles_m) + u % 8, tile_m = q % tiles_m, q = u / 8.
    const int64_t tiles_m = (g.M + t.bm - 1) / t.bm, tiles_n = (g.N + t.bn - 1) / t.bn;
    if (tiles_n % 8 == 0) {
      const int64_t per_batch = tiles_n * tiles_m;
      units = g.batch * per_batch;
      fb.line("const int bidx = unit / " + S(per_batch) + ";");
      fb.line("const int rem = unit % " + S(per_batch) + ";");
      fb.line("const int tile_n = (rem >> 3) / " + S(tiles_m) + " * 8 + (rem & 7);");
      fb.line("const int tile_m = (rem >> 3) % " + S(tiles_m) + ";");
    } else {
      const int64_t per_batch = tiles_n * tiles_m;
      units = g.batch * per_batch;
      fb.line("const int bidx = unit / " + S(per_batch) + ";");
      fb.line("const int rem = unit % " + S(per_batch) + ";");
      fb.line("const int tile_n = rem / " + S(tiles_m) + ";");
      fb.line("const int tile_m = rem % " + S(tiles_m) + ";");
    }
    std::ostringstream call;
    call << "mononn_dev::gemm_tile<" << t.bm << ", " << t.bn << ", " << t.wm << ", " << t.wn << ", " << t.wk << ", " << g.K << ", "
         << (g.b_packed ? "true" : "false") << ">(" << pa << " + (long)bidx * " << g.a_batch_stride << ", " << pb << " + (long)bidx * "
         << g.b_batch_stride << ", " << g.M << ", " << g.N << ", " << g.K << ", " << g.K << ", bidx, tile_m, tile_n, epi, smem);";
    fb.line(call.str());
    if (t.wk > 1) smem = ls.waves() * (t.bm / t.wm / 16) * (t.bn / t.wn / 16) * 64 * 16;
  } else {
    const int64_t total = g.batch * g.M * g.N;
    units = (total + ls.block_size - 1) / ls.block_size;
    fb.line("const long e = (long)unit * " + S(ls.block_size) + " + threadIdx.x;");
    fb.open("if (e < " + S(total) + "L)");
    fb.line("const int bidx = (int)(e / " + S(g.M * g.N) + ");");
    fb.line("const int m = (int)((e / " + S(g.N) + ") % " + S(g.M) + ");");
    fb.line("const int n = (int)(e % " + S(g.N) + ");");
    std::ostringstream call;
    call << "mononn_dev::gemm_naive_element(" << pa << " + (long)bidx * " << g.a_batch_stride << ", " << pb << " + (long)bidx * "
         << g.b_batch_stride << ", " << g.K << ", " << (g.a_k_contig ? g.K : 1) << ", " << (g.a_k_contig ? 1 : g.M) << ", "
         << (g.b_k_contig ? 1 : g.N) << ", " << (g.b_k_contig ? g.K : 1) << ", bidx, m, n, epi);";
    fb.line(call.str());
    fb.close();
  }
  return finish(fb.text(), ptrs, em, units, smem, pre);
}

}  // namespace

NodeFunction generate_gemm(const Program& prog, const Node& node, const LaunchShape& ls, const GemmTuning& t) {
  return gen_gemm(prog, node.members, node.outputs, node.gemm, ls, t);
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
