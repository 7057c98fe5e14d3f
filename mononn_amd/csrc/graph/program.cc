#include "graph/program.h"

#include <algorithm>
#include <functional>
#include <sstream>

#include "codegen/cluster_codegen.h"
#include "common/status.h"

namespace mononn {
namespace graph {

using hlo::Instr;

bool is_alias_op(const Instr* ins) { return ins->opcode == "bitcast" || ins->opcode == "reshape"; }

const Instr* Program::storage_root(const Instr* v) const {
  while (is_alias_op(v)) v = v->operands[0];
  return v;
}

const Node* Program::node_of(const Instr* member) const {
  for (auto& n : nodes)
    for (auto* m : n.members)
      if (m == member) return &n;
  return nullptr;
}

std::string GemmDesc::problem_hash() const {
  std::ostringstream os;
  os << (f32 ? "f32_b" : bf16 ? "bf16_b" : "f16_b") << batch << "_m" << M << "_n" << N << "_k" << K << (a_k_contig ? "_ak" : "_am") << (b_packed ? "_bp" : (b_k_contig ? "_bk" : "_bn"));
  if (is_conv) os << "_conv" << conv.R << "x" << conv.S << "s" << conv.stride_h << "x" << conv.stride_w << "p" << conv.pad_h << "x" << conv.pad_w;
  return os.str();
}

std::string Program::summary() const {
  std::ostringstream os;
  os << "stages=" << num_stages << " nodes=" << nodes.size() << " temp_bytes=" << temp_bytes << "\n";
  for (auto& n : nodes) {
    os << "  stage " << n.stage << "  " << (n.kind == NodeKind::kGemm ? "gemm   " : n.kind == NodeKind::kAttention ? "attn   " : (n.row_program ? "rowred " : "elewise")) << " " << n.name;
    if (n.kind == NodeKind::kGemm) os << "  [" << n.gemm.problem_hash() << "] members=" << n.members.size() << (n.prologue.empty() ? "" : (n.prologue_stores ? " +row-prologue(stores)" : " +row-prologue"));
    else if (n.kind == NodeKind::kAttention) os << "  [" << n.gemm.problem_hash() << " -> " << n.gemm2.problem_hash() << "] members=" << n.members.size();
    else os << "  members=" << n.members.size() << (n.row_program ? " rows=" + std::to_string(n.rows) + " len=" + std::to_string(n.row_len) : "");
    os << "\n";
  }
  return os.str();
}

namespace {

struct Builder {
  Program& p;
  const BuildOptions& opt;
  std::vector<Node> nodes;
  std::map<const Instr*, int> node_of_member;   // entry instr -> index in nodes (alive)
  std::set<std::string> absorb;                 // GEMMs (canonical names) an attention node is going to take in
  std::set<std::string> absorbed;               // ... and those it did take in

  bool enabled(const char* pass) const { return !opt.disabled_passes.count(pass); }

  // value defined by a member of node `n`?  (a fusion member defines its get-tuple-elements too)
  const Instr* defining_member(const Instr* root) const {
    if (root->opcode == "get-tuple-element") return root->operands[0];
    return root;
  }

  GemmDesc describe_gemm(const Instr* g) {
    // dimension bookkeeping of GemmImpl::setup (gemm_impl.cc:233-499)
    MONONN_CHECK(g->operands.size() == 2 || g->operands.size() == 3, kUnsupported) << g->hlo_name << ": GEMM takes 2 or 3 operands";
    const hlo::Shape &A = g->operands[0]->shape, &B = g->operands[1]->shape, &D = g->shape;
    MONONN_CHECK(A.rank() == B.rank() && A.rank() == D.rank() && A.rank() >= 2, kUnsupported) << g->hlo_name << ": A, B and D must have equal rank >= 2";
    // f16 x f16 -> f16 and f32 x f32 -> f32, both with fp32 accumulation (the reference: half and float / TF32,
    // gemm_impl.cc:56, :229)
    const bool all_f16 = A.dtype == hlo::DType::kF16 && B.dtype == hlo::DType::kF16 && D.dtype == hlo::DType::kF16;
    const bool all_f32 = A.dtype == hlo::DType::kF32 && B.dtype == hlo::DType::kF32 && D.dtype == hlo::DType::kF32;
    // bf16 x bf16 -> bf16 (not in the reference, whose CUTLASS instantiations are half and float): the same tiles on the
    // bf16 forms of the MFMAs
    const bool all_bf16 = A.dtype == hlo::DType::kBF16 && B.dtype == hlo::DType::kBF16 && D.dtype == hlo::DType::kBF16;
    MONONN_CHECK(all_f16 || all_f32 || all_bf16, kUnsupported) << g->hlo_name << ": GEMM operands and result must all be f16, all be bf16 or all be f32";
    MONONN_CHECK(g->operands.size() == 2 || g->operands[2]->shape.dtype == D.dtype, kUnsupported) << g->hlo_name << ": addend type differs from the result type";
    const int r = A.rank();
    const hlo::GemmConfig& c = g->gemm;
    GemmDesc d;
    d.f32 = all_f32;
    d.bf16 = all_bf16;
    MONONN_CHECK(c.lhs_contracting == r - 1 || c.lhs_contracting == r - 2, kUnsupported) << g->hlo_name << ": lhs contracting dim must be one of the two minor dims";
    MONONN_CHECK(c.rhs_contracting == r - 1 || c.rhs_contracting == r - 2, kUnsupported) << g->hlo_name << ": rhs contracting dim must be one of the two minor dims";
    d.a_k_contig = c.lhs_contracting == r - 1;
    d.b_k_contig = c.rhs_contracting == r - 1;
    d.K = A.dims[c.lhs_contracting];
    d.M = A.dims[d.a_k_contig ? r - 2 : r - 1];
    d.N = B.dims[d.b_k_contig ? r - 2 : r - 1];
    MONONN_CHECK(B.dims[c.rhs_contracting] == d.K, kInvalidArgument) << g->hlo_name << ": contracting extents differ";
    MONONN_CHECK(D.dims[r - 2] == d.M && D.dims[r - 1] == d.N, kInvalidArgument) << g->hlo_name << ": result shape does not match operands";
    d.batch = 1;
    for (int i = 0; i < r - 2; ++i) {
      MONONN_CHECK(A.dims[i] == B.dims[i] && A.dims[i] == D.dims[i], kUnsupported) << g->hlo_name << ": batch dims must agree";
      d.batch *= A.dims[i];
    }
    MONONN_CHECK(d.batch == c.batch_size, kInvalidArgument) << g->hlo_name << ": batch_size " << c.batch_size << " does not match the shapes (" << d.batch << ")";
    d.a_batch_stride = d.M * d.K;
    d.b_batch_stride = d.N * d.K;
    d.d_batch_stride = d.M * d.N;
    // cross-check against XLA's strides as the reference does (gemm_impl.cc:380-393)
    if (d.batch > 1) {
      MONONN_CHECK(c.lhs_stride == 0 || c.lhs_stride == d.a_batch_stride, kInvalidArgument) << g->hlo_name << ": lhs_stride mismatch";
      MONONN_CHECK(c.rhs_stride == 0 || c.rhs_stride == d.b_batch_stride, kInvalidArgument) << g->hlo_name << ": rhs_stride mismatch";
    }
    MONONN_CHECK(c.alpha_imag == 0, kUnsupported) << g->hlo_name << ": complex alpha";
    d.alpha = c.alpha_real;
    d.beta = c.beta;
    d.has_addend = g->operands.size() == 3 && c.beta != 0;
    return d;
  }

  GemmDesc describe_conv(const Instr* g) {
    const hlo::ConvConfig& c = g->conv;
    GemmDesc d;
    d.is_conv = true;
    d.conv = c;
    d.bf16 = g->operands[0]->shape.dtype == hlo::DType::kBF16;   // the same tiles on the bf16 forms of the MFMAs
    d.batch = 1;
    d.M = c.N * c.P * c.Q;
    d.N = c.K;
    d.K = c.R * c.S * c.C;
    d.a_k_contig = true;
    d.b_k_contig = true;
    d.alpha = c.result_scale;
    d.a_batch_stride = d.b_batch_stride = d.d_batch_stride = 0;
    return d;
  }

  void make_nodes() {
    const hlo::Computation* e = p.module->entry;
    for (auto& up : e->instrs) {
      const Instr* ins = up.get();
      const std::string& op = ins->opcode;
      if (op == "parameter") continue;
      if (op == "constant") continue;
      if (is_alias_op(ins) || op == "get-tuple-element" || op == "tuple") continue;
      Node n;
      n.name = ins->name;
      n.members.push_back(ins);
      if (op == "custom-call" || op == "dot") {
        n.kind = NodeKind::kGemm;
        n.gemm = ins->is_conv() ? describe_conv(ins) : describe_gemm(ins);
      } else {
        n.kind = NodeKind::kCluster;
      }
      node_of_member[ins] = static_cast<int>(nodes.size());
      nodes.push_back(std::move(n));
    }
  }

  static std::vector<const Instr*> with_prologue(const Node& n) {
    std::vector<const Instr*> v = n.prologue;
    v.insert(v.end(), n.members.begin(), n.members.end());
    return v;
  }

  // storage roots read by a set of members from outside the set
  std::vector<const Instr*> external_inputs(const std::vector<const Instr*>& members) const {
    std::set<const Instr*> in_set(members.begin(), members.end());
    std::vector<const Instr*> out;
    std::set<const Instr*> seen;
    for (auto* m : members)
      for (auto* o : m->operands) {
        const Instr* r = p.storage_root(o);
        if (in_set.count(defining_member(r))) continue;
        if (r->opcode == "constant" && r->is_scalar_constant()) continue;
        if (seen.insert(r).second) out.push_back(r);
      }
    return out;
  }

  // node indices a member set depends on (producers of its external inputs)
  std::set<int> producer_nodes(const std::vector<const Instr*>& members) const {
    std::set<int> s;
    for (auto* r : external_inputs(members)) {
      auto it = node_of_member.find(defining_member(r));
      if (it != node_of_member.end()) s.insert(it->second);
    }
    return s;
  }

  // does node `from` reach node `to` through a path that leaves the set {from}?
  bool reaches_via_outside(int from, int to, const std::vector<std::vector<int>>& succ) const {
    std::vector<int> stack;
    std::set<int> seen;
    for (int s : succ[from])
      if (s != to) stack.push_back(s);
    while (!stack.empty()) {
      int x = stack.back();
      stack.pop_back();
      if (!seen.insert(x).second) continue;
      if (x == to) return true;
      for (int s : succ[x]) stack.push_back(s);
    }
    return false;
  }

  std::vector<std::vector<int>> successors() const {
    std::vector<std::vector<int>> succ(nodes.size());
    for (size_t i = 0; i < nodes.size(); ++i) {
      if (nodes[i].members.empty()) continue;
      for (int pn : producer_nodes(with_prologue(nodes[i]))) succ[pn].push_back(static_cast<int>(i));
    }
    return succ;
  }

  // MergeDependentPass counterpart: glue a cluster onto the cluster that feeds it when the merged
  // body can still be generated as one loop nest (same row space).  Feasibility is decided by the
  // code generator itself on a dry run.
  void merge_dependent() {
    bool changed = true;
    while (changed) {
      changed = false;
      auto succ = successors();
      for (size_t ci = 0; ci < nodes.size() && !changed; ++ci) {
        Node& c = nodes[ci];
        if (c.members.empty() || c.kind != NodeKind::kCluster) continue;
        for (int pi : producer_nodes(c.members)) {
          Node& pr = nodes[pi];
          if (pr.kind != NodeKind::kCluster) continue;
          if (reaches_via_outside(pi, static_cast<int>(ci), succ)) continue;
          std::vector<const Instr*> merged = pr.members;
          merged.insert(merged.end(), c.members.begin(), c.members.end());
          std::sort(merged.begin(), merged.end(), [](const Instr* a, const Instr* b) { return a->index_in_comp < b->index_in_comp; });
          if (!codegen::can_merge_clusters(p, pr.members, c.members, merged)) continue;
          pr.members = merged;
          pr.name += "_" + c.name;
          for (auto* m : c.members) node_of_member[m] = pi;
          c.members.clear();
          changed = true;
          break;
        }
      }
    }
  }

  // A GEMM absorbs element-wise clusters that consume its result element for element; they run in
  // the epilogue on the fp32 accumulator tile (bias, GELU, residual, head split/merge transposes).
  void fuse_gemm_epilogues() {
    bool changed = true;
    while (changed) {
      changed = false;
      auto succ = successors();
      for (size_t gi = 0; gi < nodes.size() && !changed; ++gi) {
        Node& g = nodes[gi];
        if (g.members.empty() || g.kind != NodeKind::kGemm) continue;
        if (opt.gemm_split_k.count(g.members[0]->name) && opt.gemm_split_k.at(g.members[0]->name) > 1) continue;   // epilogue moves to the consumer
        if (absorb.count(g.members[0]->name)) continue;   // likewise
        for (int ci : succ[gi]) {
          Node& c = nodes[ci];
          if (c.members.empty() || c.kind != NodeKind::kCluster) continue;
          if (reaches_via_outside(static_cast<int>(gi), ci, succ)) continue;
          std::vector<const Instr*> merged = g.members;
          merged.insert(merged.end(), c.members.begin(), c.members.end());
          if (!codegen::can_fuse_epilogue(p, g.members, c.members)) continue;
          g.members = merged;
          g.name += "_" + c.name;
          for (auto* m : c.members) node_of_member[m] = static_cast<int>(gi);
          c.members.clear();
          changed = true;
          break;
        }
      }
    }
  }

  // may the kernel keep the right-hand GEMM operand `root` ([.., K, N]) transposed in memory?
  bool can_store_k_contig(const Instr* root, const Instr* operand, int rhs_contracting) const {
    if (root->opcode == "parameter" || root->opcode == "constant") return false;
    if (root->shape.dims != operand->shape.dims) return false;   // reached through a reshaping alias
    for (auto* u : root->users) {
      if (is_alias_op(u)) return false;
      bool as_b = u->is_gemm() && u->operands[1] == root && u->operands[0] != root &&
                  (u->operands.size() < 3 || u->operands[2] != root) && u->gemm.rhs_contracting == rhs_contracting;
      if (!as_b) return false;
    }
    const Instr* mroot = p.module->entry->root;
    if (mroot == root) return false;
    if (mroot->opcode == "tuple")
      for (auto* o : mroot->operands)
        if (p.storage_root(o) == root) return false;
    return true;
  }

  // A row program whose single product is the left operand of GEMMs (LayerNorm in front of the QKV /
  // FFN projections) moves into those GEMMs: every workgroup normalises the rows of its own A panel in
  // registers, so the stage of the row program and its barrier disappear.  One of the GEMMs keeps
  // writing the product for consumers in later stages (the residual connection).
  void fuse_gemm_prologues() {
    for (size_t ri = 0; ri < nodes.size(); ++ri) {
      Node& r = nodes[ri];
      if (r.members.empty() || r.kind != NodeKind::kCluster) continue;
      auto outs = codegen::external_outputs(p, r.members);
      if (outs.size() != 1) continue;
      // a row program that adds up the partial sums of a split-K GEMM stays a stage of its own
      bool reads_split = false;
      for (auto* in : external_inputs(r.members)) {
        // partial sums of a split GEMM reach the row program through the element emitter, fused or not; with
        // LayerNorm folding on, a row program that adds them up stays a stage (the fold needs the finished rows, and
        // the split is worth more than the stage: every column tile would re-read all partial sums)
        auto sk = opt.gemm_split_k.find(in->name);
        if (opt.fold_layer_norm && sk != opt.gemm_split_k.end() && sk->second > 1) reads_split = true;
        reads_split = reads_split || absorbed.count(in->name);
      }
      if (reads_split) continue;
      const Instr* h = outs[0];
      auto succ = successors();
      std::vector<int> takers;
      for (int ci : succ[ri]) {
        Node& c = nodes[ci];
        if (c.kind != NodeKind::kGemm || !c.prologue.empty() || c.gemm.is_conv || c.gemm.f32) continue;
        const Instr* g = c.members[0];
        if (p.storage_root(g->operands[0]) != h || p.storage_root(g->operands[1]) == h) continue;
        if (g->operands.size() > 2 && p.storage_root(g->operands[2]) == h) continue;
        bool reads_h_elsewhere = false;   // e.g. the epilogue of the same GEMM reading the row program's product
        for (size_t k = 1; k < c.members.size(); ++k)
          for (auto* o : c.members[k]->operands)
            if (p.storage_root(o) == h) reads_h_elsewhere = true;
        if (reads_h_elsewhere) continue;
        if (!codegen::can_fuse_prologue(p, r.members, c.members, c.gemm)) continue;
        takers.push_back(ci);
      }
      if (takers.empty()) continue;
      // consumers that cannot take the row program in must come strictly later, i.e. read the stored copy;
      // they may not be the GEMMs' own producers
      bool conflict = false;
      for (int ci : succ[ri]) {
        if (std::find(takers.begin(), takers.end(), ci) != takers.end()) continue;
        for (int t : takers)
          if (reaches_via_outside(ci, t, succ) || ci == t) conflict = true;
        for (int pn : producer_nodes(with_prologue(nodes[takers[0]])))
          if (pn == ci) conflict = true;
      }
      if (conflict) continue;
      for (size_t k = 0; k < takers.size(); ++k) {
        Node& c = nodes[takers[k]];
        c.prologue = r.members;
        c.prologue_stores = k == 0;
        c.name = r.name + "_" + c.name;
      }
      for (auto* m : r.members) node_of_member[m] = takers[0];
      r.members.clear();
    }
  }

  // GEMM -> row program -> GEMM (attention): the row program's only product feeds the second GEMM as
  // its left operand, and the first GEMM's result is read by nothing else.
  void fuse_attention() {
    bool changed = true;
    while (changed) {
      changed = false;
      auto succ = successors();
      for (size_t ri = 0; ri < nodes.size() && !changed; ++ri) {
        Node& r = nodes[ri];
        if (r.members.empty() || r.kind != NodeKind::kCluster) continue;
        // producer GEMM
        int g1i = -1;
        bool ok = true;
        for (int pn : producer_nodes(r.members)) {
          if (nodes[pn].kind == NodeKind::kGemm) {
            if (g1i >= 0) ok = false;
            g1i = pn;
          }
        }
        if (!ok || g1i < 0) continue;
        Node& g1 = nodes[g1i];
        if (g1.members.size() != 1 || succ[g1i].size() != 1 || succ[g1i][0] != static_cast<int>(ri)) continue;
        if (succ[ri].size() != 1) continue;
        int g2i = succ[ri][0];
        Node& g2 = nodes[g2i];
        if (g2.kind != NodeKind::kGemm) continue;
        const Instr* gi1 = g1.members[0];
        const Instr* gi2 = g2.members[0];
        auto outs = codegen::external_outputs(p, r.members);
        if (outs.size() != 1 || p.storage_root(gi2->operands[0]) != outs[0] || p.storage_root(gi2->operands[1]) == outs[0]) continue;
        if (reaches_via_outside(g1i, static_cast<int>(ri), succ) || reaches_via_outside(static_cast<int>(ri), g2i, succ)) continue;
        // the other producers of gemm2 (V) must not depend on gemm1 / the row program
        const GemmDesc &d1 = g1.gemm, &d2 = g2.gemm;
        if (!d1.a_k_contig || !d1.b_k_contig || !d2.a_k_contig || d2.has_addend || d1.has_addend || d1.is_conv || d2.is_conv || d1.f32 || d2.f32) continue;
        if (d2.batch != d1.batch || d2.M != d1.M || d2.K != d1.N) continue;
        // key counts off the MFMA step are taken (rounded up per wave, masked); head sizes are not
        if (d1.K % 32 != 0 || d1.N < 32 || d2.N % 16 != 0 || d1.N > 512 || d2.N > 256 || d1.K > 256) continue;
        const Instr* vroot = p.storage_root(gi2->operands[1]);
        if (!d2.b_k_contig && !(opt.assign_operand_layouts && enabled("OperandLayoutPass") && can_store_k_contig(vroot, gi2->operands[1], gi2->gemm.rhs_contracting)))
          continue;
        std::vector<const Instr*> epi(g2.members.begin() + 1, g2.members.end());
        if (!codegen::can_fuse_attention(p, gi1, d1, r.members, gi2, d2, epi)) continue;
        Node a;
        a.kind = NodeKind::kAttention;
        a.name = g1.name + "_" + r.name + "_" + g2.name;
        a.gemm = d1;
        a.gemm2 = d2;
        a.members.push_back(gi1);
        a.members.insert(a.members.end(), r.members.begin(), r.members.end());
        a.gemm2_index = a.members.size();
        a.members.insert(a.members.end(), g2.members.begin(), g2.members.end());
        for (auto* m : a.members) node_of_member[m] = g1i;
        nodes[g1i] = a;
        nodes[ri].members.clear();
        nodes[g2i].members.clear();
        changed = true;
      }
    }
  }


  // GEMMs that directly consume the single output of an attention node with a constant right operand
  std::vector<std::pair<int, int>> out_proj_candidates() const {
    std::vector<std::pair<int, int>> out;
    auto succ = successors();
    for (size_t ai = 0; ai < nodes.size(); ++ai) {
      const Node& a = nodes[ai];
      if (a.members.empty() || a.kind != NodeKind::kAttention || a.gemm3_index != 0 || a.gemm.N % 32 != 0) continue;
      auto outs = codegen::external_outputs(p, a.members);
      if (outs.size() != 1 || succ[ai].size() != 1) continue;
      const Node& g = nodes[succ[ai][0]];
      if (g.kind != NodeKind::kGemm || !g.prologue.empty() || g.gemm.is_conv) continue;
      const Instr* gi = g.members[0];
      if (!gi->is_gemm() || gi->operands.size() != 2 || p.storage_root(gi->operands[0]) != outs[0]) continue;
      const Instr* w = gi->operands[1];
      if (w->opcode != "constant" || w->shape.rank() != 2 || w->users.size() != 1) continue;
      out.emplace_back(static_cast<int>(ai), succ[ai][0]);
    }
    return out;
  }

  void fuse_attention_out_proj() {
    for (auto& pr : out_proj_candidates()) {
      Node& a = nodes[pr.first];
      Node& g = nodes[pr.second];
      const Instr* gi = g.members[0];
      if (!absorb.count(gi->name) || g.members.size() != 1) continue;
      const GemmDesc& d3 = g.gemm;
      const GemmDesc& d2 = a.gemm2;
      if (d3.batch != 1 || !d3.a_k_contig || d3.b_k_contig || d3.has_addend || d3.K % d2.N != 0 || d2.N % 32 != 0 || d3.N % 16 != 0) continue;
      const int64_t heads = d3.K / d2.N;
      if (heads < 1 || d2.batch % heads != 0 || d3.M != d2.batch / heads * d2.M) continue;
      if (gi->operands[1]->shape.dims[0] % 32 != 0 || !opt.transpose_constant_b || !enabled("ConstantLayoutPass")) continue;
      // every reader of the projection must go through the element emitter (it adds up the per-head partial sums)
      bool ok = true;
      for (auto* u : gi->users)
        if (u->is_gemm() || u->opcode == "tuple" || is_alias_op(u)) ok = false;
      if (p.module->entry->root == gi) ok = false;
      if (!ok) continue;
      std::vector<const Instr*> epi(a.members.begin() + a.gemm2_index + 1, a.members.end());
      if (!codegen::can_fuse_out_proj(p, a.members[a.gemm2_index], d2, epi, gi, d3, static_cast<int>(heads))) continue;
      a.gemm3 = d3;
      a.gemm3.split_k = static_cast<int>(heads);
      a.gemm3_index = a.members.size();
      a.heads = static_cast<int>(heads);
      a.members.push_back(gi);
      a.name += "_" + g.name;
      node_of_member[gi] = pr.first;
      g.members.clear();
      absorbed.insert(gi->name);
    }
  }

  void finalize() {
    // compact, compute inputs/outputs, stages, order
    std::vector<Node> alive;
    std::map<int, int> remap;
    for (size_t i = 0; i < nodes.size(); ++i)
      if (!nodes[i].members.empty()) {
        remap[static_cast<int>(i)] = static_cast<int>(alive.size());
        alive.push_back(nodes[i]);
      }
    for (auto& kv : node_of_member) kv.second = remap.at(kv.second);
    nodes = alive;

    // module outputs
    const Instr* root = p.module->entry->root;
    std::vector<const Instr*> outs;
    if (root->opcode == "tuple") outs.assign(root->operands.begin(), root->operands.end());
    else outs.push_back(root);
    std::set<const Instr*> live_set;
    for (auto* o : outs) {
      const Instr* r = p.storage_root(o);
      MONONN_CHECK(!r->shape.is_tuple(), kUnsupported) << "nested tuple output " << o->hlo_name;
      MONONN_CHECK(r->opcode != "parameter" && r->opcode != "constant", kUnsupported) << "module output " << o->hlo_name << " is a pass-through of an input";
      MONONN_CHECK(live_set.insert(r).second, kUnsupported) << "module output " << o->hlo_name << " appears twice in the root tuple";
      p.live_outs.push_back(r);
    }

    // users per storage root (entry level)
    std::map<const Instr*, std::set<int>> readers;
    for (size_t i = 0; i < nodes.size(); ++i) {
      nodes[i].inputs = external_inputs(with_prologue(nodes[i]));
      for (auto* r : nodes[i].inputs) readers[r].insert(static_cast<int>(i));
    }
    // outputs: values defined by a member and read by another node or live-out
    for (size_t i = 0; i < nodes.size(); ++i) {
      Node& n = nodes[i];
      std::set<const Instr*> mem(n.members.begin(), n.members.end());
      std::vector<const Instr*> cands;
      for (auto& up : p.module->entry->instrs) {
        const Instr* v = up.get();
        if (mem.count(v) && !v->shape.is_tuple()) cands.push_back(v);
        if (v->opcode == "get-tuple-element" && mem.count(v->operands[0])) cands.push_back(v);
      }
      for (auto* v : cands)
        if (readers.count(v) || live_set.count(v)) n.outputs.push_back(v);
      if (n.prologue_stores) {
        // the absorbing GEMMs compute the row program's product themselves; `readers` holds everyone else
        bool wanted = false;
        for (auto* v : codegen::external_outputs(p, n.prologue))
          if (readers.count(v) || live_set.count(v)) {
            n.outputs.push_back(v);
            wanted = true;
          }
        n.prologue_stores = wanted;
      }
      MONONN_CHECK(!n.outputs.empty(), kUnsupported) << "node " << n.name << " has no consumer (dead code in the entry computation)";
      for (auto* v : n.outputs) p.producer[v] = static_cast<int>(i);
    }
    // stages: longest path from the sources (BFS-depth rule of the reference's barrier elimination)
    std::vector<int> depth(nodes.size(), 0);
    std::vector<int> order;
    {
      std::vector<int> state(nodes.size(), 0);
      std::function<void(int)> visit = [&](int i) {
        if (state[i] == 2) return;
        MONONN_CHECK(state[i] == 0, kInternal) << "cycle through node " << nodes[i].name;
        state[i] = 1;
        int d = 1;
        for (auto* r : nodes[i].inputs) {
          auto it = p.producer.find(r);
          if (it == p.producer.end()) continue;
          visit(it->second);
          d = std::max(d, depth[it->second] + 1);
        }
        depth[i] = d;
        state[i] = 2;
        order.push_back(i);
      };
      for (size_t i = 0; i < nodes.size(); ++i) visit(static_cast<int>(i));
    }
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return depth[a] < depth[b]; });
    std::vector<Node> sorted;
    std::map<int, int> pos;
    for (int i : order) {
      pos[i] = static_cast<int>(sorted.size());
      nodes[i].stage = depth[i];
      nodes[i].id = static_cast<int>(sorted.size());
      sorted.push_back(nodes[i]);
    }
    for (auto& kv : p.producer) kv.second = pos.at(kv.second);
    p.nodes = sorted;
    p.num_stages = 0;
    for (auto& n : p.nodes) p.num_stages = std::max(p.num_stages, n.stage);
  }

  void decide_constant_layouts() {
    if (!opt.transpose_constant_b || !enabled("ConstantLayoutPass")) return;
    // a constant [K,N] matrix used only as the right operand of GEMMs is stored in fragment order by the host
    std::map<const Instr*, bool> ok;
    for (auto& up : p.module->entry->instrs) {
      const Instr* c = up.get();
      if (c->opcode != "constant" || c->is_scalar_constant() || c->shape.rank() != 2) continue;
      bool all = !c->users.empty();
      for (auto* u : c->users) {
        bool good = u->is_gemm() && u->operands.size() >= 2 && hlo::is_half_float(c->shape.dtype) &&
                    u->operands[1] == c && u->operands[0] != c && u->gemm.rhs_contracting == 0 && c->shape.dims[0] % 32 == 0 &&
                    u->gemm.lhs_contracting == u->operands[0]->shape.rank() - 1 && (u->operands.size() < 3 || u->operands[2] != c);
        if (!good) all = false;
      }
      if (all) ok[c] = true;
    }
    for (auto& n : p.nodes) {
      if (n.kind == NodeKind::kAttention && n.gemm3_index != 0) {
        const Instr* b = n.members[n.gemm3_index]->operands[1];
        MONONN_CHECK(ok.count(b), kInternal) << "weights of the absorbed projection " << n.members[n.gemm3_index]->hlo_name << " cannot be packed";
        n.gemm3.b_packed = true;
        p.constant_transform[b] = ConstantTransform::kPackMfmaB;
        continue;
      }
      if (n.kind != NodeKind::kGemm) continue;
      const Instr* b = n.members[0]->operands[1];
      if (ok.count(b)) {
        n.gemm.b_packed = true;
        p.constant_transform[b] = ConstantTransform::kPackMfmaB;
      }
    }
  }

  // LayoutAssignment: a right-hand GEMM operand [.., K, N] that this kernel produces itself (and that
  // nothing but such GEMMs reads) is stored [.., N, K]; its producer writes through the permutation.
  void assign_operand_layouts() {
    if (!opt.assign_operand_layouts || !enabled("OperandLayoutPass")) return;
    auto each_gemm = [&](auto&& fn) {
      for (auto& n : p.nodes) {
        if (n.kind == NodeKind::kGemm) fn(n.members[0], n.gemm);
        else if (n.kind == NodeKind::kAttention) fn(n.members[n.gemm2_index], n.gemm2);
      }
    };
    each_gemm([&](const Instr* g, GemmDesc& d) {
      if (d.b_k_contig || d.b_packed || !d.a_k_contig) return;
      const Instr* root = p.storage_root(g->operands[1]);
      if (!p.producer.count(root)) return;   // parameter / constant
      if (!can_store_k_contig(root, g->operands[1], g->gemm.rhs_contracting)) return;
      int r = root->shape.rank();
      std::vector<int> perm(r);
      for (int i = 0; i < r; ++i) perm[i] = i;
      std::swap(perm[r - 1], perm[r - 2]);
      p.physical_perm[root] = perm;
    });
    each_gemm([&](const Instr* g, GemmDesc& d) {
      if (p.physical_perm.count(p.storage_root(g->operands[1]))) d.b_k_contig = true;
    });
    if (opt.pack_left_operands && enabled("LeftOperandLayoutPass")) pack_left_operands();
  }

  // Operands that GEMM and attention nodes fetch with their own address arithmetic (not through the element
  // emitter) are stored in MFMA fragment order when this kernel produces them itself and every such node reads
  // them the same way: the left operand [M, K] of a plain MFMA GEMM, and the three operands of a fused attention
  // (queries and keys contracted over their minor dimension, values over the key dimension).
  void pack_left_operands() {
    using Order = Program::TileOrder;
    struct Want {
      int64_t k;
      Order order;
    };
    std::map<const Instr*, Want> want;
    std::set<const Instr*> spoiled;
    std::set<const Instr*> live(p.live_outs.begin(), p.live_outs.end());
    // a use of `operand` as [rows, k] in the given order; `perm_ok`: the root may carry the k-contiguous transposition
    auto use = [&](const Instr* operand, bool fits, int64_t rows, int64_t k, Order order, bool perm_ok) {
      const Instr* root = p.storage_root(operand);
      fits = fits && rows % 16 == 0 && k % 32 == 0 && p.producer.count(root) && !live.count(root) && (perm_ok || !p.physical_perm.count(root)) &&
             hlo::is_half_float(root->shape.dtype) && root->shape.num_elements() == rows * k &&
             (!want.count(root) || (want[root].k == k && want[root].order == order));
      if (fits) want[root] = {k, order};
      else spoiled.insert(root);
    };
    for (auto& n : p.nodes) {
      if (n.kind == NodeKind::kAttention) {
        const GemmDesc& d1 = n.gemm;
        const GemmDesc& d2 = n.gemm2;
        const Instr* g1 = n.members[0];
        const Instr* g2 = n.members[n.gemm2_index];
        const bool dense = d1.a_k_contig && d1.b_k_contig && d2.b_k_contig && d1.a_batch_stride == d1.M * d1.K && d1.b_batch_stride == d1.N * d1.K &&
                           d2.b_batch_stride == d2.N * d2.K && d1.M % 16 == 0 && d1.N % 16 == 0 && d2.N % 16 == 0;
        use(g1->operands[0], dense, d1.batch * d1.M, d1.K, Order::kRunsOf8, false);
        // a key count off the MFMA step leaves the last fragments partly empty: keys and values are then read in
        // place, row by row, with the rows past the end clamped
        const bool whole_steps = d1.N % 32 == 0;
        use(g1->operands[1], dense && whole_steps, d1.batch * d1.N, d1.K, Order::kRunsOf8, false);
        // values: stored [.., N2, keys] (transposed by the operand layout pass), contracted over the keys
        use(g2->operands[1], dense && whole_steps && p.physical_perm.count(p.storage_root(g2->operands[1])), d2.batch * d2.N, d2.K, Order::kPairsOf4, true);
        continue;
      }
      if (n.kind != NodeKind::kGemm) continue;
      const Instr* g = n.members[0];
      const GemmDesc& d = n.gemm;
      spoiled.insert(p.storage_root(g->operands[1]));
      const bool mfma = d.a_k_contig && (d.b_k_contig || d.b_packed) && d.K % 32 == 0;
      if (!n.prologue.empty()) {
        // the tile loads the rows of the row program's primary input in place of the left operand
        const Instr* primary = codegen::prologue_primary(p, n.prologue, d.M, d.K);
        if (primary) use(primary, mfma && d.batch == 1, d.M, d.K, Order::kRunsOf8, false);
        continue;
      }
      use(g->operands[0], mfma && !d.is_conv && d.batch == 1, d.M, d.K, Order::kRunsOf8, false);
    }
    // Partial sums of a split GEMM that a fused row program takes row fragment by row fragment: same order, fp32.
    for (auto& n : p.nodes) {
      if (n.kind != NodeKind::kGemm || n.prologue.empty()) continue;
      for (auto* r : n.inputs) {
        auto sk = p.split_k.find(r);
        if (sk == p.split_k.end() || p.physical_tile.count(r) || r->shape.rank() != 2) continue;
        const int64_t M = r->shape.dims[0], N = r->shape.dims[1];
        if (M == n.gemm.M && N == n.gemm.K && M % 16 == 0 && N % 32 == 0) p.physical_tile[r] = {N, Order::kRunsOf8};
      }
    }
    for (auto& kv : want)
      if (!spoiled.count(kv.first)) p.physical_tile[kv.first] = {kv.second.k, kv.second.order};
    auto tiled = [&](const Instr* operand) { return p.physical_tile.count(p.storage_root(operand)) > 0; };
    for (auto& n : p.nodes) {
      if (n.kind == NodeKind::kGemm) {
        // with a row program in front, the tile loads that program's primary input in place of the left operand
        const Instr* a = n.prologue.empty() ? n.members[0]->operands[0] : codegen::prologue_primary(p, n.prologue, n.gemm.M, n.gemm.K);
        n.gemm.a_packed = a != nullptr && tiled(a);
      } else if (n.kind == NodeKind::kAttention) {
        n.gemm.a_packed = tiled(n.members[0]->operands[0]);
        n.gemm.b_tiled = tiled(n.members[0]->operands[1]);
        n.gemm2.b_tiled = tiled(n.members[n.gemm2_index]->operands[1]);
      }
    }
  }

  // LayerNorm prologues of GEMMs with constant, packed weights that nothing else reads: folded (program.h).
  void fold_layer_norms() {
    if (!opt.fold_layer_norm || !enabled("LayerNormFoldingPass")) return;
    for (auto& n : p.nodes) {
      if (n.kind != NodeKind::kGemm || n.prologue.empty() || !n.gemm.b_packed || n.gemm.batch != 1 || n.gemm.alpha != 1.0 || n.gemm.has_addend) continue;
      const Instr* g = n.members[0];
      const Instr* w = p.storage_root(g->operands[1]);
      if (w->opcode != "constant" || w->shape.dtype != hlo::DType::kF16 || w->shape.dims != std::vector<int64_t>({n.gemm.K, n.gemm.N})) continue;
      if (w->users.size() != 1 || p.constant_row_scale.count(w)) continue;
      LayerNormFold f;
      if (!codegen::match_prologue_layer_norm(p, n.prologue, p.storage_root(g->operands[0]), n.gemm.M, n.gemm.K, &f.gamma, &f.beta, &f.eps)) continue;
      auto column_sums = [&](const char* suffix, const Instr* vec) {
        auto c = std::make_unique<hlo::Instr>();
        c->name = w->name + suffix;
        c->hlo_name = w->hlo_name + suffix;
        c->opcode = "constant";
        c->shape.dtype = hlo::DType::kF32;
        c->shape.dims = {n.gemm.N};
        c->shape.minor_to_major = {0};
        c->literal = "{...}";
        c->literal_elided = true;
        c->parent = const_cast<hlo::Computation*>(w->parent);
        const Instr* raw = c.get();
        p.derived_constants[raw] = {w, vec};
        p.synthetic.push_back(std::move(c));
        return raw;
      };
      f.colsum_gamma = column_sums("_ln_gamma_sums", f.gamma);
      f.colsum_beta = column_sums("_ln_beta_sums", f.beta);
      p.constant_row_scale[w] = f.gamma;
      n.ln_fold = f;
    }
  }

  void apply_split_k() {
    // a projection absorbed by an attention node leaves it as one partial sum per head
    for (auto& n : p.nodes)
      if (n.kind == NodeKind::kAttention && n.gemm3_index != 0) p.split_k[n.members[n.gemm3_index]] = n.heads;
    for (auto& kv : opt.gemm_split_k) {
      if (kv.second <= 1) continue;
      Node* node = nullptr;
      for (auto& n : p.nodes)
        if (n.kind == NodeKind::kGemm && n.members[0]->name == kv.first) node = &n;
      MONONN_CHECK(node != nullptr, kSpecError) << "split_k names GEMM '" << kv.first << "' which is not a GEMM node of the graph";
      const Instr* g = node->members[0];
      MONONN_CHECK(node->members.size() == 1 && node->prologue.empty() && !node->gemm.has_addend && !node->gemm.is_conv && !node->gemm.f32, kSpecError)
          << "split_k: GEMM " << kv.first << " has a fused epilogue / prologue / addend, is a convolution or an f32 GEMM";
      MONONN_CHECK(node->gemm.K % (32 * kv.second) == 0, kSpecError) << "split_k: K of " << kv.first << " is not a multiple of 32 * " << kv.second;
      for (auto* lo : p.live_outs) MONONN_CHECK(lo != g, kSpecError) << "split_k: the result of " << kv.first << " is a module output";
      for (auto& n : p.nodes)
        for (auto* r : n.inputs)
          if (r == g) {
            bool via_emitter = n.kind == NodeKind::kCluster;
            if (n.kind == NodeKind::kGemm) {   // allowed inside an epilogue, not as a matrix operand
              via_emitter = p.storage_root(n.members[0]->operands[0]) != g && p.storage_root(n.members[0]->operands[1]) != g;
            }
            MONONN_CHECK(via_emitter, kSpecError) << "split_k: " << kv.first << " is read by " << n.name << " as a matrix operand";
          }
      node->gemm.split_k = kv.second;
      p.split_k[g] = kv.second;
    }
  }

  void assign_buffers() {
    const hlo::Computation* e = p.module->entry;
    for (auto* prm : e->params) {
      MONONN_CHECK(!prm->shape.is_tuple(), kUnsupported) << "tuple-shaped entry parameter " << prm->hlo_name;
      p.parameters.push_back(prm);
      Buffer b;
      b.kind = Buffer::kParameter;
      b.index = static_cast<int>(prm->parameter_number);
      b.bytes = prm->shape.byte_size();
      p.buffers[prm] = b;
    }
    for (auto& up : e->instrs) {
      const Instr* c = up.get();
      if (c->opcode != "constant" || c->is_scalar_constant()) continue;
      if (c->users.empty()) continue;
      Buffer b;
      b.kind = Buffer::kConstant;
      b.index = static_cast<int>(p.constants.size());
      b.bytes = c->shape.byte_size();
      p.constants.push_back(c);
      p.buffers[c] = b;
    }
    for (auto& up : p.synthetic) {
      Buffer b;
      b.kind = Buffer::kConstant;
      b.index = static_cast<int>(p.constants.size());
      b.bytes = up->shape.byte_size();
      p.constants.push_back(up.get());
      p.buffers[up.get()] = b;
    }
    std::map<const Instr*, int> live_index;
    for (size_t i = 0; i < p.live_outs.size(); ++i) live_index[p.live_outs[i]] = static_cast<int>(i);
    // temp intervals
    std::vector<const Instr*> temps;
    for (auto& n : p.nodes)
      for (auto* v : n.outputs) {
        Buffer b;
        b.bytes = v->shape.byte_size();
        auto sk = p.split_k.find(v);
        if (sk != p.split_k.end()) b.bytes = v->shape.num_elements() * 4 * sk->second;
        b.def_stage = b.last_use_stage = n.stage;
        auto li = live_index.find(v);
        if (li != live_index.end()) {
          b.kind = Buffer::kLiveOut;
          b.index = li->second;
        } else {
          b.kind = Buffer::kTemp;
          temps.push_back(v);
        }
        p.buffers[v] = b;
      }
    for (auto& n : p.nodes)
      for (auto* r : n.inputs) {
        auto it = p.buffers.find(r);
        MONONN_CHECK(it != p.buffers.end(), kInternal) << "input " << r->hlo_name << " of node " << n.name << " has no buffer";
        it->second.last_use_stage = std::max(it->second.last_use_stage, n.stage);
      }
    // interval colouring over stages; a slot is reusable from the stage after its last reader
    struct Slot {
      int64_t offset, bytes;
      int free_from;
    };
    std::vector<Slot> slots;
    int64_t top = 0;
    std::stable_sort(temps.begin(), temps.end(), [&](const Instr* a, const Instr* b) { return p.buffers[a].def_stage < p.buffers[b].def_stage; });
    for (auto* v : temps) {
      Buffer& b = p.buffers[v];
      int64_t need = (b.bytes + 255) / 256 * 256;
      int best = -1;
      for (size_t s = 0; opt.reuse_temp_slots && s < slots.size(); ++s)
        if (slots[s].free_from <= b.def_stage && slots[s].bytes >= need && (best < 0 || slots[s].bytes < slots[best].bytes)) best = static_cast<int>(s);
      if (best >= 0) {
        b.offset = slots[best].offset;
        slots[best].free_from = b.last_use_stage + 1;
      } else {
        b.offset = top;
        slots.push_back({top, need, b.last_use_stage + 1});
        top += need;
      }
    }
    p.temp_bytes = top;
  }
};

}  // namespace

std::unique_ptr<Program> build_program(std::unique_ptr<hlo::Module> module, const BuildOptions& opt) {
  auto prog = std::make_unique<Program>();
  prog->module = std::move(module);
  auto run_fusions = [&](Builder& b) {
    b.make_nodes();
    // epilogues first: a bias + residual fusion behind a GEMM belongs to that GEMM, not to the LayerNorm
    // row program that follows it
    if (opt.fuse_gemm_epilogue && b.enabled("GemmEpilogueFusionPass")) b.fuse_gemm_epilogues();
    if (opt.merge_dependent && b.enabled("MergeDependentPass")) b.merge_dependent();
    if (opt.fuse_attention && b.enabled("AttentionFusionPass")) b.fuse_attention();
  };
  // An output projection that an attention node can absorb must keep its epilogue out of the GEMM (it moves
  // into the consuming row program), which has to be known before the epilogue pass runs: a first trial run
  // of the fusion passes finds the candidates, a second one proves them, the third is the real one.
  std::set<std::string> take;
  const bool want_out_proj = opt.fuse_attention_out_proj && opt.fuse_attention && Builder{*prog, opt, {}, {}, {}, {}}.enabled("AttentionOutProjFusionPass");
  if (want_out_proj) {
    Builder probe{*prog, opt, {}, {}, {}, {}};
    run_fusions(probe);
    std::set<std::string> cand;
    for (auto& pr : probe.out_proj_candidates()) cand.insert(probe.nodes[pr.second].members[0]->name);
    if (!cand.empty()) {
      Builder trial{*prog, opt, {}, {}, cand, {}};
      run_fusions(trial);
      trial.fuse_attention_out_proj();
      take = trial.absorbed;
    }
  }
  Builder b{*prog, opt, {}, {}, take, {}};
  run_fusions(b);
  if (!take.empty()) b.fuse_attention_out_proj();
  if (opt.fuse_gemm_prologue && b.enabled("GemmPrologueFusionPass")) b.fuse_gemm_prologues();
  b.finalize();
  b.decide_constant_layouts();
  b.fold_layer_norms();
  b.apply_split_k();
  b.assign_operand_layouts();
  for (auto& n : prog->nodes)
    if (n.kind == NodeKind::kCluster) codegen::classify_cluster(*prog, n);
  b.assign_buffers();
  return prog;
}

}  // namespace graph
}  // namespace mononn
