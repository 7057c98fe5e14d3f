#include "codegen/kernel_codegen.h"

#include "codegen/host_codegen.h"

#include <algorithm>
#include <cstdlib>
#include <functional>
#include <set>
#include <sstream>

#include "codegen/cluster_codegen.h"
#include "common/status.h"
#include "common/env.h"
#include "device/prelude_text.h"

namespace mononn {
namespace codegen {

using graph::Buffer;
using graph::Node;
using graph::NodeKind;

graph::BuildOptions build_options_from(const spec::GraphSpecification& s) {
  graph::BuildOptions o;
  o.merge_dependent = s.hip.merge_dependent;
  o.fuse_gemm_epilogue = s.hip.gemm_epilogue_fusion;
  o.transpose_constant_b = s.hip.transpose_constant_b;
  o.assign_operand_layouts = s.hip.assign_operand_layouts;
  o.fuse_attention = s.hip.fuse_attention;
  o.fuse_gemm_prologue = s.hip.gemm_prologue_fusion;
  o.fold_layer_norm = s.hip.layer_norm_folding;
  o.pack_left_operands = s.hip.pack_left_operands;
  o.fuse_attention_out_proj = s.hip.attention_out_proj_fusion;
  o.reuse_temp_slots = s.hip.barrier != "flags_coherent";   // the fence-free barrier needs write-once addresses
  for (auto& kv : s.gemm_spec_list)
    if (kv.second.split_k > 1) o.gemm_split_k[kv.first] = kv.second.split_k;
  for (auto& p : env::disabled_passes()) o.disabled_passes.insert(p);
  return o;
}

namespace {
// where a pointer argument of a node function comes from
struct Operand {
  std::string abs = "nullptr";   // module global (constants)
  int base = -1;                 // >= 0: kernel argument ordinal (parameters, then live-outs, then temp)
  int64_t off = 0;
  std::string ctype;             // pointer type at the call site
};

Operand make_operand(const graph::Program& prog, const hlo::Instr* root, bool is_output, hlo::DType elem,
                     const std::map<const hlo::Instr*, std::string>& const_symbol, size_t n_params, size_t n_liveouts) {
  auto it = prog.buffers.find(root);
  MONONN_CHECK(it != prog.buffers.end(), kInternal) << "no buffer for " << root->hlo_name;
  const Buffer& b = it->second;
  Operand o;
  o.ctype = std::string(is_output ? "" : "const ") + hlo::dtype_ctype(elem) + "*";
  switch (b.kind) {
    case Buffer::kParameter: o.base = b.index; break;
    case Buffer::kConstant: o.abs = const_symbol.at(root); break;
    case Buffer::kLiveOut: o.base = static_cast<int>(n_params) + b.index; break;
    case Buffer::kTemp:
      o.base = static_cast<int>(n_params + n_liveouts);
      o.off = b.offset;
      break;
  }
  return o;
}

// ---- regional synchronisation ------------------------------------------------------------------------------------
// Counterpart of RegionalSynchronizationAssignmentPass (regional_synchronization_assignment_pass.cc:35-72) on a part
// with 8 L2s: which nodes deal their units to the XCDs by ownership, and which values then never leave the XCD that
// wrote them.  Candidates come from the shapes (a k split over workgroups, the heads of an attention node, a GEMM in
// front of either); whether a value really stays inside an XCD is decided element by element: the writer's epilogue
// says where element (bidx, m, n) goes, the reader's operand map says which elements its partition fetches, and
// every element a partition reads must have been written by the same partition.
using NodeGenerator = std::function<NodeFunction(const Node&, const Partition&)>;

// owner[e] = partition that writes element e of the root's buffer, -1 = nobody; false when the map has run-time terms
bool owners_of(const WriteMap& w, const Partition& part, int64_t elements, std::vector<int8_t>& owner) {
  owner.assign(static_cast<size_t>(elements), -1);
  if (part.kind == Partition::kColumns && (w.batch != 1 || w.N % part.parts != 0)) return false;
  if (part.kind == Partition::kHeads && w.batch % part.parts != 0) return false;
  std::vector<int64_t> v(w.num_vars, 0);
  auto set = [&](int var, int64_t value) {
    if (var >= 0 && static_cast<size_t>(var) < v.size()) v[var] = value;
  };
  for (int64_t b = 0; b < w.batch; ++b)
    for (int64_t m = 0; m < w.M; ++m)
      for (int64_t n = 0; n < w.N; ++n) {
        set(w.vb, b);
        if (w.vm4 >= 0) set(w.vm4, m / 4), set(w.vr, m % 4), set(w.vnn, n);
        else if (w.vn4 >= 0) set(w.vm, m), set(w.vn4, n / 4), set(w.vr, n % 4);
        else set(w.vm, m), set(w.vnn, n);
        int64_t off = 0;
        if (!w.offset.evaluate(v, &off) || off < 0 || off >= elements) return false;
        owner[static_cast<size_t>(off)] = static_cast<int8_t>(part.kind == Partition::kColumns ? n / (w.N / part.parts) : b / (w.batch / part.parts));
      }
  return true;
}

// every element of `root` that partition x of node `r` reads has owner x
bool reads_own_partition(const graph::Program& prog, const Node& r, const Partition& part, const hlo::Instr* root, const std::vector<int8_t>& owner) {
  const int64_t elements = static_cast<int64_t>(owner.size());
  if (r.kind == NodeKind::kGemm && part.kind == Partition::kSplitK) {
    const graph::GemmDesc& g = r.gemm;
    const hlo::Instr* gi = r.members[0];
    if (g.batch != 1 || !g.a_k_contig || g.split_k != part.parts || g.K % part.parts != 0 || r.members.size() != 1 || !r.prologue.empty()) return false;
    if (prog.storage_root(gi->operands[0]) != root || prog.storage_root(gi->operands[1]) == root) return false;
    LinExpr off;
    if (g.M * g.K != elements || !operand_offset_expr(prog, gi->operands[0], elements, &off)) return false;
    const int64_t ks = g.K / part.parts;
    std::vector<int64_t> v(1);
    for (int64_t e = 0; e < elements; ++e) {
      v[0] = e;
      int64_t at = 0;
      if (!off.evaluate(v, &at) || at < 0 || at >= elements || owner[static_cast<size_t>(at)] != (e % g.K) / ks) return false;
    }
    return true;
  }
  if (r.kind == NodeKind::kAttention && part.kind == Partition::kHeads && r.gemm3_index == 0) {
    const hlo::Instr* g1 = r.members[0];
    const hlo::Instr* g2 = r.members[r.gemm2_index];
    const graph::GemmDesc &d1 = r.gemm, &d2 = r.gemm2;
    if (d1.batch % part.parts != 0 || d2.batch != d1.batch) return false;
    // the node reads batch element b of an operand from [b * per_head, (b + 1) * per_head) of its buffer
    int64_t per_head = 0;
    int uses = 0;
    if (prog.storage_root(g1->operands[0]) == root) ++uses, per_head = d1.M * d1.K, uses += (d1.a_packed || d1.a_batch_stride == per_head) ? 0 : 8;
    if (prog.storage_root(g1->operands[1]) == root) ++uses, per_head = d1.N * d1.K, uses += (d1.b_tiled || d1.b_batch_stride == per_head) ? 0 : 8;
    if (prog.storage_root(g2->operands[1]) == root) ++uses, per_head = d2.N * d2.K, uses += (d2.b_tiled || d2.b_batch_stride == per_head) ? 0 : 8;
    if (uses != 1 || per_head * d1.batch != elements) return false;
    for (size_t i = 0; i < r.members.size(); ++i) {
      if (i == 0 || i == r.gemm2_index) continue;
      for (auto* o : r.members[i]->operands)
        if (prog.storage_root(o) == root) return false;   // also read by the row program or the epilogue
    }
    const int64_t heads_per_part = d1.batch / part.parts;
    for (int64_t e = 0; e < elements; ++e)
      if (owner[static_cast<size_t>(e)] != (e / per_head) / heads_per_part) return false;
    return true;
  }
  return false;
}

void plan_regional_synchronization(const graph::Program& prog, const spec::GraphSpecification& spec, std::vector<Partition>& partition,
                                   std::vector<NodeFunction>& fns, const NodeGenerator& generate) {
  const size_t count = prog.nodes.size();
  std::map<const hlo::Instr*, std::vector<size_t>> readers;
  std::map<const hlo::Instr*, size_t> writer;
  for (size_t i = 0; i < count; ++i) {
    for (auto* r : prog.nodes[i].inputs) readers[r].push_back(i);
    for (auto* o : prog.nodes[i].outputs) writer[prog.storage_root(o)] = i;
  }
  auto direct_tile = [&](const Node& n) {
    auto it = spec.gemm_spec_list.find(n.name);
    return n.kind == NodeKind::kGemm && it != spec.gemm_spec_list.end() && it->second.stages < 2 && gemm_uses_mfma(n.gemm) && n.gemm.batch == 1 && !n.gemm.is_conv &&
           n.prologue.empty();
  };
  // candidates by shape
  for (size_t i = 0; i < count; ++i) {
    const Node& n = prog.nodes[i];
    if (n.kind == NodeKind::kAttention && n.gemm3_index == 0) {
      for (int p = 8; p >= 2; --p)
        if (n.gemm.batch % p == 0) {
          partition[i] = {Partition::kHeads, p};
          break;
        }
    } else if (direct_tile(n) && n.gemm.split_k >= 2 && n.gemm.split_k <= 8) {
      partition[i] = {Partition::kSplitK, n.gemm.split_k};
    }
  }
  for (size_t i = 0; i < count; ++i) {
    const Node& n = prog.nodes[i];
    if (!direct_tile(n) || n.gemm.split_k > 1 || n.outputs.empty()) continue;
    int parts = 0;
    bool ok = true;
    for (auto* o : n.outputs) {
      auto b = prog.buffers.find(prog.storage_root(o));
      auto rd = readers.find(prog.storage_root(o));
      ok = ok && b != prog.buffers.end() && b->second.kind == graph::Buffer::kTemp && rd != readers.end() && !rd->second.empty();
      if (!ok) break;
      for (size_t j : rd->second) {
        ok = ok && prog.nodes[j].stage == n.stage + 1 && partition[j].on() && (parts == 0 || parts == partition[j].parts);
        if (ok) parts = partition[j].parts;
      }
    }
    const spec::GemmSpec& g = spec.gemm_spec_list.at(n.name);
    if (ok && parts > 0 && n.gemm.N % parts == 0 && n.gemm.N % g.tb_n == 0 && (n.gemm.N / parts) % g.tb_n == 0) partition[i] = {Partition::kColumns, parts};
  }
  // Column slices on fewer than 8 XCDs must not cost the stage a second round of units: the GEMMs of a stage that
  // would go to the XCDs together (the projections in front of an attention node) stay round-robin when the units of
  // one XCD no longer fit its workgroups although the stage fitted the grid before.
  {
    const int64_t grid = spec.runtime.grid_dim.x;
    std::map<int, std::pair<int64_t, int64_t>> per_stage;   // stage -> (units of one XCD when partitioned, units dealt round-robin)
    auto tiles = [&](const Node& n) {
      const spec::GemmSpec& g = spec.gemm_spec_list.at(n.name);
      return ((n.gemm.M + g.tb_m - 1) / g.tb_m) * ((n.gemm.N + g.tb_n - 1) / g.tb_n);
    };
    for (size_t i = 0; i < count; ++i)
      if (partition[i].kind == Partition::kColumns) {
        auto& ps = per_stage[prog.nodes[i].stage];
        ps.first += tiles(prog.nodes[i]) / partition[i].parts;
        ps.second += tiles(prog.nodes[i]);
      }
    for (size_t i = 0; i < count; ++i)
      if (partition[i].kind == Partition::kColumns) {
        const auto& ps = per_stage.at(prog.nodes[i].stage);
        const int64_t rounds_regional = (ps.first + grid / 8 - 1) / (grid / 8), rounds_before = (ps.second + grid - 1) / grid;
        if (rounds_regional > rounds_before) partition[i] = Partition();
      }
  }
  std::vector<Partition> generated(count);
  std::set<const hlo::Instr*> roots;
  for (int round = 0; round < 4; ++round) {
    for (size_t i = 0; i < count; ++i)
      if (generated[i].kind != partition[i].kind || generated[i].parts != partition[i].parts) {
        fns[i] = generate(prog.nodes[i], partition[i]);
        generated[i] = partition[i];
      }
    // values whose every reader fetches what its own XCD wrote
    roots.clear();
    for (auto& kv : writer) {
      const hlo::Instr* root = kv.first;
      const size_t w = kv.second;
      auto b = prog.buffers.find(root);
      auto rd = readers.find(root);
      if (!(partition[w].kind == Partition::kColumns || partition[w].kind == Partition::kHeads) || b == prog.buffers.end() || b->second.kind != graph::Buffer::kTemp ||
          rd == readers.end() || rd->second.empty())
        continue;
      const WriteMap* wm = nullptr;
      int maps = 0;
      for (auto& m : fns[w].write_maps)
        if (m.root == root) wm = &m, ++maps;
      if (maps != 1) continue;
      bool ok = true;
      for (size_t j : rd->second) ok = ok && partition[j].on() && partition[j].parts == partition[w].parts && prog.nodes[j].stage > prog.nodes[w].stage;
      std::vector<int8_t> owner;
      ok = ok && owners_of(*wm, partition[w], root->shape.num_elements(), owner);
      for (size_t j : rd->second) ok = ok && reads_own_partition(prog, prog.nodes[j], partition[j], root, owner);
      if (ok) roots.insert(root);
    }
    // a partition that keeps nothing inside an XCD only costs parallelism: back to round-robin units
    bool changed = false;
    for (size_t i = 0; i < count; ++i) {
      if (!partition[i].on()) continue;
      const Node& n = prog.nodes[i];
      bool in = false, out = !n.outputs.empty();
      for (auto* r : n.inputs) in = in || roots.count(r) > 0;
      bool any_out = false;
      for (auto* o : n.outputs) {
        out = out && roots.count(prog.storage_root(o)) > 0;
        any_out = any_out || roots.count(prog.storage_root(o)) > 0;
      }
      bool keep = partition[i].kind == Partition::kColumns ? out : partition[i].kind == Partition::kSplitK ? in : (in || any_out);
      // column slices only pay when the barrier behind their stage becomes regional: every value of that stage that
      // a reader of this node takes must stay inside its XCD (the three projections in front of an attention node
      // go to the XCDs together or not at all)
      if (keep && partition[i].kind == Partition::kColumns)
        for (auto* o : n.outputs) {
          auto rd = readers.find(prog.storage_root(o));
          if (rd == readers.end()) continue;
          for (size_t j : rd->second)
            for (auto* r : prog.nodes[j].inputs) {
              auto w = writer.find(r);
              if (w != writer.end() && prog.nodes[w->second].stage == n.stage && !roots.count(r)) keep = false;
            }
        }
      if (!keep) {
        partition[i] = Partition();
        changed = true;
      }
    }
    if (!changed) break;
    if (round == 3) {   // did not settle: nothing regional
      roots.clear();
      for (auto& p : partition) p = Partition();
    }
  }
  for (size_t i = 0; i < count; ++i)
    if (generated[i].kind != partition[i].kind || generated[i].parts != partition[i].parts) {
      fns[i] = generate(prog.nodes[i], partition[i]);
      generated[i] = partition[i];
    }
  // the writers of those values take ordinary stores: generated once more with the annotation in place
  prog.regional_roots = roots;
  for (size_t i = 0; i < count; ++i) {
    bool writes = false;
    for (auto* o : prog.nodes[i].outputs) writes = writes || roots.count(prog.storage_root(o)) > 0;
    if (writes) fns[i] = generate(prog.nodes[i], partition[i]);
  }
}
}  // namespace

HipProgram generate_program(const graph::Program& prog, spec::GraphSpecification& spec, const std::string& kernel_name) {
  HipProgram hp;
  hp.kernel_name = kernel_name;
  LaunchShape ls;
  ls.block_size = spec.runtime.block_dim.x;
  hp.block = ls.block_size;
  hp.grid = spec.runtime.grid_dim.x;
  {
    // more workgroups than compute units: they share the CUs' four SIMDs, and the register budget with them
    const int cus = std::max(spec.device.sm_count, 1);
    const int per_cu = (hp.grid + cus - 1) / cus;
    ls.waves_per_simd = std::max(1, (per_cu * ls.waves() + 3) / 4);
  }
  MONONN_CHECK(hp.grid <= hp.max_grid, kSpecError) << "grid of " << hp.grid << " workgroups exceeds the barrier capacity of " << hp.max_grid;

  // every node named by the spec must exist (mononn_module.cc:83-85)
  std::set<std::string> names;
  for (auto& n : prog.nodes) names.insert(n.name);
  auto check_known = [&](const std::string& n, const char* where) {
    MONONN_CHECK(names.count(n), kSpecError) << where << " names node '" << n << "' which is not in the graph";
  };
  for (auto& kv : spec.cluster_elewise_spec) check_known(kv.first, "cluster_elewise_spec");
  for (auto& kv : spec.cluster_reduce_spec) check_known(kv.first, "cluster_reduce_spec");
  for (auto& kv : spec.gemm_spec_list) check_known(kv.first, "gemm_spec_list");
  for (auto& n : spec.codegen_allow_list) check_known(n, "codegen_allow_list");
  for (auto& n : spec.codegen_reject_list) check_known(n, "codegen_reject_list");
  std::set<std::string> allow(spec.codegen_allow_list.begin(), spec.codegen_allow_list.end());
  std::set<std::string> reject(spec.codegen_reject_list.begin(), spec.codegen_reject_list.end());

  // constants
  std::map<const hlo::Instr*, std::string> const_symbol;
  for (auto* c : prog.constants) {
    ConstantInfo ci;
    ci.name = c->name;
    ci.hlo_name = c->hlo_name;
    ci.symbol = "buffer_for_" + c->name;
    ci.bytes = c->shape.byte_size();
    ci.dtype = c->shape.dtype;
    ci.dims = c->shape.dims;
    auto tr = prog.constant_transform.find(c);
    if (tr != prog.constant_transform.end()) ci.transform = tr->second;
    ci.device_bytes = ci.bytes;
    if (ci.transform == graph::ConstantTransform::kPackMfmaB) ci.device_bytes = (ci.dims[1] + 15) / 16 * 16 * ci.dims[0] * hlo::dtype_bytes(ci.dtype);
    if (!c->literal_elided) ci.literal = c->literal;
    auto rs = prog.constant_row_scale.find(c);
    if (rs != prog.constant_row_scale.end()) ci.row_scale_by = rs->second->name;
    auto dc = prog.derived_constants.find(c);
    if (dc != prog.derived_constants.end()) {
      ci.sums_weight = dc->second.weight->name;
      ci.sums_vector = dc->second.vector->name;
      ci.role = "derived: column sums of " + dc->second.weight->hlo_name + " weighted by " + dc->second.vector->hlo_name;
    }
    auto md = c->attrs.find("metadata");
    if (md != c->attrs.end()) {
      size_t p = md->second.find("op_name=\"");
      if (p != std::string::npos) {
        size_t e = md->second.find('"', p + 9);
        if (e != std::string::npos) ci.role = md->second.substr(p + 9, e - p - 9);
      }
    }
    const_symbol[c] = ci.symbol;
    hp.constants.push_back(ci);
  }
  for (auto* p : prog.parameters) hp.param_bytes.push_back(p->shape.byte_size());
  for (auto* l : prog.live_outs) hp.liveout_bytes.push_back(l->shape.byte_size());
  hp.temp_bytes = prog.temp_bytes;

  // node functions, de-duplicated by text
  std::map<std::string, std::string> fn_by_text;
  std::vector<std::string> fn_defs;
  std::set<std::string> globals;
  struct Call {
    const Node* node;
    std::string fn;
    int fn_id = 0;
    std::vector<Operand> args;
    int64_t units;
    int parts = 0;   // regional synchronisation: XCDs that take part in the node (unit u belongs to XCD u % 8); 0 = units dealt round-robin
  };
  std::map<std::string, int> fn_ids;
  std::set<int> preload_fns;   // functions with a companion that requests constant operands ahead of the barrier wait
  std::map<int, std::vector<std::string>> fn_arg_types;   // fn id -> pointer types of its arguments
  std::map<int, std::vector<Call>> by_stage;
  int smem = 0;
  auto generate_node = [&](const Node& n, const Partition& part) {
    NodeFunction f;
    if (n.kind == NodeKind::kAttention) {
      // the fused node borrows a gemm_spec_list entry; of its fields wave_arrangement.k (key waves) and
      // threadblockshape.m (query rows per unit: 16 per wave along m, times the row blocks a wave takes in turn) are used
      auto it = spec.gemm_spec_list.find(n.name);
      if (it == spec.gemm_spec_list.end()) {
        spec::GemmSpec g;
        g.wave_k = default_attention_key_waves(n.gemm, ls);
        g.wave_m = ls.waves() / g.wave_k;
        g.wave_n = 1;
        g.tb_m = 16 * g.wave_m;
        g.tb_n = static_cast<int>(n.gemm.N);
        g.warp_m = 16;
        g.warp_n = static_cast<int>(n.gemm.N / g.wave_k);
        g.warp_k = static_cast<int>(n.gemm.K);
        auto bc = n.members[0]->attrs.find("backend_config");
        if (bc != n.members[0]->attrs.end()) g.backend_config = Json::parse(bc->second);
        it = spec.gemm_spec_list.emplace(n.name, g).first;
      }
      int row_blocks = 1;
      {
        const spec::GemmSpec& g = it->second;
        const int kw = g.wave_k > 0 ? g.wave_k : default_attention_key_waves(n.gemm, ls);
        const int rows_per_round = 16 * std::max(1, ls.waves() / std::max(1, kw));
        MONONN_CHECK(g.tb_m >= rows_per_round && g.tb_m % rows_per_round == 0, kSpecError)
            << "gemm_spec_list[" << n.name << "]: threadblockshape.m " << g.tb_m << " is not a multiple of the " << rows_per_round << " query rows the workgroup's waves take per round";
        row_blocks = g.tb_m / rows_per_round;
      }
      f = generate_attention(prog, n, ls, it->second.wave_k, spec.hip.operand_preload, row_blocks, part);
    } else if (n.kind == NodeKind::kGemm) {
      auto it = spec.gemm_spec_list.find(n.name);
      GemmTuning t;
      if (it == spec.gemm_spec_list.end()) {
        // a row program in front of the GEMM runs on register-held fragments: direct tile, unless it is a LayerNorm
        // folded away entirely (the LDS-staged tile computes its statistics and, if asked, stores its rows)
        const bool lds_ok = n.prologue.empty() || n.ln_fold.on();
        t = default_gemm_tuning(n.gemm, ls, spec.device.sm_count, lds_ok);
        if (!n.prologue.empty() && t.stages < 2) t = default_gemm_tuning(n.gemm, ls, spec.device.sm_count, false);
        spec::GemmSpec g;
        g.tb_m = t.bm;
        g.tb_n = t.bn;
        g.wave_m = t.wm;
        g.wave_n = t.wn;
        g.wave_k = t.wk;
        g.warp_m = t.bm / t.wm;
        g.warp_n = t.bn / t.wn;
        g.warp_k = static_cast<int>(n.gemm.K / t.wk);
        g.stages = t.stages;
        g.tb_k = t.bk;
        if (!gemm_uses_mfma(n.gemm)) g.operator_class = "SIMT";
        auto bc = n.members[0]->attrs.find("backend_config");
        if (bc != n.members[0]->attrs.end()) g.backend_config = Json::parse(bc->second);
        spec.gemm_spec_list[n.name] = g;
      } else {
        t.bm = it->second.tb_m;
        t.bn = it->second.tb_n;
        t.wm = it->second.wave_m;
        t.wn = it->second.wave_n;
        t.wk = it->second.wave_k;
        t.stages = it->second.stages;
        t.bk = it->second.tb_k;
      }
      t.split_k = n.gemm.split_k;
      t.part = part;
      t.preload_b = spec.hip.operand_preload;
      f = generate_gemm(prog, n, ls, t);
    } else {
      ClusterTuning t;
      if (n.has_reduce) {
        auto it = spec.cluster_reduce_spec.find(n.name);
        if (it == spec.cluster_reduce_spec.end()) {
          spec::ClusterReduceSpec r;
          r.name = n.name;
          // long rows get a whole workgroup, short ones a wave (tiers 2 / 1 of schedule_factory.cc:42-79)
          r.locality_tier = (n.row_program && n.row_len >= 512) ? 2 : 1;
          // many rows: a wave takes 8 of them at once, which keeps 8 rows' worth of bytes in flight per wave and
          // fills whole lines with every store (the generator falls back when the row length does not fit)
          if (n.row_program && n.rows >= 4096 && n.row_len >= 64 && n.row_len <= 1280 && n.row_len % 8 == 0) {
            r.locality_tier = 1;
            r.reduce_implementation = 1;
          }
          spec.cluster_reduce_spec[n.name] = r;
          it = spec.cluster_reduce_spec.find(n.name);
        }
        t.ilp_factor = it->second.ilp_factor;
        t.locality_tier = it->second.locality_tier;
        t.reduce_implementation = it->second.reduce_implementation;
      } else {
        auto it = spec.cluster_elewise_spec.find(n.name);
        if (it == spec.cluster_elewise_spec.end()) {
          spec::ClusterElewiseSpec e;
          e.name = n.name;
          spec.cluster_elewise_spec[n.name] = e;
          it = spec.cluster_elewise_spec.find(n.name);
        }
        t.ilp_factor = it->second.ilp_factor;
      }
      f = generate_cluster(prog, n, ls, t);
    }
    return f;
  };
  // Every node once with the units dealt round-robin (this also fills the specification with the defaults of nodes
  // it does not mention); with regional synchronisation the plan then names the nodes whose units go to the XCDs by
  // ownership and the values that stay inside an XCD, and those nodes are generated again.
  prog.regional_roots.clear();
  std::vector<NodeFunction> node_fns;
  for (auto& n : prog.nodes) node_fns.push_back(generate_node(n, Partition()));
  std::vector<Partition> partition(prog.nodes.size());
  const bool regional = spec.hip.regional_synchronization && spec.hip.barrier == "flags_coherent" && hp.grid % 8 == 0 && hp.grid == spec.device.sm_count &&
                        ls.waves_per_simd == 1 && !spec.hip.cooperative_launch;
  if (regional) plan_regional_synchronization(prog, spec, partition, node_fns, generate_node);
  for (size_t ni = 0; ni < prog.nodes.size(); ++ni) {
    const Node& n = prog.nodes[ni];
    NodeFunction& f = node_fns[ni];
    bool emit = (allow.empty() || allow.count(n.name)) && !reject.count(n.name);
    std::string fn;
    auto known = fn_by_text.find(f.text);
    if (known != fn_by_text.end()) {
      fn = known->second;
    } else if (emit) {
      fn = "node_fn_" + std::to_string(fn_by_text.size());
      fn_ids[fn] = static_cast<int>(fn_by_text.size());
      fn_by_text[f.text] = fn;
      std::string def = f.text;
      size_t pos;
      while ((pos = def.find("@NAME@")) != std::string::npos) def.replace(pos, 6, fn);
      fn_defs.push_back(def);
      if (!f.preload_text.empty()) {
        std::string pdef = f.preload_text;
        while ((pos = pdef.find("@NAME@")) != std::string::npos) pdef.replace(pos, 6, fn);
        fn_defs.push_back(pdef);
        preload_fns.insert(fn_ids[fn]);
      }
      for (auto& g : f.globals) globals.insert(g);
    }
    NodeReport rep;
    rep.name = n.name;
    rep.kind = n.kind == NodeKind::kGemm ? "gemm" : n.kind == NodeKind::kAttention ? "attention" : (n.row_program ? "cluster_reduce" : "cluster_elewise");
    rep.function = fn;
    rep.stage = n.stage;
    rep.units = f.num_units;
    if (partition[ni].on())
      rep.partition = std::string(partition[ni].kind == Partition::kColumns ? "columns/" : partition[ni].kind == Partition::kSplitK ? "split_k/" : "heads/") + std::to_string(partition[ni].parts);
    hp.nodes.push_back(rep);
    if (!emit) continue;
    smem = std::max(smem, f.smem_bytes);
    Call c;
    c.node = &n;
    c.parts = partition[ni].on() ? partition[ni].parts : 0;
    c.fn = fn;
    c.units = f.num_units;
    c.fn_id = fn_ids.at(fn);
    for (auto& e : f.pointers) c.args.push_back(make_operand(prog, e.root, e.is_output, e.dtype, const_symbol, hp.param_bytes.size(), hp.liveout_bytes.size()));
    if (!fn_arg_types.count(c.fn_id))
      for (auto& a : c.args) fn_arg_types[c.fn_id].push_back(a.ctype);
    by_stage[n.stage].push_back(c);
  }
  hp.smem = smem;
  spec.runtime.smem_size = smem;
  MONONN_CHECK(smem <= spec.device.max_configurable_smem_size, kResourceExhausted)
      << "kernel needs " << smem << " bytes of LDS, device offers " << spec.device.max_configurable_smem_size;

  // Barrier tiers.  A value that does not stay inside an XCD needs a barrier of the memory-side tier somewhere between
  // its writer's stage and each reader's stage; every other barrier only has to order the workgroups of one XCD.
  // Fewest memory-side barriers: readers by stage, a barrier right in front of a reader that has none yet in its range.
  std::vector<bool> regional_before(by_stage.size(), false);
  if (regional && !prog.regional_roots.empty() && allow.empty() && reject.empty()) {
    std::map<int, int> index_of_stage;
    for (auto& st : by_stage) index_of_stage.emplace(st.first, static_cast<int>(index_of_stage.size()));
    std::vector<std::pair<int, int>> need;   // (reader's stage, first stage after the writer's): emitted stage indices
    for (auto& st : by_stage)
      for (auto& c : st.second)
        for (auto* in : c.node->inputs) {
          auto pr = prog.producer.find(in);
          if (pr == prog.producer.end() || prog.regional_roots.count(in)) continue;
          const int ws = index_of_stage.at(prog.nodes[pr->second].stage), rs = index_of_stage.at(c.node->stage);
          MONONN_CHECK(ws < rs, kInternal) << c.node->name << " reads a value of its own or a later stage";
          need.emplace_back(rs, ws + 1);
        }
    std::sort(need.begin(), need.end());
    std::vector<bool> memory_side(by_stage.size(), false);
    int last = -1;
    for (auto& iv : need)
      if (last < iv.second) {
        last = iv.first;
        memory_side[last] = true;
      }
    for (size_t b = 1; b < by_stage.size(); ++b) regional_before[b] = !memory_side[b];
  }
  bool any_regional = false;
  for (bool r : regional_before) any_regional = any_regional || r;
  // The translation unit is kept in three parts so that the tuner can put many candidate kernels of
  // one node class into a single hipRTC compilation: preamble (defines + include), global
  // declarations (shared by all candidates), body (node functions + kernel).
  std::ostringstream pre, glob, src;
  pre << "// generated by mononn-hip for " << spec.device.cuda_arch << "\n";
  pre << "#define MONONN_BLOCK_SIZE " << hp.block << "\n";
  if (ls.waves_per_simd > 1) pre << "#define MONONN_WAVES_PER_SIMD " << ls.waves_per_simd << "\n";
  if (spec.hip.barrier == "flags_allfence") pre << "#define MONONN_BARRIER_FENCE 1\n";
  else if (spec.hip.barrier == "flags_coherent") pre << "#define MONONN_BARRIER_FENCE 2\n#define MONONN_COHERENT_STORES 1\n";
  else MONONN_CHECK(spec.hip.barrier == "flags", kSpecError) << "unknown barrier flavour '" << spec.hip.barrier << "'";
  {
    // see mononn_dev::thread_id(): on in kernels that hold a stage with a large register tile (an LDS-staged GEMM)
    bool opaque = spec.hip.opaque_thread_id;
    for (auto& kv : spec.gemm_spec_list) opaque = opaque || kv.second.stages >= 2;
    pre << "#define MONONN_OPAQUE_THREAD_ID " << (opaque ? 1 : 0) << "\n";
  }
  if (any_regional) pre << "#define MONONN_REGIONAL_SYNC 1\n";
  pre << "#define MONONN_BARRIER_BUDGET_TICKS " << static_cast<long long>(spec.hip.barrier_timeout_ms) * 100000 << "ull   // wall clock: 100 MHz\n";
  pre << "#include \"headers.h\"\n\n";
  for (auto& c : hp.constants) {
    std::ostringstream d;
    d << "__device__ __attribute__((aligned(256))) unsigned char " << c.symbol << "[" << std::max<int64_t>(c.device_bytes, 1) << "];";
    hp.global_decls.push_back(d.str());
  }
  {
    std::ostringstream d;
    d << "__device__ unsigned mononn_barrier_flags[" << hp.max_grid << " * mononn_dev::kFlagStride];";
    hp.global_decls.push_back(d.str());
    if (any_regional) {
      std::ostringstream r;
      r << "__device__ unsigned mononn_regional_flags[" << hp.max_grid << " * mononn_dev::kFlagStride];   // barrier tier over the workgroups of one XCD";
      hp.global_decls.push_back(r.str());
    }
    hp.global_decls.push_back("__device__ unsigned mononn_barrier_error[4];   // [0]: 0, or the ordinal (from 1) of the first barrier a wait gave up on");
  }
  hp.profiled = spec.hip.profile_stages;
  hp.cooperative = spec.hip.cooperative_launch;
  hp.num_stages = static_cast<int>(by_stage.size());
  if (hp.profiled) {
    // sized for the deepest kernel the barrier supports so that candidates of one class can share it
    std::ostringstream d;
    d << "__device__ unsigned long long mononn_stage_clock[" << std::max<size_t>(by_stage.size(), 1) * hp.grid * 2 << "];";
    hp.global_decls.push_back(d.str());
  }
  for (auto& g : globals) hp.global_decls.push_back(g);
  for (auto& g : hp.global_decls) glob << g << "\n";
  glob << "\n";
  for (auto& d : fn_defs) {
    // node functions read the thread index through mononn_dev::thread_id() (see there: keeps per-stage address
    // arithmetic inside its stage)
    std::string text = d;
    size_t pos = 0;
    while ((pos = text.find("threadIdx.x", pos)) != std::string::npos) {
      text.replace(pos, 11, "mononn_dev::thread_id()");
      pos += 23;
    }
    src << text << "\n";
  }

  // The kernel is a small interpreter over the list of calls (node function + buffers), stage by stage.
  // Every distinct node function is inlined exactly once, in one case of the dispatch switch: calling
  // the functions would cost a save / restore of the callee-saved VGPRs through scratch memory on
  // every stage, and inlining every use would multiply the code of a layer by the number of layers.
  // The parameters of a call are set up by a second switch from immediates (kernel argument + offset,
  // or the address of a module global), so no table has to be fetched from memory on the critical path.
  size_t max_ptrs = 1;
  for (auto& st : by_stage)
    for (auto& c : st.second) max_ptrs = std::max(max_ptrs, c.args.size());
  struct Flat {
    const Call* call;
    int first_unit, stage_total;
    bool new_stage;
    int rot;   // unit u of the stage runs on workgroup (u + rot) % grid
    bool regional;   // the barrier in front of the stage is one of the regional tier
  };
  std::vector<Flat> flat;
  // A workgroup that had a unit in the previous stage reaches the barrier later than an idle one and has asked for
  // its constant operands later: when the units of two consecutive stages fit side by side, the second stage is
  // placed on the workgroups the first one left idle.  Offsets are multiples of 8 so that a unit keeps its XCD.
  int64_t prev_total = 0, prev_rot = 0;
  bool any_rot = false;
  for (auto& st : by_stage) {
    // a node whose units belong to XCDs (unit % 8) starts at a multiple of 8 in the stage's unit range
    int64_t total = 0;
    for (auto& c : st.second) total = (c.parts ? (total + 7) / 8 * 8 : total) + c.units;
    MONONN_CHECK(total < (int64_t(1) << 31), kResourceExhausted) << "stage has too many work units";
    int64_t rot = 0;
    if (spec.hip.stage_rotation && hp.grid % 8 == 0 && prev_total > 0 && total + (prev_total + 7) / 8 * 8 <= hp.grid)
      rot = (prev_rot + (prev_total + 7) / 8 * 8) % hp.grid;
    any_rot = any_rot || rot != 0;
    hp.stage_nodes.emplace_back();
    int64_t first = 0;
    bool ns = true;
    for (auto& c : st.second) {
      hp.stage_nodes.back().push_back(c.node->name);
      if (c.parts) first = (first + 7) / 8 * 8;
      flat.push_back({&c, static_cast<int>(first), static_cast<int>(total), ns, static_cast<int>(rot), regional_before[hp.stage_nodes.size() - 1]});
      ns = false;
      first += c.units;
    }
    prev_total = total;
    prev_rot = rot;
  }
  hp.num_barriers = by_stage.empty() ? 0 : static_cast<int>(by_stage.size()) - 1;
  hp.regional_before = regional_before;
  for (bool r : regional_before) hp.num_regional_barriers += r ? 1 : 0;
  auto base_expr = [&](const Operand& o) -> std::string {
    if (o.base < 0) return "(char*)" + o.abs;
    std::string b;
    size_t np = hp.param_bytes.size(), nl = hp.liveout_bytes.size();
    if (static_cast<size_t>(o.base) < np) b = "(char*)arg" + std::to_string(o.base);
    else if (static_cast<size_t>(o.base) < np + nl) b = "(char*)liveout_buffer_" + std::to_string(o.base - np);
    else b = "(char*)temp_buffer";
    return o.off ? b + " + " + std::to_string(o.off) : b;
  };

  // the second bound (waves per SIMD) caps the registers of a wave so that the whole grid stays resident
  src << "extern \"C\" __launch_bounds__(" << ls.block_size;
  if (ls.waves_per_simd > 1) src << ", " << ls.waves_per_simd;
  src << ") __global__ void " << kernel_name << "(";
  for (size_t i = 0; i < hp.param_bytes.size(); ++i) src << "void* arg" << i << ", ";
  for (size_t i = 0; i < hp.liveout_bytes.size(); ++i) src << "void* liveout_buffer_" << i << ", ";
  src << "void* temp_buffer) {\n";
  src << "  extern __shared__ __attribute__((aligned(16))) char smem[];\n";
  src << "  mononn_dev::GridBarrier barrier;\n  barrier.init(mononn_barrier_flags, mononn_barrier_error);\n";
  if (any_regional) src << "  barrier.init_regional(mononn_regional_flags);\n";
  bool any_parts = false;
  for (auto& f : flat) any_parts = any_parts || f.call->parts > 0;
  src << "  int stage = -1;\n";
  const bool lazy = !preload_fns.empty();
  if (lazy) {
    // The wait half of a barrier is put off until the workgroup's first unit of the new stage, behind the
    // requests for that unit's constant operands; a workgroup without a unit in a stage does not wait for it.
    src << "  bool pending = false;   // announced the end of the previous stage, not yet waited for the others\n";
    // with two tiers: the latest announcement of each tier that the workgroup has not waited for (a barrier over all
    // workgroups also covers every regional one before it)
    if (any_regional) src << "  bool pending_memory = false, pending_regional = false;\n";
  }
  src << "  for (int c = 0; c < " << flat.size() << "; ++c) {\n";
  src << "    int fn = 0, units = 0, first = 0, total = 0" << (any_rot ? ", rot = 0" : "") << ";\n    bool new_stage = false;\n";
  if (any_regional) src << "    bool regional = false;   // the barrier in front of the stage orders the workgroups of one XCD only\n";
  if (any_parts) src << "    int parts = 0;   // > 0: unit u belongs to XCD u % 8, and only this many XCDs take part\n";
  src << "    char*";
  for (size_t i = 0; i < max_ptrs; ++i) src << (i ? ", *" : " ") << "p" << i << " = nullptr";
  src << ";\n";
  src << "    switch (c) {\n";
  for (size_t i = 0; i < flat.size(); ++i) {
    const Flat& f = flat[i];
    src << "      case " << i << ": fn = " << f.call->fn_id << "; units = " << f.call->units << "; first = " << f.first_unit << "; total = "
        << f.stage_total << "; new_stage = " << (f.new_stage ? "true" : "false") << ";";
    if (f.rot) src << " rot = " << f.rot << ";";
    if (f.regional && f.new_stage) src << " regional = true;";
    if (f.call->parts) src << " parts = " << f.call->parts << ";";
    for (size_t a = 0; a < f.call->args.size(); ++a) src << " p" << a << " = " << base_expr(f.call->args[a]) << ";";
    src << " break;   // " << f.call->node->name.substr(0, 50) << "\n";
  }
  src << "      default: break;\n    }\n";
  // stage clocks: [stage][workgroup][0] = first unit of the stage may start, [1] = the workgroup's part is done;
  // a workgroup that has no unit in a stage leaves both at zero
  const std::string clk = "mononn_stage_clock[(stage * " + std::to_string(hp.grid) + " + blockIdx.x) * 2";
  src << "    if (new_stage) {\n";
  if (!lazy) {
    if (hp.profiled) {
      src << "      if (stage >= 0) {\n        __syncthreads();\n";
      src << "        if (threadIdx.x == 0) " << clk << " + 1] = wall_clock64();\n      }\n";
    }
    if (any_regional) src << "      if (stage >= 0) {\n        if (regional) { barrier.arrive_regional(); barrier.wait_regional(); } else barrier.sync();\n      }\n      ++stage;\n";
    else src << "      if (stage >= 0) barrier.sync();\n      ++stage;\n";
    if (hp.profiled) src << "      if (threadIdx.x == 0) " << clk << "] = wall_clock64();\n";
  } else {
    src << "      if (stage >= 0) {\n";
    if (hp.profiled) {
      src << "        __syncthreads();\n";
      src << "        if (threadIdx.x == 0) {\n";
      src << "          if (pending) " << clk << "] = 0;\n";
      src << "          " << clk << " + 1] = pending ? 0 : wall_clock64();\n        }\n";
    }
    if (any_regional) {
      src << "        if (regional) { barrier.arrive_regional(); pending_regional = true; }\n";
      src << "        else { barrier.arrive(); pending_memory = true; pending_regional = false; }\n";
      src << "        pending = true;\n      }\n      ++stage;\n";
    } else {
      src << "        barrier.arrive();\n        pending = true;\n      }\n      ++stage;\n";
    }
    if (hp.profiled) src << "      if (stage == 0 && threadIdx.x == 0) " << clk << "] = wall_clock64();\n";
  }
  src << "    }\n";
  if (any_rot) src << "    for (int u = blockIdx.x >= rot ? blockIdx.x - rot : blockIdx.x + gridDim.x - rot; u < total; u += gridDim.x) {\n";
  else src << "    for (int u = blockIdx.x; u < total; u += gridDim.x) {\n";
  src << "      const int unit = u - first;\n";
  src << "      if (unit < 0 || unit >= units) continue;\n";
  if (any_parts) src << "      if (parts > 0 && (unit & 7) >= parts) continue;   // an XCD without a share of this node\n";
  // One dispatch switch; in the lazy form every case first requests what it can, then waits if a barrier is pending
  // (the wait is spelled out per case so that the requested registers flow straight into the function that uses
  // them instead of meeting at a join of all cases).
  std::string wait_text;
  if (lazy) {
    if (any_regional) wait_text = "if (pending) { if (pending_memory) barrier.wait(); if (pending_regional) barrier.wait_regional(); pending = pending_memory = pending_regional = false;";
    else wait_text = "if (pending) { barrier.wait(); pending = false;";
    if (hp.profiled) wait_text += " if (threadIdx.x == 0) " + clk + "] = wall_clock64();";
    wait_text += " } ";
  }
  src << "      switch (fn) {\n";
  for (auto& kv : fn_arg_types) {
    std::ostringstream args;
    for (size_t i = 0; i < kv.second.size(); ++i) args << ", (" << kv.second[i] << ")p" << i;
    src << "        case " << kv.first << ": { ";
    const bool pre = preload_fns.count(kv.first) > 0;
    if (pre) src << "node_fn_" << kv.first << "_preb pre_b; node_fn_" << kv.first << "_pre(unit" << args.str() << ", pre_b); ";
    src << wait_text << "node_fn_" << kv.first << "(unit" << args.str() << ", smem" << (pre ? ", pre_b" : "") << "); } break;\n";
  }
  src << "        default: break;\n      }\n    }\n  }\n";
  if (hp.profiled) {
    src << "  __syncthreads();\n";
    if (lazy) {
      src << "  if (threadIdx.x == 0 && stage >= 0) {\n    if (pending) mononn_stage_clock[(stage * " << hp.grid << " + blockIdx.x) * 2] = 0;\n";
      src << "    mononn_stage_clock[(stage * " << hp.grid << " + blockIdx.x) * 2 + 1] = pending ? 0 : wall_clock64();\n  }\n";
    } else {
      src << "  if (threadIdx.x == 0 && stage >= 0) mononn_stage_clock[(stage * " << hp.grid << " + blockIdx.x) * 2 + 1] = wall_clock64();\n";
    }
  }
  src << "}\n";
  hp.preamble = pre.str();
  hp.body = src.str();
  hp.files["headers.h"] = device::kPreludeText;
  hp.files["main.hip"] = hp.preamble + glob.str() + hp.body;
  hp.files["host_main.cpp"] = generate_host_driver(hp);
  return hp;
}

}  // namespace codegen
}  // namespace mononn
