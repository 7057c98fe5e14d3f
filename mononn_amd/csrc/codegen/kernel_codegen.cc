#include "codegen/kernel_codegen.h"

#include "codegen/host_codegen.h"

#include <algorithm>
#include <cstdlib>
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
  };
  std::map<std::string, int> fn_ids;
  std::set<int> preload_fns;   // functions with a companion that requests constant operands ahead of the barrier wait
  std::map<int, std::vector<std::string>> fn_arg_types;   // fn id -> pointer types of its arguments
  std::map<int, std::vector<Call>> by_stage;
  int smem = 0;
  for (auto& n : prog.nodes) {
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
      f = generate_attention(prog, n, ls, it->second.wave_k, spec.hip.operand_preload, row_blocks);
    } else if (n.kind == NodeKind::kGemm) {
      auto it = spec.gemm_spec_list.find(n.name);
      GemmTuning t;
      if (it == spec.gemm_spec_list.end()) {
        t = default_gemm_tuning(n.gemm, ls, spec.device.sm_count);
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
    hp.nodes.push_back(rep);
    if (!emit) continue;
    smem = std::max(smem, f.smem_bytes);
    Call c;
    c.node = &n;
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
  };
  std::vector<Flat> flat;
  // A workgroup that had a unit in the previous stage reaches the barrier later than an idle one and has asked for
  // its constant operands later: when the units of two consecutive stages fit side by side, the second stage is
  // placed on the workgroups the first one left idle.  Offsets are multiples of 8 so that a unit keeps its XCD.
  int64_t prev_total = 0, prev_rot = 0;
  bool any_rot = false;
  for (auto& st : by_stage) {
    int64_t total = 0;
    for (auto& c : st.second) total += c.units;
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
      flat.push_back({&c, static_cast<int>(first), static_cast<int>(total), ns, static_cast<int>(rot)});
      ns = false;
      first += c.units;
    }
    prev_total = total;
    prev_rot = rot;
  }
  hp.num_barriers = by_stage.empty() ? 0 : static_cast<int>(by_stage.size()) - 1;
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
  src << "  int stage = -1;\n";
  const bool lazy = !preload_fns.empty();
  if (lazy) {
    // The wait half of a barrier is put off until the workgroup's first unit of the new stage, behind the
    // requests for that unit's constant operands; a workgroup without a unit in a stage does not wait for it.
    src << "  bool pending = false;   // announced the end of the previous stage, not yet waited for the others\n";
  }
  src << "  for (int c = 0; c < " << flat.size() << "; ++c) {\n";
  src << "    int fn = 0, units = 0, first = 0, total = 0" << (any_rot ? ", rot = 0" : "") << ";\n    bool new_stage = false;\n";
  src << "    char*";
  for (size_t i = 0; i < max_ptrs; ++i) src << (i ? ", *" : " ") << "p" << i << " = nullptr";
  src << ";\n";
  src << "    switch (c) {\n";
  for (size_t i = 0; i < flat.size(); ++i) {
    const Flat& f = flat[i];
    src << "      case " << i << ": fn = " << f.call->fn_id << "; units = " << f.call->units << "; first = " << f.first_unit << "; total = "
        << f.stage_total << "; new_stage = " << (f.new_stage ? "true" : "false") << ";";
    if (f.rot) src << " rot = " << f.rot << ";";
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
    src << "      if (stage >= 0) barrier.sync();\n      ++stage;\n";
    if (hp.profiled) src << "      if (threadIdx.x == 0) " << clk << "] = wall_clock64();\n";
  } else {
    src << "      if (stage >= 0) {\n";
    if (hp.profiled) {
      src << "        __syncthreads();\n";
      src << "        if (threadIdx.x == 0) {\n";
      src << "          if (pending) " << clk << "] = 0;\n";
      src << "          " << clk << " + 1] = pending ? 0 : wall_clock64();\n        }\n";
    }
    src << "        barrier.arrive();\n        pending = true;\n      }\n      ++stage;\n";
    if (hp.profiled) src << "      if (stage == 0 && threadIdx.x == 0) " << clk << "] = wall_clock64();\n";
  }
  src << "    }\n";
  if (any_rot) src << "    for (int u = blockIdx.x >= rot ? blockIdx.x - rot : blockIdx.x + gridDim.x - rot; u < total; u += gridDim.x) {\n";
  else src << "    for (int u = blockIdx.x; u < total; u += gridDim.x) {\n";
  src << "      const int unit = u - first;\n";
  src << "      if (unit < 0 || unit >= units) continue;\n";
  // One dispatch switch; in the lazy form every case first requests what it can, then waits if a barrier is pending
  // (the wait is spelled out per case so that the requested registers flow straight into the function that uses
  // them instead of meeting at a join of all cases).
  std::string wait_text;
  if (lazy) {
    wait_text = "if (pending) { barrier.wait(); pending = false;";
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
