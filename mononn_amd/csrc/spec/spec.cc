#include "spec/spec.h"

#include <set>

#include "common/status.h"

namespace mononn {
namespace spec {

namespace {
Json dim3_json(const Dim3& d) {
  Json j = Json::object();
  j["x"] = d.x;
  j["y"] = d.y;
  j["z"] = d.z;
  return j;
}
Json shape_json(int m, int n, int k) {
  Json j = Json::object();
  j["m"] = m;
  j["n"] = n;
  j["k"] = k;
  return j;
}
Json strings_json(const std::vector<std::string>& v) {
  Json a = Json::array();
  for (auto& s : v) a.push_back(Json(s));
  return a;
}
void check_keys(const Json& j, const std::set<std::string>& allowed, const char* where) {
  MONONN_CHECK(j.is_object(), kSpecError) << where << " must be an object";
  for (auto& kv : j.members())
    MONONN_CHECK(allowed.count(kv.first), kSpecError) << "unknown field '" << kv.first << "' in " << where;
}
int geti(const Json& j, const char* k, int dflt) { return j.contains(k) ? static_cast<int>(j.at(k).as_int()) : dflt; }
std::string gets(const Json& j, const char* k, const std::string& dflt) { return j.contains(k) ? j.at(k).as_string() : dflt; }
bool getb(const Json& j, const char* k, bool dflt) { return j.contains(k) ? j.at(k).as_bool() : dflt; }
Dim3 dim3_from(const Json& j, const char* where) {
  check_keys(j, {"x", "y", "z"}, where);
  Dim3 d;
  d.x = geti(j, "x", 1);
  d.y = geti(j, "y", 1);
  d.z = geti(j, "z", 1);
  return d;
}
std::vector<std::string> strings_from(const Json& j, const char* k) {
  std::vector<std::string> v;
  if (j.contains(k))
    for (auto& s : j.at(k).items()) v.push_back(s.as_string());
  return v;
}
}  // namespace

std::string GraphSpecification::context_string() const {
  const Dim3 &g = runtime.grid_dim, &b = runtime.block_dim;
  return std::to_string(g.x) + "_" + std::to_string(g.y) + "_" + std::to_string(g.z) + "__" + std::to_string(b.x) + "_" +
         std::to_string(b.y) + "_" + std::to_string(b.z);
}

Json GraphSpecification::to_json() const {
  Json j = Json::object();
  Json ctx = Json::object();
  Json rt = Json::object();
  rt["grid_dim"] = dim3_json(runtime.grid_dim);
  rt["block_dim"] = dim3_json(runtime.block_dim);
  rt["smem_size"] = runtime.smem_size;
  rt["stream"] = runtime.stream;
  ctx["cuda_runtime_context"] = rt;
  Json dv = Json::object();
  dv["device_count"] = device.device_count;
  dv["sm_count"] = device.sm_count;
  dv["static_smem_size"] = device.static_smem_size;
  dv["max_configurable_smem_size"] = device.max_configurable_smem_size;
  dv["cuda_arch"] = device.cuda_arch;
  dv["register_per_block"] = device.register_per_block;
  dv["warp_size"] = device.warp_size;
  dv["reserved_smem_per_block"] = device.reserved_smem_per_block;
  ctx["cuda_device_context"] = dv;
  j["cuda_context"] = ctx;
  j["hlo_module_proto_file"] = hlo_module_proto_file;
  j["feeds"] = strings_json(feeds);
  j["input_data_files"] = strings_json(input_data_files);
  j["fetches"] = strings_json(fetches);
  Json ce = Json::object();
  for (auto& kv : cluster_elewise_spec) {
    Json e = Json::object();
    e["name"] = kv.second.name;
    e["ilp_factor"] = kv.second.ilp_factor;
    ce[kv.first] = e;
  }
  j["cluster_elewise_spec"] = ce;
  Json cr = Json::object();
  for (auto& kv : cluster_reduce_spec) {
    Json e = Json::object();
    e["name"] = kv.second.name;
    e["ilp_factor"] = kv.second.ilp_factor;
    e["locality_tier"] = kv.second.locality_tier;
    e["reduce_implementation"] = kv.second.reduce_implementation;
    cr[kv.first] = e;
  }
  j["cluster_reduce_spec"] = cr;
  Json gl = Json::object();
  for (auto& kv : gemm_spec_list) {
    const GemmSpec& g = kv.second;
    Json e = Json::object();
    Json cc = Json::object();
    cc["threadblockshape"] = shape_json(g.tb_m, g.tb_n, g.tb_k);
    cc["warpshape"] = shape_json(g.warp_m, g.warp_n, g.warp_k);
    cc["instructionshape"] = shape_json(g.inst_m, g.inst_n, g.inst_k);
    Json oc = Json::object();
    oc["name"] = g.operator_class;
    cc["operatorclass"] = oc;
    Json at = Json::object();
    at["name"] = g.arch_tag;
    cc["archtag"] = at;
    cc["stages"] = g.stages;
    cc["wave_arrangement"] = shape_json(g.wave_m, g.wave_n, g.wave_k);
    cc["split_k"] = g.split_k;
    e["cutlass_config"] = cc;
    e["gemm_backend_config"] = g.backend_config.is_null() ? Json::object() : g.backend_config;
    gl[kv.first] = e;
  }
  j["gemm_spec_list"] = gl;
  Json cl = Json::object();
  for (auto& kv : conv_spec_list) cl[kv.first] = kv.second;
  j["conv_spec_list"] = cl;
  j["codegen_allow_list"] = strings_json(codegen_allow_list);
  j["codegen_reject_list"] = strings_json(codegen_reject_list);
  Json h = Json::object();
  h["merge_dependent"] = hip.merge_dependent;
  h["gemm_epilogue_fusion"] = hip.gemm_epilogue_fusion;
  h["transpose_constant_b"] = hip.transpose_constant_b;
  h["assign_operand_layouts"] = hip.assign_operand_layouts;
  h["fuse_attention"] = hip.fuse_attention;
  h["gemm_prologue_fusion"] = hip.gemm_prologue_fusion;
  h["layer_norm_folding"] = hip.layer_norm_folding;
  h["barrier"] = hip.barrier;
  h["profile_stages"] = hip.profile_stages;
  h["cooperative_launch"] = hip.cooperative_launch;
  h["barrier_timeout_ms"] = hip.barrier_timeout_ms;
  h["opaque_thread_id"] = hip.opaque_thread_id;
  h["operand_preload"] = hip.operand_preload;
  h["pack_left_operands"] = hip.pack_left_operands;
  h["attention_out_proj_fusion"] = hip.attention_out_proj_fusion;
  h["stage_rotation"] = hip.stage_rotation;
  h["regional_synchronization"] = hip.regional_synchronization;
  j["mononn_hip"] = h;
  return j;
}

GraphSpecification GraphSpecification::from_json(const Json& j) {
  GraphSpecification s;
  check_keys(j,
             {"cuda_context", "hlo_module_proto_file", "feeds", "input_data_files", "fetches", "cluster_elewise_spec", "cluster_reduce_spec",
              "gemm_spec_list", "conv_spec_list", "codegen_allow_list", "codegen_reject_list", "mononn_hip"},
             "GraphSpecification");
  const Json& ctx = j.at("cuda_context");
  check_keys(ctx, {"cuda_runtime_context", "cuda_device_context"}, "cuda_context");
  const Json& rt = ctx.at("cuda_runtime_context");
  check_keys(rt, {"grid_dim", "block_dim", "smem_size", "stream"}, "cuda_runtime_context");
  s.runtime.grid_dim = dim3_from(rt.at("grid_dim"), "grid_dim");
  s.runtime.block_dim = dim3_from(rt.at("block_dim"), "block_dim");
  s.runtime.smem_size = geti(rt, "smem_size", 0);
  s.runtime.stream = gets(rt, "stream", "0");
  if (ctx.contains("cuda_device_context")) {
    const Json& dv = ctx.at("cuda_device_context");
    check_keys(dv, {"device_count", "sm_count", "static_smem_size", "max_configurable_smem_size", "cuda_arch", "register_per_block", "warp_size", "reserved_smem_per_block"},
               "cuda_device_context");
    s.device.device_count = geti(dv, "device_count", 1);
    s.device.sm_count = geti(dv, "sm_count", 256);
    s.device.static_smem_size = geti(dv, "static_smem_size", 65536);
    s.device.max_configurable_smem_size = geti(dv, "max_configurable_smem_size", 163840);
    s.device.cuda_arch = gets(dv, "cuda_arch", "gfx950");
    s.device.register_per_block = geti(dv, "register_per_block", 131072);
    s.device.warp_size = geti(dv, "warp_size", 64);
    s.device.reserved_smem_per_block = geti(dv, "reserved_smem_per_block", 0);
  }
  s.hlo_module_proto_file = gets(j, "hlo_module_proto_file", "");
  s.feeds = strings_from(j, "feeds");
  s.input_data_files = strings_from(j, "input_data_files");
  s.fetches = strings_from(j, "fetches");
  if (j.contains("cluster_elewise_spec"))
    for (auto& kv : j.at("cluster_elewise_spec").members()) {
      check_keys(kv.second, {"name", "ilp_factor"}, "cluster_elewise_spec entry");
      ClusterElewiseSpec e;
      e.name = gets(kv.second, "name", kv.first);
      e.ilp_factor = geti(kv.second, "ilp_factor", 1);
      MONONN_CHECK(e.ilp_factor >= 1 && e.ilp_factor <= 64, kSpecError) << "ilp_factor of " << kv.first << " out of range";
      s.cluster_elewise_spec[kv.first] = e;
    }
  if (j.contains("cluster_reduce_spec"))
    for (auto& kv : j.at("cluster_reduce_spec").members()) {
      check_keys(kv.second, {"name", "ilp_factor", "locality_tier", "reduce_implementation"}, "cluster_reduce_spec entry");
      ClusterReduceSpec e;
      e.name = gets(kv.second, "name", kv.first);
      e.ilp_factor = geti(kv.second, "ilp_factor", 1);
      e.locality_tier = geti(kv.second, "locality_tier", 1);
      e.reduce_implementation = geti(kv.second, "reduce_implementation", 0);
      MONONN_CHECK(e.locality_tier == 1 || e.locality_tier == 2, kSpecError) << "locality_tier of " << kv.first << " must be 1 or 2";
      MONONN_CHECK(e.reduce_implementation >= 0 && e.reduce_implementation <= 3, kSpecError) << "reduce_implementation of " << kv.first << " must be 0 ... 3";
      s.cluster_reduce_spec[kv.first] = e;
    }
  if (j.contains("gemm_spec_list"))
    for (auto& kv : j.at("gemm_spec_list").members()) {
      check_keys(kv.second, {"cutlass_config", "gemm_backend_config"}, "gemm_spec_list entry");
      GemmSpec g;
      const Json& cc = kv.second.at("cutlass_config");
      check_keys(cc, {"threadblockshape", "warpshape", "instructionshape", "operatorclass", "archtag", "stages", "wave_arrangement", "split_k"}, "cutlass_config");
      auto shp = [&](const char* k, int& m, int& n, int& kk) {
        if (!cc.contains(k)) return;
        check_keys(cc.at(k), {"m", "n", "k"}, k);
        m = geti(cc.at(k), "m", m);
        n = geti(cc.at(k), "n", n);
        kk = geti(cc.at(k), "k", kk);
      };
      shp("threadblockshape", g.tb_m, g.tb_n, g.tb_k);
      shp("warpshape", g.warp_m, g.warp_n, g.warp_k);
      shp("instructionshape", g.inst_m, g.inst_n, g.inst_k);
      shp("wave_arrangement", g.wave_m, g.wave_n, g.wave_k);
      if (cc.contains("operatorclass")) g.operator_class = gets(cc.at("operatorclass"), "name", g.operator_class);
      if (cc.contains("archtag")) g.arch_tag = gets(cc.at("archtag"), "name", g.arch_tag);
      g.stages = geti(cc, "stages", 1);
      g.split_k = geti(cc, "split_k", 1);
      MONONN_CHECK(g.split_k >= 1 && g.split_k <= 64, kSpecError) << "split_k of " << kv.first << " out of range";
      if (kv.second.contains("gemm_backend_config")) g.backend_config = kv.second.at("gemm_backend_config");
      s.gemm_spec_list[kv.first] = g;
    }
  if (j.contains("conv_spec_list"))
    for (auto& kv : j.at("conv_spec_list").members()) s.conv_spec_list[kv.first] = kv.second;
  s.codegen_allow_list = strings_from(j, "codegen_allow_list");
  s.codegen_reject_list = strings_from(j, "codegen_reject_list");
  if (j.contains("mononn_hip")) {
    const Json& h = j.at("mononn_hip");
    check_keys(h, {"merge_dependent", "gemm_epilogue_fusion", "transpose_constant_b", "assign_operand_layouts", "fuse_attention", "gemm_prologue_fusion", "layer_norm_folding", "barrier", "profile_stages", "cooperative_launch", "operand_preload", "pack_left_operands", "attention_out_proj_fusion", "stage_rotation", "barrier_timeout_ms", "opaque_thread_id", "regional_synchronization"}, "mononn_hip");
    s.hip.merge_dependent = getb(h, "merge_dependent", true);
    s.hip.gemm_epilogue_fusion = getb(h, "gemm_epilogue_fusion", true);
    s.hip.transpose_constant_b = getb(h, "transpose_constant_b", true);
    s.hip.assign_operand_layouts = getb(h, "assign_operand_layouts", true);
    s.hip.fuse_attention = getb(h, "fuse_attention", true);
    s.hip.gemm_prologue_fusion = getb(h, "gemm_prologue_fusion", false);
    s.hip.layer_norm_folding = getb(h, "layer_norm_folding", false);
    s.hip.barrier = gets(h, "barrier", "flags_coherent");
    s.hip.profile_stages = getb(h, "profile_stages", false);
    s.hip.cooperative_launch = getb(h, "cooperative_launch", false);
    s.hip.barrier_timeout_ms = geti(h, "barrier_timeout_ms", 10000);
    s.hip.opaque_thread_id = getb(h, "opaque_thread_id", false);
    MONONN_CHECK(s.hip.barrier_timeout_ms >= 1 && s.hip.barrier_timeout_ms <= 3600000, kSpecError) << "barrier_timeout_ms must lie in [1, 3600000]";
    s.hip.operand_preload = getb(h, "operand_preload", true);
    s.hip.pack_left_operands = getb(h, "pack_left_operands", true);
    s.hip.attention_out_proj_fusion = getb(h, "attention_out_proj_fusion", false);
    s.hip.stage_rotation = getb(h, "stage_rotation", true);
    s.hip.regional_synchronization = getb(h, "regional_synchronization", false);
  }
  MONONN_CHECK(s.runtime.grid_dim.x >= 1 && s.runtime.grid_dim.y == 1 && s.runtime.grid_dim.z == 1, kSpecError) << "grid must be 1-D";
  MONONN_CHECK(s.runtime.block_dim.x >= 64 && s.runtime.block_dim.x % 64 == 0 && s.runtime.block_dim.x <= 1024 && s.runtime.block_dim.y == 1 && s.runtime.block_dim.z == 1,
               kSpecError)
      << "block must be 1-D, a multiple of 64 and at most 1024 threads";
  return s;
}

}  // namespace spec
}  // namespace mononn
