// Tuning specification ("GraphSpecification") and its JSON form.
//
// The reference keeps this as a protobuf whose schema lives in its absent TensorFlow fork; the
// field names below are reconstructed from the accessors used in-tree
// (mononn_engine/core/context/cuda_context.cc:59-77, cuda_runtime_context.cc:32-55,
// cuda_device_context.cc:117-150, core/gpu/dim3.cc:26-42, core/gpu/cutlass/cutlass_config.cc:32-59,
// gemm_backend_config.cc:36-87, tuning/tuning_space_generator.cc:151-160,184-194,255-269,318-335,
// 405-414) and printed the way helpers/protobuf.cc:32-46 prints them (original field names,
// primitive fields always present).  gfx950-specific choices (wave arrangement of a GEMM tile,
// fusion decisions, barrier flavour) live in the same per-node maps / a `mononn_hip` section.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "common/json.h"

namespace mononn {
namespace spec {

struct Dim3 {
  int x = 1, y = 1, z = 1;
};

struct DeviceContext {      // cuda_device_context
  int device_count = 1;
  int sm_count = 256;                        // compute units
  int static_smem_size = 65536;              // LDS a workgroup may use without opting in
  int max_configurable_smem_size = 163840;   // 160 KiB LDS per CU
  std::string cuda_arch = "gfx950";
  int register_per_block = 131072;           // 512 VGPRs x 64 lanes x 4 SIMDs
  int warp_size = 64;
  int reserved_smem_per_block = 0;
};

struct RuntimeContext {     // cuda_runtime_context
  Dim3 grid_dim, block_dim;
  int smem_size = 0;
  std::string stream = "0";
};

struct ClusterElewiseSpec {
  std::string name;
  int ilp_factor = 1;
};

struct ClusterReduceSpec {
  std::string name;
  int ilp_factor = 1;
  int locality_tier = 1;          // 1 = wave per row, 2 = workgroup per row (reference: warp / block)
  int reduce_implementation = 0;  // tier 1: rows a wave takes at once, 0 = one, 1 / 2 / 3 = 8 / 4 / 2
};

struct GemmSpec {
  // cutlass_config fields re-used with their gfx950 meaning
  int tb_m = 32, tb_n = 32, tb_k = 32;       // threadblockshape: workgroup tile (k = one MFMA step)
  int warp_m = 32, warp_n = 32, warp_k = 32; // warpshape: per-wave tile
  int inst_m = 16, inst_n = 16, inst_k = 32; // instructionshape: v_mfma_f32_16x16x32_f16
  std::string operator_class = "MFMA";
  std::string arch_tag = "gfx950";
  int stages = 1;
  int wave_m = 1, wave_n = 1, wave_k = 4;    // arrangement of the workgroup's waves over the tile
  // > 1: the k range is also split over workgroups; fp32 partial sums go to memory and the consuming
  // cluster adds them up (only for GEMMs without fused epilogue whose readers are all clusters)
  int split_k = 1;
  Json backend_config;                       // gemm_backend_config as carried by the HLO
};

struct HipOptions {       // "mononn_hip" section
  bool merge_dependent = true;
  bool gemm_epilogue_fusion = true;
  bool transpose_constant_b = true;
  bool assign_operand_layouts = true;
  bool fuse_attention = true;
  // LayerNorm inside the consuming GEMM: removes a stage and a barrier but every column tile repeats the
  // row program on its rows, which only pays off when a GEMM has few column tiles; off unless tuned on
  bool gemm_prologue_fusion = false;
  bool layer_norm_folding = false;   // with gemm_prologue_fusion: a LayerNorm in front of a constant-weight GEMM is folded into weights and epilogue
  // "flags_coherent": fence-free flag barrier; stage outputs are written with agent-scope write-through
  // stores to temp addresses that are used once per launch, readers use cached loads.
  // "flags": the same barrier with agent-scope release/acquire (L2 write-back + invalidate) around it,
  // plain stores, temp slots re-used.  "flags_allfence": every thread fences (measurement only).
  std::string barrier = "flags_coherent";
  bool profile_stages = false;   // per-stage wall-clock stamps (performance_report.csv equivalent)
  // false: ordinary kernel launch, as the reference does (mononn_module_tuner.cc:135-139); the grid is checked
  // against the co-resident capacity at load time, and launches of such kernels must not overlap on the device
  // (two half-resident grids would wait for each other at their first barrier).  true: cooperative launch, the
  // runtime keeps such kernels apart at the price of ~20 us more per launch.
  bool cooperative_launch = false;
  // A grid-barrier wait that is still polling this long after the kernel started gives up (the kernel then runs to
  // its end and the host finds an error word): what stands between a grid that is not wholly resident and a hang.
  int barrier_timeout_ms = 10000;
  // Node functions re-read the thread index where they use it instead of letting the compiler derive lane numbers and
  // address parts of all stages once, ahead of the stage loop (values that then live through every stage).  Always
  // on in kernels with an LDS-staged GEMM, whose register tile would push those values out to scratch.
  bool opaque_thread_id = false;
  // GEMM stages request their packed weights between announcing the end of the previous stage and waiting for the
  // other workgroups (the wait moves behind the requests; idle workgroups skip it)
  bool operand_preload = true;
  // values of this kernel that only GEMMs read as their left operand are stored in MFMA fragment order
  bool pack_left_operands = true;
  // the projection of the merged heads runs inside the attention stage, one fp32 partial sum per head; the stage
  // of the projection disappears, its bias / residual epilogue moves into the row program that follows
  bool attention_out_proj_fusion = false;
  // a stage whose units fit beside those of the stage before it runs on the workgroups that stage left idle
  bool stage_rotation = true;
  // Regional synchronisation (regional_synchronization_assignment_pass.cc:35-72 in the reference): chains of stages
  // whose hand-overs can be kept inside one XCD (a GEMM's column slices feeding the k slices of the next GEMM; the
  // heads of a projection feeding the attention and its output projection) are dealt to the XCDs by ownership, their
  // intermediate results are written with ordinary stores and the barrier between them is one over the XCD's 32
  // workgroups through its L2.  Takes effect on a grid of one workgroup per compute unit with the "flags_coherent" barrier.
  bool regional_synchronization = false;
};

struct GraphSpecification {
  RuntimeContext runtime;
  DeviceContext device;
  std::string hlo_module_proto_file;
  std::vector<std::string> feeds, input_data_files, fetches;
  std::map<std::string, ClusterElewiseSpec> cluster_elewise_spec;
  std::map<std::string, ClusterReduceSpec> cluster_reduce_spec;
  std::map<std::string, GemmSpec> gemm_spec_list;
  std::map<std::string, Json> conv_spec_list;
  std::vector<std::string> codegen_allow_list, codegen_reject_list;
  HipOptions hip;

  Json to_json() const;
  // unknown keys are rejected like the reference's loader does (helpers/protobuf.cc:48-65)
  static GraphSpecification from_json(const Json& j);
  // "<gx>_<gy>_<gz>__<bx>_<by>_<bz>" (mononn_module_tuner.cc:374-383)
  std::string context_string() const;
};

}  // namespace spec
}  // namespace mononn
