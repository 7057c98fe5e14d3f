// Whole-program code generation: one `extern "C" __global__` function for the module.
//
// Reference counterpart: GraphCodegen::generate (mononn_engine/codegen/graph_codegen.cc:637-842):
// helper prelude, one device function per cluster, then the kernel whose body is buffer-pointer
// setup followed by the nodes in topological order with grid barriers between dependent groups.
// Argument order is the reference's (mononn_engine/module/mononn_module.cc:91-143): entry
// parameters, one `liveout_buffer_<i>` per live-out, then `temp_buffer`; non-scalar constants are
// `buffer_for_<node>` device globals that the host fills before launch (graph_codegen.cc:71-86).
// Unlike the reference, node functions that come out textually identical (the same layer
// repeated) are emitted once and called with different pointers, which keeps the instruction
// working set of a 12-layer kernel at one layer's worth.
#pragma once
#include <map>
#include <string>
#include <vector>

#include "graph/program.h"
#include "spec/spec.h"

namespace mononn {
namespace codegen {

struct ConstantInfo {
  std::string name;        // canonical HLO name
  std::string hlo_name;
  std::string symbol;      // buffer_for_<name>
  std::string role;        // metadata op_name when present
  int64_t bytes = 0;          // payload size in the HLO layout (what the host passes in)
  int64_t device_bytes = 0;   // size of the module global (padded when re-laid out)
  hlo::DType dtype = hlo::DType::kInvalid;
  std::vector<int64_t> dims;
  graph::ConstantTransform transform = graph::ConstantTransform::kNone;
  std::string literal;     // payload text when the HLO carries it (not elided)
  // folded LayerNorms (graph::LayerNormFold): a weight matrix whose row k is multiplied by element k of the named
  // [K] constant before it is laid out for the device ...
  std::string row_scale_by;
  // ... and a constant the host never supplies: f32[N] = sum_k vector[k] * weight[k, n] of two named constants
  std::string sums_weight, sums_vector;
  bool derived() const { return !sums_weight.empty(); }
};

struct NodeReport {
  std::string name, kind, function;
  int stage = 0;
  int64_t units = 0;
  std::string partition;   // regional synchronisation: "columns/8", "split_k/8", "heads/6", or empty
};

struct HipProgram {
  std::string kernel_name;
  std::map<std::string, std::string> files;   // "headers.h" (device runtime) and "main.hip"
  // main.hip = preamble + global_decls + body; kept apart for multi-candidate translation units
  std::string preamble, body;
  std::vector<std::string> global_decls;
  std::vector<int64_t> param_bytes, liveout_bytes;
  int64_t temp_bytes = 0;
  std::vector<ConstantInfo> constants;
  std::vector<NodeReport> nodes;
  int num_barriers = 0;
  // of which barriers of the regional tier (over the workgroups of one XCD); regional_before[s]: the barrier in front
  // of emitted stage s is one
  int num_regional_barriers = 0;
  std::vector<bool> regional_before;
  bool cooperative = false;   // launch through the cooperative-launch entry point
  int grid = 0, block = 0, smem = 0;
  int max_grid = 4096;       // barrier flag capacity
  int num_stages = 0;        // stages that were emitted
  bool profiled = false;     // kernel writes mononn_stage_clock[stage][workgroup][2]
  std::vector<std::vector<std::string>> stage_nodes;   // node names per emitted stage
};

// Fills `spec` with defaults for nodes it does not mention, validates the rest (a spec naming a
// node the graph does not have is an error, cf. mononn_module.cc:83-85) and generates the source.
HipProgram generate_program(const graph::Program& prog, spec::GraphSpecification& spec, const std::string& kernel_name);

graph::BuildOptions build_options_from(const spec::GraphSpecification& spec);

}  // namespace codegen
}  // namespace mononn
