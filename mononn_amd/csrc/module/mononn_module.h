// MonoNNModule: one HLO module + one tuning specification -> HIP source -> gfx950 code object,
// and, once loaded on a GPU, a single kernel launch per forward pass.
//
// Mirrors mononn_engine/module/mononn_module.h:31-87 (generate_code, build_assembly, get_ptx /
// get_cubin / get_tuning_spec / get_cuda_program).  Differences forced by the platform: the HLO
// arrives as text (no xla::HloModule), buffer offsets are assigned here rather than taken from
// XLA's BufferAssignment, the "assembly" is a code object produced in process by hipRTC, and the
// module also owns the device-side state the reference's TensorFlow fork keeps (loaded kernel,
// constant buffers).
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "codegen/kernel_codegen.h"
#include "graph/program.h"
#include "runtime/device_module.h"
#include "spec/spec.h"

namespace mononn {
namespace module {

class MonoNNModule {
 public:
  // spec_json may be empty: defaults are derived for every node
  MonoNNModule(const std::string& hlo_text, const std::string& spec_json, const std::string& kernel_name = "");
  ~MonoNNModule();
  bool owns_temp() const { return false; }   // the caller always brings the temp buffer (reference contract)

  void generate_code();                       // parse, run the passes, emit HIP source
  void build_assembly();                      // hipRTC -> code object (needs generate_code)
  bool has_code_object() const { return !code_object_.empty(); }
  void set_code_object(const std::vector<char>& co) { code_object_ = co; }   // cached build (best_tuning_spec.hsaco)
  // Key of what a code object of this module is built from: the generated sources (kernel, device prelude) and the
  // compiler options.  Written beside a cached code object, compared before that cache is used.
  std::string source_key() const;

  const std::string& kernel_name() const { return kernel_name_; }
  const std::string& module_name() const { return module_name_; }
  const spec::GraphSpecification& tuning_spec() const { return spec_; }
  spec::GraphSpecification& mutable_tuning_spec() { return spec_; }
  std::string tuning_spec_json() const { return spec_.to_json().dump(1); }
  const codegen::HipProgram& hip_program() const { return hip_; }
  const std::vector<char>& code_object() const { return code_object_; }
  const std::string& compile_log() const { return compile_log_; }
  const graph::Program& program() const { return *program_; }
  std::string summary() const;

  // ---- device side ---------------------------------------------------------------------------
  // Payload of a non-scalar constant, in the layout the HLO declares; the module re-lays it out
  // when a pass decided so (transposed GEMM operands).  Accepts the canonical or the HLO name.
  void set_constant(const std::string& name, const void* host_data, size_t bytes);
  void load(int device);                      // load code object, fit grid to the device, upload constants
  bool loaded() const { return dev_.loaded(); }
  // args: entry parameters in order, live-out buffers in order, temp buffer (device pointers)
  void launch(void* const* device_ptrs, size_t n, void* stream);
  // the same launch with the library's static device arena as temp buffer: device_ptrs = parameters, live-outs
  void launch_static_temp(void* const* device_ptrs, size_t n, void* stream);
  // waits for `stream` and reports a grid-barrier wait that gave up (kRuntimeError; flags are reset, the module stays usable)
  void synchronize(void* stream);
  void* global_address(const std::string& symbol, size_t* bytes) const;
  float time_kernel(void* const* device_ptrs, size_t n, void* stream, int warmup, int iters, std::vector<float>* each = nullptr);
  int grid() const { return grid_; }
  int block() const { return hip_.block; }
  int smem() const { return hip_.smem; }
  size_t num_args() const { return hip_.param_bytes.size() + hip_.liveout_bytes.size() + 1; }
  std::vector<std::string> missing_constants() const;
  // Stage clocks of the last launch of a kernel built with mononn_hip.profile_stages: for every
  // emitted stage and workgroup, [begin, end-of-work] wall-clock ticks.  Returns ticks per microsecond.
  double read_stage_clock(std::vector<unsigned long long>* ticks, int* n_stages, int* grid);

  // ---- dump (TF_MONONN_DUMP_DIR layout, mononn_module_tuner.cc:457-603) ------------------------
  // writes <dir>/<cluster_N>/<context>.json, <context>.hsaco, <context>_src/{headers.h,main.hip}
  void dump_candidate(const std::string& dump_dir) const;
  // writes best_tuning_spec.{json,hsaco}
  void dump_best(const std::string& dump_dir) const;
  std::string cluster_dir(const std::string& dump_dir) const;

 private:
  void prepare_args(std::vector<void*>& vals) const;
  void upload_constant(const codegen::ConstantInfo& ci, const std::vector<char>& payload);
  std::string hlo_text_;
  std::string module_name_;
  std::string kernel_name_;
  spec::GraphSpecification spec_;
  bool spec_given_ = false;
  std::unique_ptr<graph::Program> program_;
  codegen::HipProgram hip_;
  std::vector<char> code_object_;
  std::string compile_log_;
  runtime::DeviceModule dev_;
  int grid_ = 0;
  std::map<std::string, std::vector<char>> host_constants_;   // canonical name -> payload as given
  std::map<std::string, bool> uploaded_;
  // payloads that outlive load(): the sources of folded LayerNorms (weights, gamma, beta), from which scaled weights
  // and column sums are rebuilt whenever one of them is supplied again
  std::map<std::string, std::vector<char>> fold_sources_;
  bool is_fold_source(const std::string& name) const;
  const std::vector<char>* raw_payload(const std::string& name, std::vector<char>* scratch) const;
  // bytes of the module global of `ci`, built from whatever payloads are at hand; false while a source is missing
  bool resolve_device_bytes(const codegen::ConstantInfo& ci, std::vector<char>* out) const;
  void upload_resolved(const codegen::ConstantInfo& ci);
  std::string static_scratch_error_;   // why the static temp arena has no address on this device ("" when it has)
};

// helpers shared with the tuner / CLI
void write_file(const std::string& path, const std::string& data);
void write_file(const std::string& path, const std::vector<char>& data);
bool read_file(const std::string& path, std::string* out);
void make_dirs(const std::string& path);

}  // namespace module
}  // namespace mononn
