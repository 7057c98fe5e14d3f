// A code object loaded on one GPU: kernel handle, module globals, cooperative launch, timing.
// Reference counterpart: the stream-executor calls of profile_kernel
// (mononn_engine/module/mononn_module_tuner.cc:90-151: CreateKernel, FuncSetAttribute(max dynamic
// shared size), Launch, BlockHostUntilDone) and the device query of
// mononn_engine/core/context/cuda_device_context.cc:42-80 / cuda_utils.cu.cc:51-104.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

struct ihipModule_t;
struct ihipModuleSymbol_t;
struct ihipStream_t;

namespace mononn {
namespace runtime {

struct DeviceProperties {
  int device = 0;
  int compute_units = 0;
  int wave_size = 0;
  int max_lds_per_block = 0;
  int regs_per_block = 0;
  int cooperative_launch = 0;
  std::string arch;     // "gfx950"
  std::string name;
};

int device_count();                           // 0 when no GPU is visible (never throws)
// a profiler tool library (rocprofv3 and its predecessors) is mapped into this process or named in its environment
bool profiler_tool_attached();
DeviceProperties query_device(int device);    // throws Error(kRuntimeError) without a GPU

class DeviceModule {
 public:
  DeviceModule() = default;
  ~DeviceModule();
  DeviceModule(const DeviceModule&) = delete;
  DeviceModule& operator=(const DeviceModule&) = delete;

  void load(int device, const std::vector<char>& code_object, const std::string& kernel_name);
  bool loaded() const { return module_ != nullptr; }
  void use_kernel(const std::string& kernel_name);   // switch to another kernel of the loaded code object
  int device() const { return device_; }

  // address and size of a module global
  void* global(const std::string& symbol, size_t* bytes) const;
  void upload(void* dst, const void* host_src, size_t bytes) const;
  void zero(void* dst, size_t bytes) const;
  void download(void* host_dst, const void* src, size_t bytes) const;   // synchronises the device first
  void synchronize(void* stream) const;
  double wall_clock_ticks_per_us() const;

  // workgroups of `block` threads and `smem` bytes of LDS that can be resident on the whole device
  int max_coresident_blocks(int block, int smem) const;
  void set_dynamic_smem(int smem) const;
  // one cooperative launch; args = array of pointers to the argument values
  void launch(int grid, int block, int smem, void** args, void* stream, bool cooperative = false) const;
  // average milliseconds per launch over `iters` launches after `warmup`
  float time_launches(int grid, int block, int smem, void** args, void* stream, int warmup, int iters,
                      std::vector<float>* per_launch_ms = nullptr, bool cooperative = false) const;
  void unload();

 private:
  int device_ = -1;
  ihipModule_t* module_ = nullptr;
  ihipModuleSymbol_t* function_ = nullptr;
  int compute_units_ = 0;
};

}  // namespace runtime
}  // namespace mononn
