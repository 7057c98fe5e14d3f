#include "runtime/device_module.h"

#include <hip/hip_runtime.h>

#include <dlfcn.h>

#include <cstdlib>

#include <algorithm>
#include <mutex>

#include "common/status.h"

#define HIP_OK(expr)                                                                                         \
  do {                                                                                                       \
    hipError_t e_ = (expr);                                                                                  \
    if (e_ != hipSuccess) MONONN_FAIL(kRuntimeError) << #expr << ": " << hipGetErrorString(e_);              \
  } while (0)

namespace mononn {
namespace runtime {

int device_count() {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

bool profiler_tool_attached() {
  // rocprofv3 starts its target with the tool library named in ROCP_TOOL_LIBRARIES and mapped into the process
  for (const char* var : {"ROCP_TOOL_LIBRARIES", "HSA_TOOLS_LIB"}) {
    const char* v = std::getenv(var);
    if (v && *v) return true;
  }
  for (const char* lib : {"librocprofiler-sdk-tool.so", "librocprofiler-sdk-tool.so.1", "librocprofiler64.so.2"}) {
    if (void* h = dlopen(lib, RTLD_NOLOAD | RTLD_LAZY)) {
      dlclose(h);
      return true;
    }
  }
  return false;
}

DeviceProperties query_device(int device) {
  MONONN_CHECK(device >= 0 && device < device_count(), kRuntimeError) << "no GPU with ordinal " << device << " is visible";
  hipDeviceProp_t p;
  HIP_OK(hipGetDeviceProperties(&p, device));
  DeviceProperties d;
  d.device = device;
  d.compute_units = p.multiProcessorCount;
  d.wave_size = p.warpSize;
  d.max_lds_per_block = static_cast<int>(p.sharedMemPerBlock);
  d.regs_per_block = p.regsPerBlock;
  d.cooperative_launch = p.cooperativeLaunch;
  d.arch = p.gcnArchName;
  size_t colon = d.arch.find(':');
  if (colon != std::string::npos) d.arch = d.arch.substr(0, colon);
  d.name = p.name;
  return d;
}

DeviceModule::~DeviceModule() {
  if (module_) (void)hipModuleUnload(module_);
}

void DeviceModule::unload() {
  if (module_) {
    (void)hipModuleUnload(module_);
    module_ = nullptr;
    function_ = nullptr;
  }
}

void DeviceModule::load(int device, const std::vector<char>& code_object, const std::string& kernel_name) {
  MONONN_CHECK(!code_object.empty(), kInvalidArgument) << "module has no code object";
  DeviceProperties props = query_device(device);
  MONONN_CHECK(props.cooperative_launch, kRuntimeError) << "device " << device << " does not support cooperative launch";
  HIP_OK(hipSetDevice(device));
  unload();
  hipModule_t m;
  HIP_OK(hipModuleLoadData(&m, code_object.data()));
  hipFunction_t f;
  hipError_t e = hipModuleGetFunction(&f, m, kernel_name.c_str());
  if (e != hipSuccess) {
    (void)hipModuleUnload(m);
    MONONN_FAIL(kRuntimeError) << "kernel '" << kernel_name << "' not found in the code object: " << hipGetErrorString(e);
  }
  module_ = m;
  function_ = f;
  device_ = device;
  compute_units_ = props.compute_units;
}

void DeviceModule::use_kernel(const std::string& kernel_name) {
  MONONN_CHECK(module_ != nullptr, kRuntimeError) << "module is not loaded";
  hipFunction_t f;
  hipError_t e = hipModuleGetFunction(&f, module_, kernel_name.c_str());
  if (e != hipSuccess) MONONN_FAIL(kRuntimeError) << "kernel '" << kernel_name << "' not found in the code object: " << hipGetErrorString(e);
  function_ = f;
}

void* DeviceModule::global(const std::string& symbol, size_t* bytes) const {
  MONONN_CHECK(module_ != nullptr, kRuntimeError) << "module is not loaded";
  hipDeviceptr_t p = nullptr;
  size_t n = 0;
  hipError_t e = hipModuleGetGlobal(&p, &n, module_, symbol.c_str());
  if (e != hipSuccess) MONONN_FAIL(kNotFound) << "module global '" << symbol << "': " << hipGetErrorString(e);
  if (bytes) *bytes = n;
  return p;
}

void DeviceModule::upload(void* dst, const void* host_src, size_t bytes) const {
  HIP_OK(hipSetDevice(device_));
  HIP_OK(hipMemcpy(dst, host_src, bytes, hipMemcpyHostToDevice));
}

void DeviceModule::zero(void* dst, size_t bytes) const {
  HIP_OK(hipSetDevice(device_));
  HIP_OK(hipMemset(dst, 0, bytes));
  HIP_OK(hipDeviceSynchronize());
}

void DeviceModule::download(void* host_dst, const void* src, size_t bytes) const {
  HIP_OK(hipSetDevice(device_));
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipMemcpy(host_dst, src, bytes, hipMemcpyDeviceToHost));
}

void DeviceModule::synchronize(void* stream) const {
  HIP_OK(hipSetDevice(device_));
  HIP_OK(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}

double DeviceModule::wall_clock_ticks_per_us() const {
  int khz = 0;
  HIP_OK(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device_));
  return khz / 1000.0;
}

int DeviceModule::max_coresident_blocks(int block, int smem) const {
  MONONN_CHECK(module_ != nullptr, kRuntimeError) << "module is not loaded";
  int per_cu = 0;
  HIP_OK(hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, function_, block, static_cast<size_t>(smem)));
  return per_cu * compute_units_;
}

void DeviceModule::set_dynamic_smem(int smem) const {
  if (smem > 48 * 1024) HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(function_), hipFuncAttributeMaxDynamicSharedMemorySize, smem));
}

void DeviceModule::launch(int grid, int block, int smem, void** args, void* stream, bool cooperative) const {
  MONONN_CHECK(module_ != nullptr, kRuntimeError) << "module is not loaded";
  if (cooperative) HIP_OK(hipModuleLaunchCooperativeKernel(function_, grid, 1, 1, block, 1, 1, smem, static_cast<hipStream_t>(stream), args));
  else HIP_OK(hipModuleLaunchKernel(function_, grid, 1, 1, block, 1, 1, smem, static_cast<hipStream_t>(stream), args, nullptr));
}

float DeviceModule::time_launches(int grid, int block, int smem, void** args, void* stream, int warmup, int iters,
                                  std::vector<float>* per_launch_ms, bool cooperative) const {
  hipStream_t s = static_cast<hipStream_t>(stream);
  for (int i = 0; i < warmup; ++i) launch(grid, block, smem, args, stream, cooperative);
  HIP_OK(hipStreamSynchronize(s));
  std::vector<hipEvent_t> ev(static_cast<size_t>(iters) + 1);
  for (auto& e : ev) HIP_OK(hipEventCreate(&e));
  HIP_OK(hipEventRecord(ev[0], s));
  for (int i = 0; i < iters; ++i) {
    launch(grid, block, smem, args, stream, cooperative);
    HIP_OK(hipEventRecord(ev[i + 1], s));
  }
  HIP_OK(hipEventSynchronize(ev[iters]));
  float total = 0.f;
  HIP_OK(hipEventElapsedTime(&total, ev[0], ev[iters]));
  if (per_launch_ms) {
    per_launch_ms->resize(iters);
    for (int i = 0; i < iters; ++i) HIP_OK(hipEventElapsedTime(&(*per_launch_ms)[i], ev[i], ev[i + 1]));
  }
  for (auto& e : ev) (void)hipEventDestroy(e);
  return total / static_cast<float>(iters);
}

}  // namespace runtime
}  // namespace mononn
