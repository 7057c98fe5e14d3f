// The one translation unit of the library that carries device data: a fixed arena in the library's gfx950 image.
// mononn_launch_static_temp hands it to the kernel as the temp buffer, so that entry point allocates nothing.
#include "runtime/static_scratch.h"

#include <hip/hip_runtime.h>

#include <mutex>

namespace {

constexpr size_t kScratchBytes = size_t(64) << 20;   // BERT-base b1 s128 needs 48 MB with write-once temp addresses
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
struct PerDevice {
  bool tried = false;
  void* ptr = nullptr;   // device address of `scratch` on this GPU (each GPU has its own copy at its own address)
  std::string error;
};
PerDevice g_devices[kMaxDevices];
std::mutex g_mutex;

}  // namespace

namespace mononn {
namespace runtime {

size_t static_scratch_bytes() { return kScratchBytes; }

bool static_scratch_setup(int device, std::string* error) {
  if (device < 0 || device >= kMaxDevices) {
    if (error) *error = "device ordinal outside the static scratch table";
    return false;
  }
  std::lock_guard<std::mutex> lock(g_mutex);
  PerDevice& d = g_devices[device];
  if (!d.tried) {
    d.tried = true;
    // In host code the array's name is only a handle for the runtime; the address the kernels can use comes from here.
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      (void)hipGetLastError();
      d.error = std::string("hipGetSymbolAddress(static scratch): ") + hipGetErrorString(e);
    } else {
      d.ptr = p;
    }
  }
  if (!d.ptr && error) *error = d.error;
  return d.ptr != nullptr;
}

void* static_scratch_address(int device) {
  if (device < 0 || device >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_mutex);
  return g_devices[device].ptr;
}

}  // namespace runtime
}  // namespace mononn
