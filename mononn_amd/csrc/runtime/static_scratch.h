// A temp arena that lives in the library's own device image, for callers of the launch path that must not allocate
// device memory (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).
#pragma once
#include <cstddef>
#include <string>

namespace mononn {
namespace runtime {

// size of the arena every GPU holds from the first set-up on that GPU until the process ends
size_t static_scratch_bytes();
// Looks the arena's device address up once per device; `device` must be the current device.  Returns false and
// fills `error` when the runtime refuses; later calls for the same device return the recorded outcome.
bool static_scratch_setup(int device, std::string* error);
// device address of the arena on `device`, nullptr before a successful set-up
void* static_scratch_address(int device);

}  // namespace runtime
}  // namespace mononn
