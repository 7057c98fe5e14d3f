// Standalone host driver for a generated kernel: a self-contained HIP program that loads the code object,
// fills the module's constants, allocates the buffers, runs the kernel and reports its time, with no
// dependency on this library ("use the kernel without the framework").
//
// Reference counterpart: HostCodegen::generate (mononn_engine/codegen/host_codegen.cc:31-73) together with the
// README's recipe for running the dumped kernel by hand (README.md:179-200).
#pragma once
#include <string>

#include "codegen/kernel_codegen.h"

namespace mononn {
namespace codegen {

// Text of host_main.cpp for `hp`.  The program takes: <code object> [constants dir] [iterations].
std::string generate_host_driver(const HipProgram& hp);

}  // namespace codegen
}  // namespace mononn
