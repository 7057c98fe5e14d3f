// hipRTC front end: generated HIP source -> gfx950 code object, in process.
// The reference writes the sources to a temp dir and forks `make` + nvcc
// (mononn_engine/module/mononn_module.cc:161-193, codegen/cuda_program.cc:131-167).
#pragma once
#include <map>
#include <string>
#include <vector>

namespace mononn {
namespace runtime {

struct CompileResult {
  std::vector<char> code_object;
  std::string log;
};

// `files` must contain `main_file`; every other entry is offered as an include.
// Throws Error(kCompileError) with the compiler log on failure.
CompileResult compile_hip(const std::map<std::string, std::string>& files, const std::string& main_file,
                          const std::string& arch, const std::vector<std::string>& extra_options = {});

}  // namespace runtime
}  // namespace mononn
