#include "runtime/rtc.h"

#include <cstdlib>
#include <sstream>

#include <hip/hiprtc.h>

#include "common/status.h"

namespace mononn {
namespace runtime {

CompileResult compile_hip(const std::map<std::string, std::string>& files, const std::string& main_file,
                          const std::string& arch, const std::vector<std::string>& extra_options) {
  auto mf = files.find(main_file);
  MONONN_CHECK(mf != files.end(), kInternal) << "compile_hip: no file named " << main_file;
  std::vector<const char*> hdr_src, hdr_name;
  for (auto& kv : files) {
    if (kv.first == main_file) continue;
    hdr_src.push_back(kv.second.c_str());
    hdr_name.push_back(kv.first.c_str());
  }
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, mf->second.c_str(), main_file.c_str(), static_cast<int>(hdr_src.size()),
                                       hdr_src.data(), hdr_name.data());
  MONONN_CHECK(r == HIPRTC_SUCCESS, kCompileError) << "hiprtcCreateProgram: " << hiprtcGetErrorString(r);
  std::vector<std::string> opts = {"--offload-arch=" + arch, "-O3", "-std=c++17",
                                   // keep the compiler from forming packed fp32 instructions
                                   "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  for (auto& o : extra_options) opts.push_back(o);
  // extra compiler options, blank separated (e.g. "-mllvm -amdgpu-sched-strategy=max-ilp")
  if (const char* x = std::getenv("MONONN_HIPRTC_FLAGS")) {
    std::istringstream is(x);
    std::string tok;
    while (is >> tok) opts.push_back(tok);
  }
  std::vector<const char*> copts;
  for (auto& o : opts) copts.push_back(o.c_str());
  r = hiprtcCompileProgram(prog, static_cast<int>(copts.size()), copts.data());
  CompileResult out;
  size_t log_size = 0;
  if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
    out.log.resize(log_size);
    hiprtcGetProgramLog(prog, &out.log[0]);
    while (!out.log.empty() && out.log.back() == '\0') out.log.pop_back();
  }
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    MONONN_FAIL(kCompileError) << "hipRTC compilation failed (" << hiprtcGetErrorString(r) << "):\n" << out.log;
  }
  size_t code_size = 0;
  r = hiprtcGetCodeSize(prog, &code_size);
  MONONN_CHECK(r == HIPRTC_SUCCESS && code_size > 0, kCompileError) << "hiprtcGetCodeSize: " << hiprtcGetErrorString(r);
  out.code_object.resize(code_size);
  r = hiprtcGetCode(prog, out.code_object.data());
  hiprtcDestroyProgram(&prog);
  MONONN_CHECK(r == HIPRTC_SUCCESS, kCompileError) << "hiprtcGetCode: " << hiprtcGetErrorString(r);
  return out;
}

}  // namespace runtime
}  // namespace mononn
