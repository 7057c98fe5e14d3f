#include "codegen/host_codegen.h"

#include <sstream>

namespace mononn {
namespace codegen {

std::string generate_host_driver(const HipProgram& hp) {
  std::ostringstream s;
  s << "// Standalone driver for kernel " << hp.kernel_name << " (generated; no library needed).\n"
    << "//   build:  hipcc -O2 host_main.cpp -o host_main\n"
    << "//   run:    ./host_main <code object .hsaco> [constants dir] [iterations]\n"
    << "// Constants are read from <constants dir>/<symbol>.bin (bytes in the layout of the module global, as written\n"
    << "// by the module dump); a constant without a file is filled with small fp16 values so that the kernel still\n"
    << "// does representative work.  Parameters are zero-filled; live-outs are written to liveout_<i>.bin.\n"
    << "#include <hip/hip_runtime.h>\n\n#include <cstdio>\n#include <cstdlib>\n#include <cstring>\n#include <fstream>\n#include <string>\n#include <vector>\n\n"
    << "#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::fprintf(stderr, \"%s:%d: %s\\n\", __FILE__, __LINE__, hipGetErrorString(e_)); return 1; } } while (0)\n\n"
    << "struct Constant { const char* symbol; size_t bytes; };\n"
    << "static const Constant kConstants[] = {\n";
  for (auto& c : hp.constants) s << "  {\"" << c.symbol << "\", " << c.device_bytes << "},\n";
  s << "  {nullptr, 0}};\n";
  auto list = [&](const char* name, const std::vector<int64_t>& v) {
    s << "static const size_t " << name << "[] = {";
    for (size_t i = 0; i < v.size(); ++i) s << (i ? ", " : "") << v[i];
    if (v.empty()) s << "0";
    s << "};\n";
  };
  list("kParamBytes", hp.param_bytes);
  list("kLiveoutBytes", hp.liveout_bytes);
  s << "static const int kNumParams = " << hp.param_bytes.size() << ", kNumLiveouts = " << hp.liveout_bytes.size() << ";\n"
    << "static const size_t kTempBytes = " << hp.temp_bytes << ";\n"
    << "static const int kGrid = " << hp.grid << ", kBlock = " << hp.block << ", kSmem = " << hp.smem << ";\n"
    << "static const bool kCooperative = " << (hp.cooperative ? "true" : "false") << ";\n"
    << "static const char* kKernel = \"" << hp.kernel_name << "\";\n\n"
    << R"(static bool read_file(const std::string& path, std::vector<char>* out) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return false;
  out->assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
  return true;
}

int main(int argc, char** argv) {
  if (argc < 2) {
    std::fprintf(stderr, "usage: %s <code object> [constants dir] [iterations]\n", argv[0]);
    return 2;
  }
  const std::string const_dir = argc > 2 ? argv[2] : "";
  const int iters = argc > 3 ? std::atoi(argv[3]) : 100;
  std::vector<char> image;
  if (!read_file(argv[1], &image)) {
    std::fprintf(stderr, "cannot read %s\n", argv[1]);
    return 2;
  }
  CHECK(hipSetDevice(0));
  hipModule_t mod;
  hipFunction_t fn;
  CHECK(hipModuleLoadData(&mod, image.data()));
  CHECK(hipModuleGetFunction(&fn, mod, kKernel));
  if (kSmem > 48 * 1024) CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, kSmem));

  // constants: module globals buffer_for_<node>, filled by the host before the first launch
  for (const Constant* c = kConstants; c->symbol; ++c) {
    hipDeviceptr_t dst;
    size_t n = 0;
    CHECK(hipModuleGetGlobal(&dst, &n, mod, c->symbol));
    std::vector<char> data;
    if (const_dir.empty() || !read_file(const_dir + "/" + c->symbol + ".bin", &data)) {
      data.resize(c->bytes);
      unsigned short* h = reinterpret_cast<unsigned short*>(data.data());
      for (size_t i = 0; i < c->bytes / 2; ++i) h[i] = static_cast<unsigned short>(0x2000u + ((i * 2654435761u) >> 22));   // ~0.008 .. 0.016
    }
    if (data.size() > n) data.resize(n);
    CHECK(hipMemcpyHtoD(dst, data.data(), data.size()));
  }
  {
    hipDeviceptr_t flags;
    size_t n = 0;
    CHECK(hipModuleGetGlobal(&flags, &n, mod, "mononn_barrier_flags"));
    CHECK(hipMemsetD8(flags, 0, n));
  }

  // buffers: entry parameters, live-outs, temp arena -- the kernel's arguments, in that order
  std::vector<void*> bufs;
  auto alloc = [&](size_t bytes) -> int {
    void* p = nullptr;
    CHECK(hipMalloc(&p, bytes ? bytes : 256));
    CHECK(hipMemset(p, 0, bytes ? bytes : 256));
    bufs.push_back(p);
    return 0;
  };
  for (int i = 0; i < kNumParams; ++i)
    if (alloc(kParamBytes[i])) return 1;
  for (int i = 0; i < kNumLiveouts; ++i)
    if (alloc(kLiveoutBytes[i])) return 1;
  if (alloc(kTempBytes)) return 1;
  for (int i = 0; i < kNumParams; ++i) {   // optional inputs: param_<i>.bin next to the constants
    std::vector<char> data;
    if (!const_dir.empty() && read_file(const_dir + "/param_" + std::to_string(i) + ".bin", &data) && data.size() == kParamBytes[i])
      CHECK(hipMemcpy(bufs[i], data.data(), data.size(), hipMemcpyHostToDevice));
  }
  std::vector<void*> args(bufs.size());
  for (size_t i = 0; i < bufs.size(); ++i) args[i] = &bufs[i];

  auto launch = [&]() -> hipError_t {
    return kCooperative ? hipModuleLaunchCooperativeKernel(fn, kGrid, 1, 1, kBlock, 1, 1, kSmem, nullptr, args.data())
                        : hipModuleLaunchKernel(fn, kGrid, 1, 1, kBlock, 1, 1, kSmem, nullptr, args.data(), nullptr);
  };
  for (int i = 0; i < 10; ++i) CHECK(launch());
  CHECK(hipDeviceSynchronize());
  hipEvent_t t0, t1;
  CHECK(hipEventCreate(&t0));
  CHECK(hipEventCreate(&t1));
  CHECK(hipEventRecord(t0, nullptr));
  for (int i = 0; i < iters; ++i) CHECK(launch());
  CHECK(hipEventRecord(t1, nullptr));
  CHECK(hipEventSynchronize(t1));
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, t0, t1));
  std::printf("%s: grid %d x block %d, %d iterations, %.2f us per launch\n", kKernel, kGrid, kBlock, iters, ms * 1000.f / iters);
  {
    // a grid-barrier wait that ran out of time leaves the ordinal of its barrier here (the kernel still ends)
    hipDeviceptr_t err;
    size_t n = 0;
    unsigned word = 0;
    CHECK(hipModuleGetGlobal(&err, &n, mod, "mononn_barrier_error"));
    CHECK(hipMemcpyDtoH(&word, err, sizeof(word)));
    if (word != 0) {
      std::fprintf(stderr, "a workgroup gave up waiting at grid barrier %u: the grid was not resident as a whole; results are invalid\n", word);
      return 3;
    }
  }

  for (int i = 0; i < kNumLiveouts; ++i) {
    std::vector<char> out(kLiveoutBytes[i]);
    CHECK(hipMemcpy(out.data(), bufs[kNumParams + i], out.size(), hipMemcpyDeviceToHost));
    std::ofstream f("liveout_" + std::to_string(i) + ".bin", std::ios::binary);
    f.write(out.data(), static_cast<std::streamsize>(out.size()));
  }
  for (void* p : bufs) (void)hipFree(p);
  (void)hipModuleUnload(mod);
  return 0;
}
)";
  return s.str();
}

}  // namespace codegen
}  // namespace mononn
