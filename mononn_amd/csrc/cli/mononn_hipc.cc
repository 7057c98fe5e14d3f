// mononn_hipc: command line front end of the host compiler.
//   mononn_hipc <module.hlo> [--spec spec.json | --spec-dir DIR] [--dump DIR] [--no-build] [--print-source]
// Compiles one HLO module into its monolithic kernel and prints the buffer summary the reference
// logs (README.md:189-196).  With --dump it writes the TF_MONONN_DUMP_DIR tree.
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>

#include "mononn_hip.h"

static bool slurp(const char* path, std::string* out) {
  std::ifstream f(path, std::ios::binary);
  if (!f.good()) return false;
  std::ostringstream ss;
  ss << f.rdbuf();
  *out = ss.str();
  return true;
}

int main(int argc, char** argv) {
  const char *hlo_path = nullptr, *spec_path = nullptr, *spec_dir = nullptr, *dump_dir = nullptr;
  bool build = true, print_source = false;
  for (int i = 1; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--spec") && i + 1 < argc) spec_path = argv[++i];
    else if (!std::strcmp(argv[i], "--spec-dir") && i + 1 < argc) spec_dir = argv[++i];
    else if (!std::strcmp(argv[i], "--dump") && i + 1 < argc) dump_dir = argv[++i];
    else if (!std::strcmp(argv[i], "--no-build")) build = false;
    else if (!std::strcmp(argv[i], "--print-source")) print_source = true;
    else if (argv[i][0] != '-') hlo_path = argv[i];
    else {
      std::fprintf(stderr, "unknown option %s\n", argv[i]);
      return 2;
    }
  }
  if (!hlo_path) {
    std::fprintf(stderr, "usage: mononn_hipc <module.hlo> [--spec spec.json | --spec-dir DIR] [--dump DIR] [--no-build] [--print-source]\n");
    return 2;
  }
  std::string hlo, spec;
  if (!slurp(hlo_path, &hlo)) {
    std::fprintf(stderr, "cannot read %s\n", hlo_path);
    return 1;
  }
  if (spec_path && !slurp(spec_path, &spec)) {
    std::fprintf(stderr, "cannot read %s\n", spec_path);
    return 1;
  }
  mononn_module* m = nullptr;
  int rc = spec_dir ? mononn_compile_from_spec_dir(hlo.data(), hlo.size(), spec_dir, &m)
                    : mononn_compile(hlo.data(), hlo.size(), spec_path ? spec.c_str() : nullptr, nullptr, build ? 1 : 0, &m);
  if (rc != MONONN_OK) {
    std::fprintf(stderr, "error %d: %s\n", rc, mononn_last_error());
    return 1;
  }
  const char* text = nullptr;
  size_t len = 0;
  if (mononn_module_summary(m, &text, &len) == MONONN_OK) std::fwrite(text, 1, len, stdout);
  if (print_source && mononn_module_source(m, "main.hip", &text, &len) == MONONN_OK) std::fwrite(text, 1, len, stdout);
  if (dump_dir && mononn_module_dump(m, dump_dir) != MONONN_OK) {
    std::fprintf(stderr, "dump failed: %s\n", mononn_last_error());
    mononn_module_destroy(m);
    return 1;
  }
  mononn_module_destroy(m);
  return 0;
}
