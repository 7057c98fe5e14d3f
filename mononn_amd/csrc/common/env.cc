#include "common/env.h"

#include <cstdlib>
#include <thread>

namespace mononn {
namespace env {

bool is_set(const char* name) { return std::getenv(name) != nullptr; }
bool is_true(const char* name) {
  const char* v = std::getenv(name);
  if (!v) return false;
  std::string s = v;
  return s == "True" || s == "true" || s == "1";
}
std::string get(const char* name, const std::string& dflt) {
  const char* v = std::getenv(name);
  return v ? std::string(v) : dflt;
}
int get_int(const char* name, int dflt) {
  const char* v = std::getenv(name);
  if (!v || !*v) return dflt;
  char* end = nullptr;
  long x = std::strtol(v, &end, 10);
  return (end && *end == 0) ? static_cast<int>(x) : dflt;
}
std::vector<std::string> split(const std::string& s, char sep) {
  std::vector<std::string> out;
  std::string cur;
  for (char c : s) {
    if (c == sep) {
      if (!cur.empty()) out.push_back(cur);
      cur.clear();
    } else {
      cur.push_back(c);
    }
  }
  if (!cur.empty()) out.push_back(cur);
  return out;
}
std::vector<std::string> disabled_passes() { return split(get("MONONN_OPTIMIZATION_DISABLED_PASS"), ','); }
std::vector<std::string> allow_list_override() { return split(get("MONONN_CODEGEN_ALLOW_LIST_OVERRIDE"), ','); }
int threadpool_size() {
  int n = get_int("TF_MONONN_THREADPOOL_SIZE", 0);
  if (n > 0) return n;
  unsigned hw = std::thread::hardware_concurrency();
  return hw ? static_cast<int>(hw) : 4;
}

}  // namespace env
}  // namespace mononn
