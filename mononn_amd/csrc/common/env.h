// Environment variables and process-wide knobs.  Names and truthiness follow the reference
// (EnvVars.md:1-24; truthy = True|true|1, mononn_engine/helpers/env_variable.cc:20-26;
// MONONN_OPTIMIZATION_DISABLED_PASS is a comma list, mononn_engine/config/config.cc:82-86).
#pragma once
#include <string>
#include <vector>

namespace mononn {
namespace env {

bool is_set(const char* name);
bool is_true(const char* name);
std::string get(const char* name, const std::string& dflt = "");
int get_int(const char* name, int dflt);
std::vector<std::string> split(const std::string& s, char sep);
std::vector<std::string> disabled_passes();            // MONONN_OPTIMIZATION_DISABLED_PASS
std::vector<std::string> allow_list_override();        // MONONN_CODEGEN_ALLOW_LIST_OVERRIDE
int threadpool_size();                                 // TF_MONONN_THREADPOOL_SIZE or hardware threads

}  // namespace env
}  // namespace mononn
