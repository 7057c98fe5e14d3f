// C ABI over the host compiler; see include/mononn_hip.h for the contract of every entry point.
#include "mononn_hip.h"

#include <cstring>
#include <memory>
#include <string>

#include "common/env.h"
#include "common/status.h"
#include "hlo/hlo.h"
#include "module/mononn_module.h"
#include "runtime/device_module.h"
#include "runtime/static_scratch.h"
#include "tuner/tuner.h"

using mononn::Error;
using mononn::module::MonoNNModule;

struct mononn_module {
  std::unique_ptr<MonoNNModule> impl;
  std::string spec_json, summary;   // storage for returned strings
  std::vector<std::string> names;
};

namespace {
thread_local std::string g_last_error;

template <class F>
int guarded(F&& f) {
  try {
    g_last_error.clear();
    f();
    return MONONN_OK;
  } catch (const Error& e) {
    g_last_error = e.what();
    return static_cast<int>(e.code());
  } catch (const std::exception& e) {
    g_last_error = std::string("internal error: ") + e.what();
    return MONONN_INTERNAL;
  } catch (...) {
    g_last_error = "unknown internal error";
    return MONONN_INTERNAL;
  }
}

void require(bool cond, const char* what) {
  if (!cond) throw Error(mononn::kInvalidArgument, what);
}
}  // namespace

extern "C" {

const char* mononn_last_error(void) { return g_last_error.c_str(); }
const char* mononn_version(void) { return "mononn-hip 0.1 (gfx950)"; }

int mononn_compile(const char* hlo_text, size_t hlo_len, const char* spec_json, const char* kernel_name, int build,
                   mononn_module** out) {
  return guarded([&] {
    require(hlo_text != nullptr && out != nullptr, "hlo_text and out must not be NULL");
    *out = nullptr;
    auto h = std::make_unique<mononn_module>();
    h->impl = std::make_unique<MonoNNModule>(std::string(hlo_text, hlo_len), spec_json ? std::string(spec_json) : std::string(),
                                             kernel_name ? std::string(kernel_name) : std::string());
    h->impl->generate_code();
    if (build) h->impl->build_assembly();
    *out = h.release();
  });
}

int mononn_tune(const char* hlo_text, size_t hlo_len, int device, const char* dump_dir, int budget, mononn_module** out) {
  return guarded([&] {
    require(hlo_text != nullptr && out != nullptr, "hlo_text and out must not be NULL");
    *out = nullptr;
    mononn::tuner::TuneParams p;
    p.hlo_text = std::string(hlo_text, hlo_len);
    p.device = device;
    p.dump_dir = dump_dir ? std::string(dump_dir) : mononn::env::get("TF_MONONN_DUMP_DIR");
    p.budget = budget;
    auto h = std::make_unique<mononn_module>();
    h->impl = mononn::tuner::MonoNNModuleTuner::tune(p);
    *out = h.release();
  });
}

int mononn_compile_from_spec_dir(const char* hlo_text, size_t hlo_len, const char* spec_dir, mononn_module** out) {
  return guarded([&] {
    require(hlo_text != nullptr && out != nullptr, "hlo_text and out must not be NULL");
    *out = nullptr;
    std::string dir = spec_dir ? std::string(spec_dir) : mononn::env::get("TF_MONONN_EXISTING_TUNING_SPEC_DIR");
    require(!dir.empty(), "no spec directory given and TF_MONONN_EXISTING_TUNING_SPEC_DIR is not set");
    std::string text(hlo_text, hlo_len);
    auto parsed = mononn::hlo::parse_module(text);
    std::string cdir = dir + "/" + mononn::hlo::module_short_name(mononn::hlo::canonical_name(parsed->name));
    std::string spec;
    if (!mononn::module::read_file(cdir + "/best_tuning_spec.json", &spec))
      throw Error(mononn::kNotFound, "cannot read " + cdir + "/best_tuning_spec.json");
    auto h = std::make_unique<mononn_module>();
    h->impl = std::make_unique<MonoNNModule>(text, spec, "");
    h->impl->generate_code();
    // The cached code object is used only when it was built from exactly the sources just generated (same HLO, same
    // specification, same device prelude, same compiler options): grid, LDS size, argument order, constant packing
    // and the number of barrier flags on the host side come from the fresh code, and a kernel that disagrees with
    // them computes garbage or never passes its first barrier.
    std::string co, key;
    if (!mononn::env::is_true("TF_MONONN_NO_USE_PTX_CACHE") && mononn::module::read_file(cdir + "/best_tuning_spec.hsaco", &co) && !co.empty() &&
        mononn::module::read_file(cdir + "/best_tuning_spec.hsaco.key", &key) && key == h->impl->source_key())
      h->impl->set_code_object(std::vector<char>(co.begin(), co.end()));
    else
      h->impl->build_assembly();
    *out = h.release();
  });
}

void mononn_module_destroy(mononn_module* m) { delete m; }

const char* mononn_module_kernel_name(const mononn_module* m) { return m ? m->impl->kernel_name().c_str() : ""; }

int mononn_module_spec_json(mononn_module* m, const char** text, size_t* len) {
  return guarded([&] {
    require(m && text, "NULL argument");
    m->spec_json = m->impl->tuning_spec_json();
    *text = m->spec_json.c_str();
    if (len) *len = m->spec_json.size();
  });
}

int mononn_module_source(const mononn_module* m, const char* file, const char** text, size_t* len) {
  return guarded([&] {
    require(m && file && text, "NULL argument");
    auto& files = m->impl->hip_program().files;
    auto it = files.find(file);
    if (it == files.end()) throw Error(mononn::kNotFound, std::string("no generated file named ") + file);
    *text = it->second.c_str();
    if (len) *len = it->second.size();
  });
}

int mononn_module_code_object(const mononn_module* m, const void** data, size_t* len) {
  return guarded([&] {
    require(m && data && len, "NULL argument");
    if (!m->impl->has_code_object()) throw Error(mononn::kNotFound, "module has not been built");
    *data = m->impl->code_object().data();
    *len = m->impl->code_object().size();
  });
}

int mononn_module_summary(mononn_module* m, const char** text, size_t* len) {
  return guarded([&] {
    require(m && text, "NULL argument");
    m->summary = m->impl->summary();
    *text = m->summary.c_str();
    if (len) *len = m->summary.size();
  });
}

int mononn_module_buffer_info(const mononn_module* m, int* n_params, const int64_t** param_bytes, int* n_liveouts,
                              const int64_t** liveout_bytes, int64_t* temp_bytes) {
  return guarded([&] {
    require(m != nullptr, "NULL module");
    auto& hp = m->impl->hip_program();
    if (n_params) *n_params = static_cast<int>(hp.param_bytes.size());
    if (param_bytes) *param_bytes = hp.param_bytes.data();
    if (n_liveouts) *n_liveouts = static_cast<int>(hp.liveout_bytes.size());
    if (liveout_bytes) *liveout_bytes = hp.liveout_bytes.data();
    if (temp_bytes) *temp_bytes = hp.temp_bytes;
  });
}

int mononn_module_owns_temp(const mononn_module* m) { return (m && m->impl->owns_temp()) ? 1 : 0; }

int mononn_module_launch_dims(const mononn_module* m, int* grid, int* block, int* smem, int* barriers) {
  return guarded([&] {
    require(m != nullptr, "NULL module");
    if (grid) *grid = m->impl->grid();
    if (block) *block = m->impl->block();
    if (smem) *smem = m->impl->smem();
    if (barriers) *barriers = m->impl->hip_program().num_barriers;
  });
}

int mononn_module_regional_barriers(const mononn_module* m, int* regional) {
  return guarded([&] {
    require(m != nullptr && regional != nullptr, "NULL argument");
    *regional = m->impl->hip_program().num_regional_barriers;
  });
}

int mononn_module_num_constants(const mononn_module* m) { return m ? static_cast<int>(m->impl->hip_program().constants.size()) : 0; }

int mononn_module_constant_info(const mononn_module* m, int index, const char** hlo_name, const char** role, int64_t* bytes,
                                int* needs_payload) {
  return guarded([&] {
    require(m != nullptr, "NULL module");
    auto& cs = m->impl->hip_program().constants;
    require(index >= 0 && index < static_cast<int>(cs.size()), "constant index out of range");
    if (hlo_name) *hlo_name = cs[index].hlo_name.c_str();
    if (role) *role = cs[index].role.c_str();
    if (bytes) *bytes = cs[index].bytes;
    if (needs_payload) *needs_payload = cs[index].literal.empty() && !cs[index].derived() ? 1 : 0;   // derived: built by the module from other payloads
  });
}

int mononn_module_set_constant(mononn_module* m, const char* name, const void* host_data, size_t bytes) {
  return guarded([&] {
    require(m && name && host_data, "NULL argument");
    m->impl->set_constant(name, host_data, bytes);
  });
}

int mononn_module_load(mononn_module* m, int device) {
  return guarded([&] {
    require(m != nullptr, "NULL module");
    m->impl->load(device);
  });
}

int mononn_launch(mononn_module* m, void* const* device_ptrs, size_t n_ptrs, void* stream) {
  return guarded([&] {
    require(m && device_ptrs, "NULL argument");
    m->impl->launch(device_ptrs, n_ptrs, stream);
  });
}

int mononn_launch_static_temp(mononn_module* m, void* const* device_ptrs, size_t n_ptrs, void* stream) {
  return guarded([&] {
    require(m && device_ptrs, "NULL argument");
    m->impl->launch_static_temp(device_ptrs, n_ptrs, stream);
  });
}

size_t mononn_static_temp_bytes(void) { return mononn::runtime::static_scratch_bytes(); }

int mononn_module_synchronize(mononn_module* m, void* stream) {
  return guarded([&] {
    require(m != nullptr, "NULL module");
    m->impl->synchronize(stream);
  });
}

int mononn_module_global(const mononn_module* m, const char* symbol, void** device_ptr, size_t* bytes) {
  return guarded([&] {
    require(m && symbol && device_ptr, "NULL argument");
    *device_ptr = m->impl->global_address(symbol, bytes);
  });
}

int mononn_time_kernel(mononn_module* m, void* const* device_ptrs, size_t n_ptrs, void* stream, int warmup, int iters,
                       float* avg_ms, float* each_ms) {
  return guarded([&] {
    require(m && device_ptrs && avg_ms, "NULL argument");
    require(iters > 0 && warmup >= 0, "iters must be positive");
    std::vector<float> each;
    *avg_ms = m->impl->time_kernel(device_ptrs, n_ptrs, stream, warmup, iters, each_ms ? &each : nullptr);
    if (each_ms) std::memcpy(each_ms, each.data(), each.size() * sizeof(float));
  });
}

int mononn_module_stage_clock(mononn_module* m, uint64_t* ticks, size_t capacity, int* n_stages, int* grid, double* ticks_per_us) {
  return guarded([&] {
    require(m && n_stages && grid && ticks_per_us, "NULL argument");
    std::vector<unsigned long long> t;
    *ticks_per_us = m->impl->read_stage_clock(&t, n_stages, grid);
    if (ticks)
      for (size_t i = 0; i < t.size() && i < capacity; ++i) ticks[i] = t[i];
  });
}

const char* mononn_module_stage_name(mononn_module* m, int stage) {
  if (!m) return "";
  auto& sn = m->impl->hip_program().stage_nodes;
  if (stage < 0 || stage >= static_cast<int>(sn.size())) return "";
  m->names.resize(sn.size());
  std::string& s = m->names[stage];
  s.clear();
  for (auto& n : sn[stage]) s += (s.empty() ? "" : "+") + n;
  return s.c_str();
}

int mononn_module_dump(mononn_module* m, const char* dump_dir) {
  return guarded([&] {
    require(m && dump_dir, "NULL argument");
    m->impl->dump_candidate(dump_dir);
    m->impl->dump_best(dump_dir);
  });
}

int mononn_device_count(void) { return mononn::runtime::device_count(); }

int mononn_device_info(int device, int* compute_units, int* wave_size, int* max_lds_per_block, char* arch, size_t arch_len) {
  return guarded([&] {
    auto p = mononn::runtime::query_device(device);
    if (compute_units) *compute_units = p.compute_units;
    if (wave_size) *wave_size = p.wave_size;
    if (max_lds_per_block) *max_lds_per_block = p.max_lds_per_block;
    if (arch && arch_len) {
      std::strncpy(arch, p.arch.c_str(), arch_len - 1);
      arch[arch_len - 1] = 0;
    }
  });
}

}  // extern "C"
