#include "module/mononn_module.h"

#include <sys/stat.h>

#include <unistd.h>

#include <atomic>
#include <cstring>
#include <fstream>
#include <sstream>

#include "common/env.h"
#include "common/status.h"
#include "hlo/hlo.h"
#include "runtime/rtc.h"
#include "runtime/static_scratch.h"

namespace mononn {
namespace module {

void make_dirs(const std::string& path) {
  std::string cur;
  for (size_t i = 0; i <= path.size(); ++i) {
    if (i == path.size() || path[i] == '/') {
      if (!cur.empty()) {
        if (::mkdir(cur.c_str(), 0755) != 0 && errno != EEXIST) MONONN_FAIL(kRuntimeError) << "cannot create directory " << cur;
      }
    }
    if (i < path.size()) cur.push_back(path[i]);
  }
}
void write_file(const std::string& path, const std::string& data) {
  std::ofstream f(path, std::ios::binary);
  MONONN_CHECK(f.good(), kRuntimeError) << "cannot write " << path;
  f.write(data.data(), static_cast<std::streamsize>(data.size()));
}
void write_file(const std::string& path, const std::vector<char>& data) {
  std::ofstream f(path, std::ios::binary);
  MONONN_CHECK(f.good(), kRuntimeError) << "cannot write " << path;
  f.write(data.data(), static_cast<std::streamsize>(data.size()));
}
bool read_file(const std::string& path, std::string* out) {
  std::ifstream f(path, std::ios::binary);
  if (!f.good()) return false;
  std::ostringstream ss;
  ss << f.rdbuf();
  *out = ss.str();
  return true;
}

MonoNNModule::MonoNNModule(const std::string& hlo_text, const std::string& spec_json, const std::string& kernel_name)
    : hlo_text_(hlo_text), kernel_name_(kernel_name) {
  if (!spec_json.empty()) {
    spec_ = spec::GraphSpecification::from_json(Json::parse(spec_json));
    spec_given_ = true;
  } else {
    spec_.runtime.grid_dim.x = spec_.device.sm_count;
    spec_.runtime.block_dim.x = 256;
  }
}

MonoNNModule::~MonoNNModule() = default;

void MonoNNModule::generate_code() {
  auto mod = hlo::parse_module(hlo_text_);
  module_name_ = mod->name;
  if (kernel_name_.empty()) {
    // kernel naming convention mononn_cluster_<id> (README.md:186)
    std::string shortn = "cluster_0";
    try {
      shortn = hlo::module_short_name(hlo::canonical_name(module_name_));
    } catch (const Error&) {
    }
    kernel_name_ = "mononn_" + shortn;
  }
  // MONONN_CODEGEN_ALLOW_LIST_OVERRIDE (mononn_module.cc:62-89)
  auto override_list = env::allow_list_override();
  if (!override_list.empty()) spec_.codegen_allow_list = override_list;
  program_ = graph::build_program(std::move(mod), codegen::build_options_from(spec_));
  hip_ = codegen::generate_program(*program_, spec_, kernel_name_);
  grid_ = hip_.grid;
  code_object_.clear();
}

void MonoNNModule::build_assembly() {
  MONONN_CHECK(program_ != nullptr, kInvalidArgument) << "build_assembly called before generate_code";
  try {
    auto res = runtime::compile_hip(hip_.files, "main.hip", spec_.device.cuda_arch);
    code_object_ = std::move(res.code_object);
    compile_log_ = res.log;
  } catch (const Error& e) {
    // Keep what failed for inspection, as the reference's tuner does before it aborts
    // (mononn_module_tuner.cc:261-285: sources and graph_spec.json under /tmp/mononn_codegen/<uuid>); here the
    // caller gets the error code and the directory instead of an abort.
    static std::atomic<unsigned> serial{0};
    std::string dir = "/tmp/mononn_codegen/" + std::to_string(static_cast<long long>(getpid())) + "_" + std::to_string(serial.fetch_add(1));
    std::string where;
    try {
      make_dirs(dir);
      for (auto& kv : hip_.files) write_file(dir + "/" + kv.first, kv.second);
      write_file(dir + "/graph_spec.json", tuning_spec_json());
      where = " [sources and graph_spec.json kept in " + dir + "]";
    } catch (const Error&) {
      // the dump is a convenience; the compile error is what the caller needs to see
    }
    throw Error(e.code(), std::string(e.what()) + where);
  }
}

std::string MonoNNModule::summary() const {
  std::ostringstream os;
  os << "module " << module_name_ << " kernel " << kernel_name_ << "\n";
  if (program_) os << program_->summary();
  os << "grid=" << hip_.grid << " block=" << hip_.block << " smem=" << hip_.smem << " barriers=" << hip_.num_barriers;
  if (hip_.num_regional_barriers > 0) os << " (" << hip_.num_regional_barriers << " of them over one XCD's workgroups)";
  os << "\n";
  for (size_t i = 0; i < hip_.param_bytes.size(); ++i) os << "Parameter " << i << ": " << hip_.param_bytes[i] << " bytes.\n";
  for (size_t i = 0; i < hip_.liveout_bytes.size(); ++i) os << "Liveout(output) buffer " << i << " size: " << hip_.liveout_bytes[i] << " bytes.\n";
  os << "Temporary buffer size: " << hip_.temp_bytes << " bytes.\n";
  return os.str();
}

// ---------------------------------------------------------------------------------------------
static const codegen::ConstantInfo* find_constant(const codegen::HipProgram& hp, const std::string& name) {
  std::string canon = hlo::canonical_name(name);
  for (auto& c : hp.constants)
    if (c.name == canon || c.hlo_name == name || c.symbol == name) return &c;
  return nullptr;
}

static std::vector<char> device_payload(const codegen::ConstantInfo& ci, const std::vector<char>& payload);
static std::vector<char> literal_payload(const codegen::ConstantInfo& ci);

void MonoNNModule::set_constant(const std::string& name, const void* host_data, size_t bytes) {
  MONONN_CHECK(program_ != nullptr, kInvalidArgument) << "set_constant called before generate_code";
  const codegen::ConstantInfo* ci = find_constant(hip_, name);
  MONONN_CHECK(ci != nullptr, kNotFound) << "the module has no constant named '" << name << "'";
  MONONN_CHECK(static_cast<int64_t>(bytes) == ci->bytes, kInvalidArgument)
      << "constant '" << name << "' needs " << ci->bytes << " bytes, got " << bytes;
  MONONN_CHECK(!ci->derived(), kInvalidArgument) << "constant '" << name << "' is built by the module from " << ci->sums_weight << " and " << ci->sums_vector;
  std::vector<char> payload(static_cast<const char*>(host_data), static_cast<const char*>(host_data) + bytes);
  if (!dev_.loaded()) {
    host_constants_[ci->name] = std::move(payload);
    return;
  }
  if (!is_fold_source(ci->name)) {
    upload_constant(*ci, payload);
    return;
  }
  // a source of a folded LayerNorm supplied after load: everything built from it is built and sent again
  fold_sources_[ci->name] = std::move(payload);
  for (auto& c : hip_.constants)
    if (c.name == ci->name || c.row_scale_by == ci->name || c.sums_weight == ci->name || c.sums_vector == ci->name) upload_resolved(c);
}

bool MonoNNModule::is_fold_source(const std::string& name) const {
  for (auto& c : hip_.constants)
    if (c.row_scale_by == name || c.sums_weight == name || c.sums_vector == name || (c.name == name && !c.row_scale_by.empty())) return true;
  return false;
}

const std::vector<char>* MonoNNModule::raw_payload(const std::string& name, std::vector<char>* scratch) const {
  auto f = fold_sources_.find(name);
  if (f != fold_sources_.end()) return &f->second;
  auto h = host_constants_.find(name);
  if (h != host_constants_.end()) return &h->second;
  for (auto& c : hip_.constants)
    if (c.name == name && !c.literal.empty()) {
      *scratch = literal_payload(c);
      return scratch;
    }
  return nullptr;
}

static float half_bits_to_float(uint16_t b) {
  _Float16 h;
  std::memcpy(&h, &b, 2);
  return static_cast<float>(h);
}

bool MonoNNModule::resolve_device_bytes(const codegen::ConstantInfo& ci, std::vector<char>* out) const {
  std::vector<char> s0, s1;
  if (ci.derived()) {
    // f32[N]: sum over k of vector[k] * weight[k, n], accumulated in double
    const std::vector<char>* w = raw_payload(ci.sums_weight, &s0);
    const std::vector<char>* v = raw_payload(ci.sums_vector, &s1);
    if (!w || !v) return false;
    const int64_t N = ci.dims[0], K = static_cast<int64_t>(v->size() / 2);
    MONONN_CHECK(static_cast<int64_t>(w->size()) == K * N * 2, kInternal) << "sources of " << ci.name << " do not match";
    const uint16_t* wp = reinterpret_cast<const uint16_t*>(w->data());
    const uint16_t* vp = reinterpret_cast<const uint16_t*>(v->data());
    // The sums that go with the scaled weights (vector = the gamma those weights were multiplied by) are taken over
    // the products as the MFMAs read them, rounded to half: the epilogue's x . W' - mean * colsum(W') is then
    // (x - mean) . W' exactly, whatever the row's mean.  (Over the unrounded products an error of mean * sum of the
    // rounding errors of a column stays behind, which grows with |mean| / sigma of the row.)
    bool of_scaled_weights = false;
    for (auto& other : hip_.constants) of_scaled_weights = of_scaled_weights || (other.name == ci.sums_weight && other.row_scale_by == ci.sums_vector);
    std::vector<double> acc(static_cast<size_t>(N), 0.0);
    for (int64_t k = 0; k < K; ++k) {
      const float vk = half_bits_to_float(vp[k]);
      for (int64_t n = 0; n < N; ++n) {
        const float w = half_bits_to_float(wp[k * N + n]);
        acc[n] += of_scaled_weights ? static_cast<double>(static_cast<float>(static_cast<_Float16>(w * vk))) : static_cast<double>(vk) * w;
      }
    }
    out->assign(static_cast<size_t>(N) * 4, 0);
    for (int64_t n = 0; n < N; ++n) {
      const float f = static_cast<float>(acc[n]);
      std::memcpy(out->data() + n * 4, &f, 4);
    }
    return true;
  }
  const std::vector<char>* raw = raw_payload(ci.name, &s0);
  if (!raw) return false;
  if (ci.row_scale_by.empty()) {
    *out = device_payload(ci, *raw);
    return true;
  }
  // weight[k, n] * vector[k], rounded to half once, then laid out like any other weight matrix
  const std::vector<char>* v = raw_payload(ci.row_scale_by, &s1);
  if (!v) return false;
  const int64_t K = ci.dims[0], N = ci.dims[1];
  MONONN_CHECK(static_cast<int64_t>(v->size()) == K * 2 && static_cast<int64_t>(raw->size()) == K * N * 2, kInternal) << "sources of " << ci.name << " do not match";
  std::vector<char> scaled(raw->size());
  const uint16_t* wp = reinterpret_cast<const uint16_t*>(raw->data());
  const uint16_t* vp = reinterpret_cast<const uint16_t*>(v->data());
  for (int64_t k = 0; k < K; ++k) {
    const float vk = half_bits_to_float(vp[k]);
    for (int64_t n = 0; n < N; ++n) {
      const _Float16 h = static_cast<_Float16>(vk * half_bits_to_float(wp[k * N + n]));
      std::memcpy(scaled.data() + (k * N + n) * 2, &h, 2);
    }
  }
  *out = device_payload(ci, scaled);
  return true;
}

void MonoNNModule::upload_resolved(const codegen::ConstantInfo& ci) {
  std::vector<char> bytes;
  if (!resolve_device_bytes(ci, &bytes)) return;
  size_t n = 0;
  void* dst = dev_.global(ci.symbol, &n);
  MONONN_CHECK(n >= bytes.size(), kRuntimeError) << "global " << ci.symbol << " is smaller than its constant in device layout";
  dev_.upload(dst, bytes.data(), bytes.size());
  uploaded_[ci.name] = true;
}

// bytes of the module global for a payload given in the HLO's layout
static std::vector<char> device_payload(const codegen::ConstantInfo& ci, const std::vector<char>& payload) {
  if (ci.transform != graph::ConstantTransform::kPackMfmaB) return payload;
  // [K,N] row-major -> [ceil(N/16)][K/32][64][8]: one MFMA B operand per contiguous KiB
  const int es = hlo::dtype_bytes(ci.dtype);
  const int64_t K = ci.dims[0], N = ci.dims[1];
  const int64_t nt_count = (N + 15) / 16, ksteps = K / 32;
  MONONN_CHECK(es == 2 && K % 32 == 0, kInternal) << "constant " << ci.hlo_name << " cannot be packed";
  std::vector<char> t(static_cast<size_t>(ci.device_bytes), 0);
  const uint16_t* src = reinterpret_cast<const uint16_t*>(payload.data());
  uint16_t* dstp = reinterpret_cast<uint16_t*>(t.data());
  for (int64_t nt = 0; nt < nt_count; ++nt)
    for (int64_t ks = 0; ks < ksteps; ++ks)
      for (int l = 0; l < 64; ++l) {
        const int64_t n = nt * 16 + (l & 15);
        if (n >= N) continue;
        const int64_t k0 = ks * 32 + (l >> 4) * 8;
        uint16_t* o = dstp + ((nt * ksteps + ks) * 64 + l) * 8;
        for (int j = 0; j < 8; ++j) o[j] = src[(k0 + j) * N + n];
      }
  return t;
}

void MonoNNModule::upload_constant(const codegen::ConstantInfo& ci, const std::vector<char>& payload) {
  size_t n = 0;
  void* dst = dev_.global(ci.symbol, &n);
  MONONN_CHECK(static_cast<int64_t>(n) >= ci.bytes, kRuntimeError) << "global " << ci.symbol << " is smaller than its constant";
  std::vector<char> t = device_payload(ci, payload);
  MONONN_CHECK(n >= t.size(), kRuntimeError) << "global " << ci.symbol << " is smaller than its constant in device layout";
  dev_.upload(dst, t.data(), t.size());
  uploaded_[ci.name] = true;
}

std::vector<std::string> MonoNNModule::missing_constants() const {
  std::vector<std::string> out;
  for (auto& c : hip_.constants)
    if (!c.derived() && c.literal.empty() && !uploaded_.count(c.name) && !host_constants_.count(c.name) && !fold_sources_.count(c.name)) out.push_back(c.hlo_name);
  return out;
}

static std::vector<char> literal_payload(const codegen::ConstantInfo& ci) {
  // parse "{ {1, 2}, {3, 4} }" into the constant's element type
  std::vector<char> out(static_cast<size_t>(ci.bytes));
  std::string tok;
  int64_t i = 0;
  const int es = hlo::dtype_bytes(ci.dtype);
  auto flush = [&]() {
    if (tok.empty()) return;
    MONONN_CHECK(i * es < ci.bytes, kParseError) << "constant " << ci.hlo_name << ": literal has too many elements";
    double d = 0;
    long long ll = 0;
    if (tok == "true") d = 1, ll = 1;
    else if (tok == "false") d = 0, ll = 0;
    else if (tok == "inf") d = __builtin_inf();
    else if (tok == "-inf") d = -__builtin_inf();
    else if (tok == "nan") d = __builtin_nan("");
    else {
      d = std::strtod(tok.c_str(), nullptr);
      ll = std::strtoll(tok.c_str(), nullptr, 10);
    }
    char* p = &out[static_cast<size_t>(i * es)];
    switch (ci.dtype) {
      case hlo::DType::kF16: { _Float16 v = static_cast<_Float16>(d); std::memcpy(p, &v, 2); break; }
      case hlo::DType::kBF16: {
        // round to nearest even on the upper 16 bits of the f32 pattern (NaN stays NaN)
        float f = static_cast<float>(d);
        uint32_t u;
        std::memcpy(&u, &f, 4);
        uint16_t h = f != f ? static_cast<uint16_t>((u >> 16) | 0x40) : static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
        std::memcpy(p, &h, 2);
        break;
      }
      case hlo::DType::kF32: { float v = static_cast<float>(d); std::memcpy(p, &v, 4); break; }
      case hlo::DType::kF64: std::memcpy(p, &d, 8); break;
      case hlo::DType::kPred: case hlo::DType::kS8: case hlo::DType::kU8: { int8_t v = static_cast<int8_t>(ll); std::memcpy(p, &v, 1); break; }
      case hlo::DType::kS16: case hlo::DType::kU16: { int16_t v = static_cast<int16_t>(ll); std::memcpy(p, &v, 2); break; }
      case hlo::DType::kS32: case hlo::DType::kU32: { int32_t v = static_cast<int32_t>(ll); std::memcpy(p, &v, 4); break; }
      default: { int64_t v = ll; std::memcpy(p, &v, 8); }
    }
    ++i;
    tok.clear();
  };
  for (char ch : ci.literal) {
    if (ch == '{' || ch == '}' || ch == ',' || isspace(static_cast<unsigned char>(ch))) flush();
    else tok.push_back(ch);
  }
  flush();
  MONONN_CHECK(i * es == ci.bytes, kParseError) << "constant " << ci.hlo_name << ": literal has " << i << " elements, expected " << ci.bytes / es;
  return out;
}

void MonoNNModule::load(int device) {
  MONONN_CHECK(has_code_object(), kInvalidArgument) << "load called before build_assembly";
  runtime::DeviceProperties props = runtime::query_device(device);
  MONONN_CHECK(props.arch == spec_.device.cuda_arch, kRuntimeError)
      << "code object was built for " << spec_.device.cuda_arch << " but device " << device << " is " << props.arch;
  // Known defect, fenced off: a process that used the cooperative launch entry point under rocprofv3 died with a
  // segmentation fault in an exit handler, after the profiler had written its output (five runs; no frame of this
  // library on the stack: the fault lies in the teardown of the runtime's cooperative queue after the tool has
  // finalised).  The ordinary launch under the same profiler exits cleanly.
  MONONN_CHECK(!(hip_.cooperative && runtime::profiler_tool_attached()), kRuntimeError)
      << "cooperative_launch is refused while a profiler tool library is attached to the process (the combination crashes at process exit); "
         "profile the ordinary launch: \"cooperative_launch\": false in the specification's mononn_hip section";
  dev_.load(device, code_object_, kernel_name_);
  dev_.set_dynamic_smem(hip_.smem);
  // The grid barrier needs every workgroup resident at once.  The reference's barrier would
  // deadlock on an over-sized grid; here it is rejected from the occupancy query before launch.
  int capacity = dev_.max_coresident_blocks(hip_.block, hip_.smem);
  if (capacity < hip_.grid) dev_.unload();   // a refused module must not be launchable
  MONONN_CHECK(capacity >= hip_.grid, kResourceExhausted)
      << "grid of " << hip_.grid << " workgroups x " << hip_.block << " threads exceeds the co-resident capacity of device " << device << " ("
      << capacity << ")";
  grid_ = hip_.grid;
  // once per device, with that device current: the address of the library's static temp arena on this GPU
  static_scratch_error_.clear();
  runtime::static_scratch_setup(device, &static_scratch_error_);
  size_t flag_bytes = 0;
  void* flags = dev_.global("mononn_barrier_flags", &flag_bytes);
  dev_.zero(flags, flag_bytes);
  size_t err_bytes = 0;
  void* err = dev_.global("mononn_barrier_error", &err_bytes);
  dev_.zero(err, err_bytes);
  uploaded_.clear();
  // the sources of folded LayerNorms stay on the host: scaled weights and column sums are built from them, now and
  // whenever one of them is supplied again
  for (auto& kv : host_constants_)
    if (is_fold_source(kv.first)) fold_sources_[kv.first] = kv.second;
  for (auto& ci : hip_.constants) {
    if (ci.derived() || !ci.row_scale_by.empty() || is_fold_source(ci.name)) {
      upload_resolved(ci);
      continue;
    }
    if (!ci.literal.empty()) {
      upload_constant(ci, literal_payload(ci));
      continue;
    }
    auto it = host_constants_.find(ci.name);
    if (it != host_constants_.end()) upload_constant(ci, it->second);
  }
  host_constants_.clear();
}

void MonoNNModule::launch_static_temp(void* const* device_ptrs, size_t n, void* stream) {
  // Same kernel, same launch; the temp arena is the library's own fixed device array instead of a caller's buffer.
  // Nothing here allocates device memory, and the argument tables live on the stack.
  MONONN_CHECK(dev_.loaded(), kInvalidArgument) << "launch called before load";
  MONONN_CHECK(n + 1 == num_args(), kInvalidArgument) << "kernel takes " << num_args() - 1 << " buffers (parameters, live-outs) besides the temp arena, got " << n;
  constexpr size_t kMaxArgs = 1024;   // the reference's own limit on kernel arguments (mononn_module_tuner.cc:113-127)
  MONONN_CHECK(n + 1 <= kMaxArgs, kInvalidArgument) << "more than " << kMaxArgs << " kernel arguments";
  MONONN_CHECK(hip_.temp_bytes <= static_cast<int64_t>(runtime::static_scratch_bytes()), kResourceExhausted)
      << "kernel " << kernel_name_ << " needs a temp arena of " << hip_.temp_bytes << " bytes, the library's static arena holds "
      << runtime::static_scratch_bytes() << ": use mononn_launch with a buffer of the caller";
  void* arena = runtime::static_scratch_address(dev_.device());
  MONONN_CHECK(arena != nullptr, kRuntimeError) << "the static arena has no address on device " << dev_.device() << ": " << static_scratch_error_;
  for (auto& c : hip_.constants)
    MONONN_CHECK(!c.literal.empty() || uploaded_.count(c.name) || host_constants_.count(c.name), kInvalidArgument)
        << "constant " << c.hlo_name << " has no payload yet";
  void* vals[kMaxArgs];
  void* args[kMaxArgs];
  for (size_t i = 0; i < n; ++i) {
    MONONN_CHECK(device_ptrs[i] != nullptr, kInvalidArgument) << "buffer " << i << " is null";
    MONONN_CHECK(reinterpret_cast<uintptr_t>(device_ptrs[i]) % 16 == 0, kInvalidArgument) << "buffer " << i << " is not 16-byte aligned";
    vals[i] = device_ptrs[i];
    args[i] = &vals[i];
  }
  vals[n] = arena;
  args[n] = &vals[n];
  dev_.launch(grid_, hip_.block, hip_.smem, args, stream, hip_.cooperative);
}

void MonoNNModule::launch(void* const* device_ptrs, size_t n, void* stream) {
  MONONN_CHECK(dev_.loaded(), kInvalidArgument) << "launch called before load";
  MONONN_CHECK(n == num_args(), kInvalidArgument) << "kernel takes " << num_args() << " buffers (parameters, live-outs, temp), got " << n;
  auto missing = missing_constants();
  MONONN_CHECK(missing.empty(), kInvalidArgument) << missing.size() << " constants have no payload yet, first: " << missing[0];
  std::vector<void*> vals(device_ptrs, device_ptrs + n);
  std::vector<void*> args(n);
  prepare_args(vals);
  for (size_t i = 0; i < n; ++i) args[i] = &vals[i];
  dev_.launch(grid_, hip_.block, hip_.smem, args.data(), stream, hip_.cooperative);
}

void MonoNNModule::synchronize(void* stream) {
  MONONN_CHECK(dev_.loaded(), kInvalidArgument) << "synchronize called before load";
  dev_.synchronize(stream);
  size_t err_bytes = 0;
  void* err = dev_.global("mononn_barrier_error", &err_bytes);
  unsigned word[4] = {0, 0, 0, 0};
  dev_.download(word, err, sizeof(word));
  if (word[0] == 0) return;
  // the workgroups left the kernel at different epochs: start over from a clean slate so that the module stays usable
  size_t flag_bytes = 0;
  void* flags = dev_.global("mononn_barrier_flags", &flag_bytes);
  dev_.zero(flags, flag_bytes);
  if (hip_.num_regional_barriers > 0) {
    size_t regional_bytes = 0;
    void* regional = dev_.global("mononn_regional_flags", &regional_bytes);
    dev_.zero(regional, regional_bytes);
  }
  dev_.zero(err, err_bytes);
  // error word of the device runtime: bit 31 = two workgroups with the same index modulo 8 found themselves on different XCDs (bits 24-26 and 20-22),
  // bit 30 = the wait that gave up belongs to the regional tier
  MONONN_CHECK((word[0] & 0x80000000u) == 0, kRuntimeError)
      << "kernel " << kernel_name_ << ": workgroup " << (word[0] & 0xfffffu) << " runs on XCD " << ((word[0] >> 24) & 7u) << ", a workgroup with the same index modulo 8 on XCD "
      << ((word[0] >> 20) & 7u) << " (regional synchronisation assumes that a grid of one workgroup per compute unit is dealt to the 8 XCDs round-robin); the outputs of this launch are invalid";
  MONONN_CHECK((word[0] & 0x40000000u) == 0, kRuntimeError)
      << "kernel " << kernel_name_ << ": a workgroup gave up waiting at regional barrier " << (word[0] & 0x3fffffffu) << " of " << hip_.num_regional_barriers << " after "
      << spec_.hip.barrier_timeout_ms << " ms (mononn_hip.barrier_timeout_ms): the grid of " << grid_
      << " workgroups was not resident as a whole (another kernel running on the device?); the outputs of this launch are invalid";
  MONONN_FAIL(kRuntimeError) << "kernel " << kernel_name_ << ": a workgroup gave up waiting at grid barrier " << word[0] << " of " << hip_.num_barriers
                             << " after " << spec_.hip.barrier_timeout_ms << " ms (mononn_hip.barrier_timeout_ms): the grid of " << grid_
                             << " workgroups was not resident as a whole (another kernel running on the device?); the outputs of this launch are invalid";
}

void* MonoNNModule::global_address(const std::string& symbol, size_t* bytes) const {
  MONONN_CHECK(dev_.loaded(), kInvalidArgument) << "module globals have addresses once the module is loaded";
  return dev_.global(symbol, bytes);
}

double MonoNNModule::read_stage_clock(std::vector<unsigned long long>* ticks, int* n_stages, int* grid) {
  MONONN_CHECK(dev_.loaded(), kInvalidArgument) << "read_stage_clock called before load";
  MONONN_CHECK(hip_.profiled, kInvalidArgument) << "kernel was built without mononn_hip.profile_stages";
  size_t bytes = 0;
  void* src = dev_.global("mononn_stage_clock", &bytes);
  ticks->resize(bytes / sizeof(unsigned long long));
  dev_.download(ticks->data(), src, bytes);
  *n_stages = hip_.num_stages;
  *grid = hip_.grid;
  return dev_.wall_clock_ticks_per_us();
}

void MonoNNModule::prepare_args(std::vector<void*>& vals) const {
  const size_t n = vals.size();
  for (size_t i = 0; i < n; ++i) {
    MONONN_CHECK(vals[i] != nullptr || (i + 1 == n && hip_.temp_bytes == 0), kInvalidArgument) << "buffer " << i << " is null";
    MONONN_CHECK(reinterpret_cast<uintptr_t>(vals[i]) % 16 == 0, kInvalidArgument) << "buffer " << i << " is not 16-byte aligned";
  }
}

float MonoNNModule::time_kernel(void* const* device_ptrs, size_t n, void* stream, int warmup, int iters, std::vector<float>* each) {
  MONONN_CHECK(dev_.loaded(), kInvalidArgument) << "time_kernel called before load";
  MONONN_CHECK(n == num_args(), kInvalidArgument) << "kernel takes " << num_args() << " buffers, got " << n;
  std::vector<void*> vals(device_ptrs, device_ptrs + n);
  std::vector<void*> args(n);
  prepare_args(vals);
  for (size_t i = 0; i < n; ++i) args[i] = &vals[i];
  // one checked launch first: a kernel whose barrier waits give up (a grid that is not resident as a whole) is
  // reported now, not after warmup + iters launches that each spin for the whole barrier budget
  dev_.launch(grid_, hip_.block, hip_.smem, args.data(), stream, hip_.cooperative);
  synchronize(stream);
  float ms = dev_.time_launches(grid_, hip_.block, hip_.smem, args.data(), stream, warmup, iters, each, hip_.cooperative);
  synchronize(stream);
  return ms;
}

// ---------------------------------------------------------------------------------------------
std::string MonoNNModule::cluster_dir(const std::string& dump_dir) const {
  std::string shortn = hlo::module_short_name(hlo::canonical_name(module_name_));
  return dump_dir + "/" + shortn;
}

std::string MonoNNModule::source_key() const {
  // FNV-1a over file names and contents in name order, then the extra compiler options of the environment
  unsigned long long h = 1469598103934665603ull;
  auto mix = [&](const std::string& t) {
    for (unsigned char c : t) {
      h ^= c;
      h *= 1099511628211ull;
    }
    h ^= 0xff;
    h *= 1099511628211ull;
  };
  for (auto& kv : hip_.files) {
    mix(kv.first);
    mix(kv.second);
  }
  mix(env::get("MONONN_HIPRTC_FLAGS"));
  char buf[40];
  std::snprintf(buf, sizeof buf, "fnv1a64:%016llx", h);
  return buf;
}

void MonoNNModule::dump_candidate(const std::string& dump_dir) const {
  std::string dir = cluster_dir(dump_dir);
  std::string ctx = spec_.context_string();
  make_dirs(dir + "/" + ctx + "_src");
  write_file(dir + "/" + ctx + ".json", tuning_spec_json());
  if (has_code_object()) write_file(dir + "/" + ctx + ".hsaco", code_object_);
  for (auto& kv : hip_.files) write_file(dir + "/" + ctx + "_src/" + kv.first, kv.second);
}

void MonoNNModule::dump_best(const std::string& dump_dir) const {
  std::string dir = cluster_dir(dump_dir);
  make_dirs(dir);
  write_file(dir + "/best_tuning_spec.json", tuning_spec_json());
  if (has_code_object()) {
    write_file(dir + "/best_tuning_spec.hsaco", code_object_);
    write_file(dir + "/best_tuning_spec.hsaco.key", source_key());
  }
  // source of the kernel and of the standalone driver (host_main.cpp), and what that driver feeds the module
  // globals with: literal constants always, elided ones when the host has supplied them and the module has not
  // been loaded yet (payloads are handed to the device at load time)
  make_dirs(dir + "/best_tuning_spec_src");
  for (auto& kv : hip_.files) write_file(dir + "/best_tuning_spec_src/" + kv.first, kv.second);
  bool any = false;
  for (auto& c : hip_.constants) {
    std::vector<char> bytes;
    if (!resolve_device_bytes(c, &bytes)) continue;
    if (!any) make_dirs(dir + "/constants");
    any = true;
    write_file(dir + "/constants/" + c.symbol + ".bin", bytes);
  }
}

}  // namespace module
}  // namespace mononn
