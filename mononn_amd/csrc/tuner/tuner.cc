#include "tuner/tuner.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <map>
#include <mutex>
#include <set>
#include <sstream>
#include <thread>

#include "codegen/cluster_codegen.h"
#include "common/env.h"
#include "common/status.h"
#include "runtime/device_module.h"
#include "runtime/rtc.h"

namespace mononn {
namespace tuner {

using module::MonoNNModule;
using spec::GraphSpecification;

namespace {

// Worker pool for candidate compilation (reference: CompilationThreadpool, size from
// TF_MONONN_THREADPOOL_SIZE or the hardware concurrency, compilation_threadpool.cc:35-39).
template <class F>
void parallel_for(size_t n, int threads, F&& f) {
  std::atomic<size_t> next{0};
  std::vector<std::thread> pool;
  threads = std::max(1, std::min<int>(threads, static_cast<int>(n)));
  for (int t = 0; t < threads; ++t)
    pool.emplace_back([&] {
      for (;;) {
        size_t i = next.fetch_add(1);
        if (i >= n) return;
        f(i);
      }
    });
  for (auto& th : pool) th.join();
}

struct DeviceBuffers {
  int device;
  std::vector<void*> ptrs;   // params, live-outs, temp (may be null)
  size_t temp_capacity = 0;
  // candidates differ in temp size (split-K partial sums, slot re-use): the arena grows to the largest
  void ensure_temp(size_t bytes);
  ~DeviceBuffers() {
    for (auto* p : ptrs)
      if (p) (void)hipFree(p);
  }
};

void alloc_zero(void** p, size_t bytes) {
  bytes = std::max<size_t>(bytes, 256);
  hipError_t e = hipMalloc(p, bytes);
  if (e != hipSuccess) MONONN_FAIL(kRuntimeError) << "hipMalloc(" << bytes << "): " << hipGetErrorString(e);
  e = hipMemset(*p, 0, bytes);
  if (e != hipSuccess) MONONN_FAIL(kRuntimeError) << "hipMemset: " << hipGetErrorString(e);
}

void DeviceBuffers::ensure_temp(size_t bytes) {
  if (bytes <= temp_capacity) return;
  MONONN_CHECK(!ptrs.empty(), kInternal) << "tuner buffers not allocated";
  if (ptrs.back()) (void)hipFree(ptrs.back());
  ptrs.back() = nullptr;
  temp_capacity = 0;
  alloc_zero(&ptrs.back(), bytes);
  temp_capacity = std::max<size_t>(bytes, 256);
}

// Every wave arrangement x per-wave fragment tile that the code generator accepts for this problem
// (reference: all CUTLASS tiles that fit, tuning_space_generator.cc:139-307).
std::vector<codegen::GemmTuning> gemm_candidates(const graph::GemmDesc& g, int waves, int budget) {
  std::vector<codegen::GemmTuning> out;
  if (!codegen::gemm_uses_mfma(g)) return out;
  const int ksteps = static_cast<int>((g.K + 31) / 32);
  for (int wk = 1; wk <= waves; wk *= 2) {
    if (wk > ksteps) break;
    for (int wm = 1; wm * wk <= waves; wm *= 2) {
      int wn = waves / (wk * wm);
      if (wm * wn * wk != waves) continue;
      for (int tm : {1, 2, 3, 4, 6, 8})
        for (int tn : {1, 2, 3, 4, 6, 8}) {
          // 16 accumulator fragments per wave at most.  Larger blocks (the generator takes up to 64) win the isolated
          // stage clocks on large problems and lose in the whole kernel, where they slow down the stages around them:
          // with them among the candidates the tuned GPT-2 / ViT kernels came out 19% / 8% slower than without.
          if (tm * tn > 16) continue;
          codegen::GemmTuning t;
          t.wm = wm;
          t.wn = wn;
          t.wk = wk;
          t.bm = wm * tm * 16;
          t.bn = wn * tn * 16;
          // tiles much larger than the problem only add idle lanes
          if (t.bm >= 2 * g.M + 16 && tm * wm > 1) continue;
          if (t.bn >= 2 * g.N + 16 && tn * wn > 1) continue;
          // LDS for the cross-wave reduction
          if (wk > 1 && waves * tm * tn * 1024 > 64 * 1024) continue;
          out.push_back(t);
        }
    }
  }
  // Every shape only on request (MONONN_TUNER_ALL_TILES=1 at full budget): a full-budget run over ViT-B/16 (1576
  // rows), whose only kernels that no reduced-budget run had built are those of the shapes left out below, ended in
  // a GPU memory fault whose cause has not been shown; BERT-base and GPT-2 went through with all of them.
  if (budget >= 1 || !env::is_true("MONONN_TUNER_ALL_TILES")) {
    // keep the shapes with a balanced per-wave tile
    std::vector<codegen::GemmTuning> kept;
    for (auto& t : out) {
      int tm = t.bm / t.wm / 16, tn = t.bn / t.wn / 16;
      if (tm * tn >= 2 && tm * tn <= 8 && (budget < 2 || (tm <= 2 && tn <= 2))) kept.push_back(t);
    }
    out = kept;
  }
  // large problems: operand tiles staged through LDS once per workgroup (the reference's tiles with shared-memory
  // stages, tile_description.cc:84-258); four waves as 2 x 2, per-wave blocks of up to 128 x 128
  if (waves == 4 && g.K % 32 == 0 && g.K >= 128 && g.split_k <= 1 && g.M >= 128 && g.N >= 128 && g.a_k_contig && (g.b_k_contig || g.b_packed)) {
    struct Shape { int bm, bn, bk; };
    for (const Shape& sh : {Shape{256, 256, 32}, Shape{192, 256, 32}, Shape{256, 192, 32}, Shape{256, 128, 64}, Shape{128, 256, 64}, Shape{192, 128, 64},
                            Shape{128, 192, 64}, Shape{128, 128, 64}}) {
      if (sh.bm > g.M || sh.bn > g.N) continue;
      if (budget >= 2 && sh.bm * sh.bn < 192 * 128) continue;
      codegen::GemmTuning t;
      t.bm = sh.bm;
      t.bn = sh.bn;
      t.wm = 2;
      t.wn = 2;
      t.wk = 1;
      t.stages = 2;
      t.bk = sh.bk;
      out.push_back(t);
    }
  }
  return out;
}

// barrier time budget of the kernels the tuner times (candidates of a class, whole-kernel candidates); the module it
// hands back keeps the specification's own
constexpr int kTrialBarrierTimeoutMs = 1000;

struct ClassInfo {
  std::string function;                 // de-duplicated device function name under the default spec
  std::vector<std::string> nodes;       // node names sharing it
  std::string kind;                     // gemm | cluster_reduce | cluster_elewise
  const graph::Node* sample = nullptr;
};

struct Trial {
  std::string label;
  GraphSpecification spec;
  std::unique_ptr<MonoNNModule> mod;
  std::string error;
  double us = -1;        // mean time of one profiled stage
  double total_us = -1;  // all profiled stages of one launch together
};

void apply_gemm(GraphSpecification& s, const std::string& node, const codegen::GemmTuning& t, int64_t K) {
  spec::GemmSpec& g = s.gemm_spec_list[node];
  g.tb_m = t.bm;
  g.tb_n = t.bn;
  g.wave_m = t.wm;
  g.wave_n = t.wn;
  g.wave_k = t.wk;
  g.warp_m = t.bm / t.wm;
  g.warp_n = t.bn / t.wn;
  g.warp_k = static_cast<int>(K / t.wk);
  g.stages = t.stages;
  g.tb_k = t.bk;
}

double time_module(MonoNNModule& m, int device, DeviceBuffers& bufs, int warmup, int iters) {
  m.load(device);
  std::vector<void*> ptrs = bufs.ptrs;
  float ms = m.time_kernel(ptrs.data(), ptrs.size(), nullptr, warmup, iters);
  return ms * 1000.0;
}

}  // namespace

std::unique_ptr<MonoNNModule> MonoNNModuleTuner::tune(const TuneParams& params) {
  runtime::DeviceProperties props = runtime::query_device(params.device);
  MONONN_CHECK(props.wave_size == 64, kRuntimeError) << "device " << params.device << " does not run 64-wide wavefronts";
  const int threads = env::threadpool_size();
  const int budget = std::max(params.budget, env::is_true("MONONN_FASTEST_TUNING") ? 2 : (env::is_true("MONONN_FASTER_TUNING") ? 1 : 0));
  std::ostringstream log, report;
  log << "Tuning result for each thread grid setting:\n";

  // launch contexts: workgroups per CU x threads per workgroup
  // (reference: {1,2,3} blocks per SM x {128,256} threads, tuning_space_generator.cc:65-66)
  struct Ctx {
    int per_cu, block;
  };
  std::vector<Ctx> contexts = {{1, 256}, {1, 512}};
  if (budget == 0) {
    // the reference's space also holds more workgroups per SM and smaller workgroups (tuning_space_generator.cc:65-66)
    contexts.push_back({2, 256});
    contexts.push_back({3, 256});
    contexts.push_back({1, 128});
  }
  if (budget >= 2) contexts = {{1, 256}};
  // MONONN_TUNER_LAUNCH_CONTEXTS="1x256,2x256": workgroups per CU x threads, instead of the list above (large models:
  // one context of a full search takes minutes)
  {
    const std::string only = env::get("MONONN_TUNER_LAUNCH_CONTEXTS", "");
    std::vector<Ctx> chosen;
    size_t st = 0;
    while (!only.empty() && st <= only.size()) {
      size_t e = only.find(',', st);
      const std::string item = only.substr(st, e == std::string::npos ? std::string::npos : e - st);
      const size_t x = item.find('x');
      const int per_cu = x == std::string::npos ? 0 : std::atoi(item.substr(0, x).c_str());
      const int block = x == std::string::npos ? 0 : std::atoi(item.substr(x + 1).c_str());
      MONONN_CHECK(per_cu >= 1 && per_cu <= 4 && block >= 64 && block <= 1024 && block % 64 == 0, kInvalidArgument)
          << "MONONN_TUNER_LAUNCH_CONTEXTS: '" << item << "' is not <workgroups per CU>x<threads per workgroup>";
      chosen.push_back({per_cu, block});
      if (e == std::string::npos) break;
      st = e + 1;
    }
    if (!chosen.empty()) contexts = chosen;
  }

  std::unique_ptr<MonoNNModule> best;
  double best_us = -1;
  DeviceBuffers bufs{params.device, {}};

  for (auto& cx : contexts) {
    GraphSpecification base;
    base.device.sm_count = props.compute_units;
    base.device.cuda_arch = props.arch;
    base.device.max_configurable_smem_size = std::max(props.max_lds_per_block, 65536);
    base.runtime.grid_dim.x = props.compute_units * cx.per_cu;
    base.runtime.block_dim.x = cx.block;
    if (env::is_true("MONONN_TUNER_GEMM_PROLOGUE")) base.hip.gemm_prologue_fusion = true;
    if (env::is_true("MONONN_TUNER_LAYER_NORM_FOLDING")) base.hip.gemm_prologue_fusion = base.hip.layer_norm_folding = true;
    const std::string ctx_str = base.context_string();

    // default module of this context: classes of identical node functions
    auto def_holder = std::make_unique<MonoNNModule>(params.hlo_text, base.to_json().dump(0), params.kernel_name);
    def_holder->generate_code();
    // MONONN_TUNER_SEED_SPEC_DIR: a dump directory of an earlier tuning run of the same module.  Its entries join
    // the candidates that are tried in the whole kernel, so a new run ends no worse than the one it starts from
    // (the stage clocks are noisy, and the order in which classes are decided matters).
    std::unique_ptr<GraphSpecification> seed;
    {
      const char* sd = std::getenv("MONONN_TUNER_SEED_SPEC_DIR");
      if (sd && *sd) {
        try {
          std::string text;
          MONONN_CHECK(module::read_file(def_holder->cluster_dir(sd) + "/best_tuning_spec.json", &text), kInvalidArgument) << "no best_tuning_spec.json";
          auto sp = std::make_unique<GraphSpecification>(GraphSpecification::from_json(Json::parse(text)));
          if (sp->context_string() == ctx_str) seed = std::move(sp);
        } catch (const Error& e) {
          log << "  seed specification in " << sd << " not usable: " << e.what() << "\n";
        }
      }
    }
    // the stage-fusion decisions of the seed are where the search starts (its entries name the nodes of that graph)
    if (seed && (seed->hip.gemm_prologue_fusion != base.hip.gemm_prologue_fusion || seed->hip.layer_norm_folding != base.hip.layer_norm_folding ||
                 seed->hip.attention_out_proj_fusion != base.hip.attention_out_proj_fusion || seed->hip.regional_synchronization != base.hip.regional_synchronization)) {
      base.hip.gemm_prologue_fusion = base.hip.gemm_prologue_fusion || seed->hip.gemm_prologue_fusion;
      base.hip.layer_norm_folding = base.hip.layer_norm_folding || seed->hip.layer_norm_folding;
      base.hip.attention_out_proj_fusion = seed->hip.attention_out_proj_fusion;
      base.hip.regional_synchronization = seed->hip.regional_synchronization;
      def_holder = std::make_unique<MonoNNModule>(params.hlo_text, base.to_json().dump(0), params.kernel_name);
      def_holder->generate_code();
      log << "  [" << ctx_str << "] stage-fusion decisions taken from the seed specification\n";
    }
    // MONONN_TUNER_KEEP_SEED_SPLIT_K=<F>: the seed's k splits by at least F are in place from the start.  With
    // LayerNorm folding a split and a fold exclude each other at one LayerNorm (the row program that adds the partial
    // sums up stays a stage), and the split-K search below only compares a GEMM and its consumer, so which of the
    // two a LayerNorm gets is decided here: deep splits (BERT's second feed-forward GEMM, K 3072 by 8) are worth more
    // than the stage they keep, shallow ones (K 768 by 2) less.
    if (seed) {
      const int keep_from = std::atoi(env::get("MONONN_TUNER_KEEP_SEED_SPLIT_K", "0").c_str());
      int kept = 0;
      if (keep_from >= 2)
        for (auto& kv : seed->gemm_spec_list)
          if (kv.second.split_k >= keep_from) {
            base.gemm_spec_list[kv.first] = kv.second;
            ++kept;
          }
      if (kept) {
        try {
          auto again = std::make_unique<MonoNNModule>(params.hlo_text, base.to_json().dump(0), params.kernel_name);
          again->generate_code();
          def_holder = std::move(again);
          log << "  [" << ctx_str << "] " << kept << " k splits of the seed specification kept from the start\n";
        } catch (const Error& e) {
          log << "  [" << ctx_str << "] the seed's k splits do not apply here: " << e.what() << "\n";
          base.gemm_spec_list.clear();
        }
      }
    }
    MonoNNModule& def = *def_holder;
    GraphSpecification filled = def.tuning_spec();
    if (bufs.ptrs.empty()) {
      hipError_t e = hipSetDevice(params.device);
      if (e != hipSuccess) MONONN_FAIL(kRuntimeError) << "hipSetDevice: " << hipGetErrorString(e);
      auto& hp = def.hip_program();
      for (auto b : hp.param_bytes) {
        bufs.ptrs.push_back(nullptr);
        alloc_zero(&bufs.ptrs.back(), static_cast<size_t>(b));
      }
      for (auto b : hp.liveout_bytes) {
        bufs.ptrs.push_back(nullptr);
        alloc_zero(&bufs.ptrs.back(), static_cast<size_t>(b));
      }
      bufs.ptrs.push_back(nullptr);
      bufs.ensure_temp(static_cast<size_t>(hp.temp_bytes));
    }
    // Node classes: nodes that came out as the same device function.  GEMM classes that solve the same
    // problem in the same stages (the Q, K and V projections of a layer) are tuned as one class, because
    // their tiles share the workgroups of that stage.
    std::map<std::string, ClassInfo> by_fn;
    std::map<std::string, std::vector<int>> stages_of_fn;
    for (auto& r : def.hip_program().nodes) {
      ClassInfo& c = by_fn[r.function];
      c.function = r.function;
      c.kind = r.kind;
      c.nodes.push_back(r.name);
      stages_of_fn[r.function].push_back(r.stage);
    }
    for (auto& n : def.program().nodes)
      for (auto& kv : by_fn)
        if (!kv.second.sample && kv.second.nodes[0] == n.name) kv.second.sample = &n;
    std::map<std::string, ClassInfo> classes;
    for (auto& kv : by_fn) {
      std::string key = kv.first;
      if (kv.second.kind == "gemm" && kv.second.sample) {
        const graph::GemmDesc& g = kv.second.sample->gemm;
        std::ostringstream k;
        k << "gemm|" << g.batch << "x" << g.M << "x" << g.N << "x" << g.K << "|" << (kv.second.sample->prologue.empty() ? 0 : 1) << "|";
        std::set<int> distinct(stages_of_fn[kv.first].begin(), stages_of_fn[kv.first].end());
        for (int st : distinct) k << st << ",";
        key = k.str();
      }
      ClassInfo& c = classes[key];
      if (c.nodes.empty()) {
        c = kv.second;
        c.function = key;
      } else {
        c.nodes.insert(c.nodes.end(), kv.second.nodes.begin(), kv.second.nodes.end());
      }
    }

    // ---- candidates of every class ------------------------------------------------------------
    std::vector<Trial> trials;
    std::map<std::string, std::vector<size_t>> trials_of_class;
    for (auto& kv : classes) {
      ClassInfo& c = kv.second;
      auto add = [&](const std::string& label, GraphSpecification s) {
        s.codegen_allow_list = c.nodes;
        s.hip.profile_stages = true;
        // a candidate's stages take microseconds: one whose grid turns out not to be resident must not spin at its
        // first barrier for the full budget of a production launch
        s.hip.barrier_timeout_ms = std::min(s.hip.barrier_timeout_ms, kTrialBarrierTimeoutMs);
        Trial t;
        t.label = label;
        t.spec = std::move(s);
        trials_of_class[c.function].push_back(trials.size());
        trials.push_back(std::move(t));
      };
      add("default", filled);
      // MONONN_TUNER_ONLY_FUSION_DECISIONS (with a seed specification): the seed's tiles stand, only the stage-fusion
      // decisions are searched (large models, whose class search takes many minutes); with
      // MONONN_TUNER_ROW_PROGRAMS_TOO the row-program classes are searched as well (few candidates each)
      if (seed && env::is_true("MONONN_TUNER_ONLY_FUSION_DECISIONS") && !(c.kind == "cluster_reduce" && env::is_true("MONONN_TUNER_ROW_PROGRAMS_TOO"))) continue;
      if (c.kind == "gemm") {
        for (auto& t : gemm_candidates(c.sample->gemm, cx.block / 64, budget)) {
          GraphSpecification s = filled;
          for (auto& n : c.nodes) apply_gemm(s, n, t, c.sample->gemm.K);
          char lbl[96];
          if (t.stages >= 2) std::snprintf(lbl, sizeof lbl, "tile%dx%dx%d_lds_waves%dx%d", t.bm, t.bn, t.bk, t.wm, t.wn);
          else std::snprintf(lbl, sizeof lbl, "tile%dx%d_waves%dx%dx%d", t.bm, t.bn, t.wm, t.wn, t.wk);
          add(lbl, s);
        }
      } else if (c.kind == "attention") {
        // key waves per row block: 1 (no exchange through LDS, a wave owns whole rows) .. all waves
        // and the blocks of 16 query rows a wave takes in turn with the keys and values it loaded once, as long as
        // the units still cover the grid
        for (int kw = 1; kw <= cx.block / 64; kw *= 2) {
          if (c.sample->gemm.N % 32 == 0 && c.sample->gemm.N % (32 * kw) != 0) continue;   // a ragged key count is rounded up per wave
          for (int rb : {1, 2, 3, 4, 6, 8}) {
            const int wave_m = cx.block / 64 / kw;
            const int64_t rows = 16 * wave_m * rb;
            const int64_t units = c.sample->gemm.batch * ((c.sample->gemm.M + rows - 1) / rows);
            if (rb > 1 && (c.sample->gemm3_index != 0 || 2 * units < base.runtime.grid_dim.x || rows >= c.sample->gemm.M + 16 * wave_m)) continue;
            GraphSpecification s = filled;
            for (auto& n : c.nodes) {
              spec::GemmSpec& g = s.gemm_spec_list[n];
              g.wave_k = kw;
              g.wave_m = wave_m;
              g.tb_m = static_cast<int>(rows);
              g.warp_n = static_cast<int>(c.sample->gemm.N / kw);
            }
            add("key_waves" + std::to_string(kw) + (rb > 1 ? "_rows" + std::to_string(rows) : ""), s);
          }
        }
      } else if (c.kind == "cluster_reduce") {
        for (int tier : {1, 2})
          for (int ilp : {1, 2, 4, 8}) {
            if (budget >= 2 && ilp > 2) continue;
            GraphSpecification s = filled;
            for (auto& n : c.nodes) {
              s.cluster_reduce_spec[n].locality_tier = tier;
              s.cluster_reduce_spec[n].ilp_factor = ilp;
              s.cluster_reduce_spec[n].reduce_implementation = 0;
            }
            add("tier" + std::to_string(tier) + "_ilp" + std::to_string(ilp), s);
          }
        {
          // a wave on 8 rows at once (rows of whole 16-byte runs; other rows fall back to one row per wave)
          GraphSpecification s = filled;
          for (auto& n : c.nodes) {
            s.cluster_reduce_spec[n].locality_tier = 1;
            s.cluster_reduce_spec[n].ilp_factor = 1;
            s.cluster_reduce_spec[n].reduce_implementation = 1;
          }
          add("tier1_rows8", s);
          // 4 and 2 rows per wave: the same scheme for row counts that leave most waves idle at 8 rows each
          for (int impl : {2, 3}) {
            for (auto& n : c.nodes) s.cluster_reduce_spec[n].reduce_implementation = impl;
            add(impl == 2 ? "tier1_rows4" : "tier1_rows2", s);
          }
        }
      } else if (c.kind == "cluster_elewise") {
        for (int ilp : {2, 4, 8}) {
          GraphSpecification s = filled;
          for (auto& n : c.nodes) s.cluster_elewise_spec[n].ilp_factor = ilp;
          add("ilp" + std::to_string(ilp), s);
        }
      }
    }
    // ---- code generation in the pool; one hipRTC compilation and one module load per class -----------
    const bool progress = env::is_true("TF_MONONN_ENABLE_WORKER_THRAED_LOGGING") || env::is_true("MONONN_TUNER_VERBOSE");
    std::atomic<size_t> generated{0};
    parallel_for(trials.size(), threads, [&](size_t i) {
      Trial& t = trials[i];
      try {
        t.mod = std::make_unique<MonoNNModule>(params.hlo_text, t.spec.to_json().dump(0), "mononn_tune_" + std::to_string(i));
        t.mod->generate_code();
      } catch (const Error& e) {
        t.error = e.what();
        t.mod.reset();
      }
      const size_t done = ++generated;
      if (progress && (done % 16 == 0 || done == trials.size()))
        std::fprintf(stderr, "[mononn tuner] %s code generated for %zu of %zu candidates\n", ctx_str.c_str(), done, trials.size());
    });
    GraphSpecification stitched = filled;
    // runners-up of every class by the isolated stage clocks, for the whole-kernel refinement below
    struct Alternative {
      std::string label;
      double us;
      GraphSpecification spec;
    };
    std::map<std::string, std::vector<Alternative>> runners_up;   // class function -> candidates after the best
    const bool verbose = env::is_true("TF_MONONN_ENABLE_WORKER_THRAED_LOGGING") || env::is_true("MONONN_TUNER_VERBOSE");
    // Compiles the candidates `live` as one translation unit (shared preamble, one namespace per candidate),
    // loads it once and times the profiled stages of every candidate.
    auto measure = [&](const std::vector<size_t>& live) {
      std::map<std::string, std::string> files;
      std::string tu = trials[live[0]].mod->hip_program().preamble;
      std::set<std::string> decls;
      // candidates that differ in their number of profiled stages (a split adds one) declare stamp arrays of different
      // lengths: the translation unit gets the longest
      const std::string clock_decl = "__device__ unsigned long long mononn_stage_clock[";
      size_t clock_len = 0;
      for (size_t i : live)
        for (auto& d : trials[i].mod->hip_program().global_decls) {
          if (d.compare(0, clock_decl.size(), clock_decl) == 0) {
            clock_len = std::max<size_t>(clock_len, std::strtoull(d.c_str() + clock_decl.size(), nullptr, 10));
            continue;
          }
          if (decls.insert(d).second) tu += d + "\n";
        }
      if (clock_len > 0) tu += clock_decl + std::to_string(clock_len) + "];\n";
      for (size_t i : live) tu += "namespace cand_" + std::to_string(i) + " {\n" + trials[i].mod->hip_program().body + "}\n";
      files["headers.h"] = trials[live[0]].mod->hip_program().files.at("headers.h");
      files["main.hip"] = tu;
      auto res = runtime::compile_hip(files, "main.hip", props.arch);
      runtime::DeviceModule dm;
      dm.load(params.device, res.code_object, trials[live[0]].mod->kernel_name());
      size_t fb = 0, eb = 0;
      void* const flags = dm.global("mononn_barrier_flags", &fb);
      void* const error_word = dm.global("mononn_barrier_error", &eb);
      dm.zero(flags, fb);
      // A barrier wait that gave up leaves the workgroups at different epochs: the candidate is out, and the flags
      // start from zero again so that the candidates behind it (same translation unit, same flags) are not held up
      auto gave_up = [&]() {
        unsigned word[4] = {0, 0, 0, 0};
        dm.download(word, error_word, sizeof(word));
        if (word[0] == 0) return false;
        dm.zero(flags, fb);
        dm.zero(error_word, eb);
        try {
          size_t rb = 0;
          void* regional = dm.global("mononn_regional_flags", &rb);   // only in kernels with a regional tier
          dm.zero(regional, rb);
        } catch (const Error&) {
        }
        return true;
      };
      for (size_t i : live) {
        Trial& t = trials[i];
        const codegen::HipProgram& hp = t.mod->hip_program();
        try {
          dm.use_kernel(t.mod->kernel_name());
          dm.set_dynamic_smem(hp.smem);
          if (dm.max_coresident_blocks(hp.block, hp.smem) < hp.grid) {
            t.error = "grid exceeds the co-resident capacity";
            continue;
          }
          bufs.ensure_temp(static_cast<size_t>(hp.temp_bytes));
          std::vector<void*> vals = bufs.ptrs, args(vals.size());
          for (size_t a = 0; a < vals.size(); ++a) args[a] = &vals[a];
          const int warm = 3, iters = budget >= 1 ? 8 : 20;   // launches are short: the compilation of the candidates dominates
          size_t cb = 0;
          void* clk = dm.global("mononn_stage_clock", &cb);
          std::vector<unsigned long long> ticks(cb / sizeof(unsigned long long));
          const double tpu = dm.wall_clock_ticks_per_us();
          double total = 0;
          int count = 0;
          for (int it = 0; it < warm + iters; ++it) {
            dm.launch(hp.grid, hp.block, hp.smem, args.data(), nullptr);
            if (it == 0 && gave_up()) MONONN_FAIL(kRuntimeError) << "a grid-barrier wait gave up (the grid was not resident as a whole)";
            if (it < warm) continue;
            dm.download(ticks.data(), clk, cb);
            // A stage is charged from the moment the last workgroup finished the stage before it (the first stage:
            // from its first workgroup's entry) to the moment its own last workgroup finishes: the barrier in front
            // of it is included, and so is whatever of its operand traffic a candidate hides behind that barrier.
            // Workgroups without a unit in a stage leave zero stamps.
            unsigned long long prev_hi = 0;
            for (int st = 0; st < hp.num_stages; ++st) {
              unsigned long long lo = ~0ull, hi = 0;
              for (int w = 0; w < hp.grid; ++w) {
                const unsigned long long in = ticks[(static_cast<size_t>(st) * hp.grid + w) * 2], out = ticks[(static_cast<size_t>(st) * hp.grid + w) * 2 + 1];
                if (in == 0 || out == 0) continue;
                lo = std::min(lo, in);
                hi = std::max(hi, out);
              }
              if (hi == 0) continue;
              const unsigned long long from = st == 0 || prev_hi == 0 ? lo : prev_hi;
              total += static_cast<double>(hi - from) / tpu;
              prev_hi = hi;
              ++count;
            }
          }
          t.us = count ? total / count : -1;
          t.total_us = count ? total / iters : -1;
          if (gave_up()) MONONN_FAIL(kRuntimeError) << "a grid-barrier wait gave up (the grid was not resident as a whole)";
        } catch (const Error& e) {
          t.error = e.what();
          t.us = -1;
        }
      }
    };
    for (auto& kv : classes) {
      ClassInfo& c = kv.second;
      std::vector<size_t> live;
      for (size_t i : trials_of_class[c.function])
        if (trials[i].mod) live.push_back(i);
      if (live.empty()) continue;
      double best_class = -1;
      size_t best_i = live[0];
      try {
        measure(live);
        for (size_t i : live)
          if (trials[i].us > 0 && (best_class < 0 || trials[i].us < best_class)) {
            best_class = trials[i].us;
            best_i = i;
          }
      } catch (const Error& e) {
        log << "  [" << ctx_str << "] class of " << c.nodes[0] << " failed: " << e.what() << "\n";
        if (verbose) std::fprintf(stderr, "[mononn tuner] %s class of %s failed: %.300s\n", ctx_str.c_str(), c.nodes[0].c_str(), e.what());
      }
      for (size_t i : trials_of_class[c.function]) trials[i].mod.reset();
      if (verbose) std::fprintf(stderr, "[mononn tuner] %s %s x%zu: %zu candidates, best %.2f us\n", ctx_str.c_str(), c.kind.c_str(), c.nodes.size(), live.size(), best_class);
      if (best_class < 0) continue;
      if (seed) {
        bool all = true;
        for (auto& n : c.nodes) {
          if (c.kind == "gemm" || c.kind == "attention") all = all && seed->gemm_spec_list.count(n) && seed->gemm_spec_list.at(n).split_k <= 1;
          else if (c.kind == "cluster_reduce") all = all && seed->cluster_reduce_spec.count(n);
          else if (c.kind == "cluster_elewise") all = all && seed->cluster_elewise_spec.count(n);
        }
        if (all) runners_up[c.function].push_back({"seed", -1.0, *seed});
      }
      if (c.nodes.size() >= 2) {
        std::vector<size_t> order;
        for (size_t i : live)
          if (i != best_i && trials[i].us > 0 && trials[i].us < 1.25 * best_class) order.push_back(i);
        std::sort(order.begin(), order.end(), [&](size_t a, size_t b) { return trials[a].us < trials[b].us; });
        const size_t keep = budget == 0 ? 6 : budget == 1 ? 2 : 1;
        for (size_t k = 0; k < order.size() && k < keep; ++k) runners_up[c.function].push_back({trials[order[k]].label, trials[order[k]].us, trials[order[k]].spec});
      }
      // The default of a class that lost on the stage clocks always gets its turn in the whole kernel, however far
      // behind it was: an isolated stage finds its operands in the caches of the launch before, the real one does
      // not (BERT-large: wave-per-row LayerNorm wins 2:1 in isolation and costs 14% of the whole kernel).
      if (trials[best_i].label != "default") {
        bool listed = false;
        for (auto& alt : runners_up[c.function]) listed = listed || alt.label == "default";
        for (size_t i : live)
          if (!listed && trials[i].label == "default" && trials[i].us > 0) {
            runners_up[c.function].push_back({"default", trials[i].us, trials[i].spec});
            break;
          }
        if (runners_up[c.function].empty()) runners_up.erase(c.function);
      }
      const GraphSpecification& w = trials[best_i].spec;
      for (auto& n : c.nodes) {
        if (c.kind == "gemm" || c.kind == "attention") stitched.gemm_spec_list[n] = w.gemm_spec_list.at(n);
        else if (c.kind == "cluster_reduce") stitched.cluster_reduce_spec[n] = w.cluster_reduce_spec.at(n);
        else if (c.kind == "cluster_elewise") stitched.cluster_elewise_spec[n] = w.cluster_elewise_spec.at(n);
        report << ctx_str << "," << n << "," << best_class << "\n";
      }
      log << "  [" << ctx_str << "] " << c.kind << " x" << c.nodes.size() << " (" << c.nodes[0] << "): best " << trials[best_i].label << " "
          << best_class << " us per stage;";
      for (size_t i : trials_of_class[c.function])
        if (trials[i].us > 0) log << " " << trials[i].label << "=" << trials[i].us;
      log << "\n";
    }

    // ---- split-K: GEMM classes with a long k range and few output tiles ---------------------------------
    // A split GEMM writes fp32 partial sums and its fused epilogue moves into the consuming cluster, so the
    // graph changes shape: the candidates are compared on GEMM stage + consumer stage together, against the
    // same pair of stages of the unsplit graph.
    double stitched_us = -1;
    std::string why_not;   // why the last whole kernel was not built or timed; written beside its -1 in the log
    auto whole_kernel_us = [&](GraphSpecification s) -> double {
      s.codegen_allow_list.clear();
      s.hip.profile_stages = false;
      s.hip.barrier_timeout_ms = std::min(s.hip.barrier_timeout_ms, kTrialBarrierTimeoutMs);
      why_not.clear();
      try {
        MonoNNModule m(params.hlo_text, s.to_json().dump(0), params.kernel_name);
        m.generate_code();
        m.build_assembly();
        bufs.ensure_temp(static_cast<size_t>(m.hip_program().temp_bytes));
        const double us = time_module(m, params.device, bufs, 5, 40);
        if (verbose) std::fprintf(stderr, "[mononn tuner] %s   a whole kernel built and timed: %.2f us\n", ctx_str.c_str(), us);
        return us;
      } catch (const Error& e) {
        if (verbose) std::fprintf(stderr, "[mononn tuner] %s   a whole kernel was not built: %.200s\n", ctx_str.c_str(), e.what());
        why_not = e.what();
        for (char& ch : why_not)
          if (ch == '\n') ch = ' ';
        if (why_not.size() > 160) why_not = why_not.substr(0, 160) + "...";
        return -1;
      }
    };
    // " <label>=<us>", with the reason in brackets behind a candidate that produced no kernel
    auto timed = [&](const std::string& label, double us) {
      char buf[64];
      std::snprintf(buf, sizeof buf, "=%.2f", us);
      return " " + label + buf + (us < 0 && !why_not.empty() ? " [" + why_not + "]" : std::string());
    };
    // ---- whole-kernel refinement ------------------------------------------------------------------------
    // A class is timed above in a kernel that holds nothing but its own stages, where every workgroup reaches
    // the barrier at the same moment and the caches hold only that class's operands.  In the real kernel the
    // stage follows a different one, part of its operand traffic hides behind the barrier wait, and the
    // ranking of close candidates can change: the runners-up of every class are tried in the whole kernel and
    // the fastest whole kernel wins.
    // The seed as a whole: its classes were tuned against each other, which a class-by-class comparison cannot see.
    if (seed) {
      GraphSpecification whole = filled;
      whole.gemm_spec_list = seed->gemm_spec_list;
      whole.cluster_reduce_spec = seed->cluster_reduce_spec;
      whole.cluster_elewise_spec = seed->cluster_elewise_spec;
      if (stitched_us < 0) stitched_us = whole_kernel_us(stitched);
      const double seed_us = whole_kernel_us(whole);
      log << "  [" << ctx_str << "] whole kernel: " << stitched_us << " us with the best of every class by the stage clocks, " << seed_us
          << " us with the seed specification; the search goes on from the faster one\n";
      if (verbose) std::fprintf(stderr, "[mononn tuner] %s whole kernel %.2f us tuned, %.2f us seed\n", ctx_str.c_str(), stitched_us, seed_us);
      if (seed_us > 0 && (stitched_us < 0 || seed_us < 0.999 * stitched_us)) {
        // the winners by the stage clocks get their turn against the seed, class by class
        for (auto& kv : classes) runners_up[kv.second.function].insert(runners_up[kv.second.function].begin(), {"best_by_stage_clocks", -1.0, stitched});
        stitched = std::move(whole);
        stitched_us = seed_us;
      }
    }
    // A launch context that starts out well behind the best one so far is not worth the whole-kernel builds.
    bool promising = true;
    if (!env::is_true("MONONN_TUNER_NO_REFINEMENT")) {
      if (stitched_us < 0) stitched_us = whole_kernel_us(stitched);
      promising = best_us < 0 || (stitched_us > 0 && stitched_us < 1.08 * best_us);
      if (!promising) log << "  [" << ctx_str << "] " << stitched_us << " us before refinement, best context so far " << best_us << " us: not refined\n";
    }
    // several sweeps: what one sweep changes in one class can change the ranking in another
    auto refine = [&](int max_sweeps) {
    for (int sweep = 0, changed = 1; sweep < max_sweeps && changed && promising && !runners_up.empty() && !env::is_true("MONONN_TUNER_NO_REFINEMENT"); ++sweep) {
      changed = 0;
      for (auto& kv : classes) {
        ClassInfo& c = kv.second;
        auto ru = runners_up.find(c.function);
        if (ru == runners_up.end() || stitched_us < 0) continue;
        std::string line;
        double best_alt_us = -1;
        const Alternative* best_alt = nullptr;
        for (auto& alt : ru->second) {
          GraphSpecification s = stitched;
          for (auto& n : c.nodes) {
            if (c.kind == "gemm" || c.kind == "attention") s.gemm_spec_list[n] = alt.spec.gemm_spec_list.at(n);
            else if (c.kind == "cluster_reduce") s.cluster_reduce_spec[n] = alt.spec.cluster_reduce_spec.at(n);
            else if (c.kind == "cluster_elewise") s.cluster_elewise_spec[n] = alt.spec.cluster_elewise_spec.at(n);
          }
          const double us = whole_kernel_us(s);
          line += timed(alt.label, us);
          if (us > 0 && (best_alt_us < 0 || us < best_alt_us)) {
            best_alt_us = us;
            best_alt = &alt;
          }
        }
        log << "  [" << ctx_str << "] whole kernel with runners-up of " << c.kind << " x" << c.nodes.size() << " (" << c.nodes[0] << "): now " << stitched_us
            << " us;" << line << "\n";
        if (verbose) std::fprintf(stderr, "[mononn tuner] %s refinement %s (%s): now %.2f us;%s\n", ctx_str.c_str(), c.kind.c_str(), c.nodes[0].c_str(), stitched_us, line.c_str());
        if (best_alt && best_alt_us < 0.997 * stitched_us) {
          const Alternative replaced{"previous", stitched_us, stitched};   // stays a candidate of the next sweep
          const Alternative adopted = *best_alt;
          best_alt = &adopted;
          for (auto& alt : ru->second)
            if (alt.label == adopted.label) alt = replaced;
          for (auto& n : c.nodes) {
            if (c.kind == "gemm" || c.kind == "attention") stitched.gemm_spec_list[n] = best_alt->spec.gemm_spec_list.at(n);
            else if (c.kind == "cluster_reduce") stitched.cluster_reduce_spec[n] = best_alt->spec.cluster_reduce_spec.at(n);
            else if (c.kind == "cluster_elewise") stitched.cluster_elewise_spec[n] = best_alt->spec.cluster_elewise_spec.at(n);
          }
          stitched_us = best_alt_us;
          changed = 1;
        }
      }
    }
    };
    refine(budget == 0 ? 3 : 1);
    bool split_adopted = false;
    if (promising && !env::is_true("MONONN_TUNER_NO_SPLIT_K")) {
      for (auto& kv : classes) {
        ClassInfo& c = kv.second;
        if (c.kind != "gemm" || !c.sample || !c.sample->prologue.empty()) continue;
        const graph::GemmDesc g = c.sample->gemm;
        if (!codegen::gemm_uses_mfma(g) || g.batch != 1 || g.K < 512) continue;
        // GEMM instruction behind every node of the class (node names differ once an epilogue is fused)
        std::vector<std::string> instrs;
        for (auto& n : def.program().nodes)
          if (n.kind == graph::NodeKind::kGemm && std::find(c.nodes.begin(), c.nodes.end(), n.name) != c.nodes.end())
            instrs.push_back(n.members[0]->name);
        if (instrs.size() != c.nodes.size()) continue;
        // node names in use before this class is touched
        auto names_and_consumers = [&](const graph::Program& p, const std::set<std::string>& gemm_instrs, std::vector<std::string>* allow,
                                       std::vector<std::string>* consumers) {
          std::set<const hlo::Instr*> outs;
          for (auto& n : p.nodes)
            if (n.kind == graph::NodeKind::kGemm && gemm_instrs.count(n.members[0]->name)) {
              allow->push_back(n.name);
              for (auto* o : n.outputs) outs.insert(o);
            }
          for (auto& n : p.nodes) {
            if (std::find(allow->begin(), allow->end(), n.name) != allow->end()) continue;
            bool reads = false;
            for (auto* in : n.inputs) reads = reads || outs.count(in);
            if (reads) consumers->push_back(n.name);
          }
        };
        auto drop_unknown = [&](GraphSpecification& s, const graph::Program& p) {
          std::set<std::string> known;
          for (auto& n : p.nodes) known.insert(n.name);
          for (auto it = s.gemm_spec_list.begin(); it != s.gemm_spec_list.end();) it = known.count(it->first) ? std::next(it) : s.gemm_spec_list.erase(it);
          for (auto it = s.cluster_reduce_spec.begin(); it != s.cluster_reduce_spec.end();)
            it = known.count(it->first) ? std::next(it) : s.cluster_reduce_spec.erase(it);
          for (auto it = s.cluster_elewise_spec.begin(); it != s.cluster_elewise_spec.end();)
            it = known.count(it->first) ? std::next(it) : s.cluster_elewise_spec.erase(it);
        };
        const std::set<std::string> instr_set(instrs.begin(), instrs.end());
        std::vector<Trial> cand;
        // unsplit pair of stages
        std::vector<std::string> base_consumers;
        int base_barriers = 0;
        {
          GraphSpecification s = stitched;
          s.hip.profile_stages = true;
          s.hip.barrier_timeout_ms = std::min(s.hip.barrier_timeout_ms, kTrialBarrierTimeoutMs);
          s.codegen_allow_list.clear();
          MonoNNModule probe(params.hlo_text, s.to_json().dump(0), "mononn_probe");
          try {
            probe.generate_code();
          } catch (const Error&) {
            continue;
          }
          std::vector<std::string> allow;
          names_and_consumers(probe.program(), instr_set, &allow, &base_consumers);
          if (base_consumers.empty()) continue;
          base_barriers = probe.hip_program().num_barriers;
          // the consuming clusters must be row programs (they get the partial sums for free in registers)
          allow.insert(allow.end(), base_consumers.begin(), base_consumers.end());
          s.codegen_allow_list = allow;
          Trial t;
          t.label = "unsplit";
          t.spec = s;
          cand.push_back(std::move(t));
        }
        // the tuned row-program knobs of the unsplit consumer carry over to the split one
        spec::ClusterReduceSpec consumer_knobs;
        bool have_knobs = false;
        for (auto& n : base_consumers) {
          auto it = stitched.cluster_reduce_spec.find(n);
          if (it != stitched.cluster_reduce_spec.end()) {
            consumer_knobs = it->second;
            have_knobs = true;
            break;
          }
        }
        for (int S : {2, 4, 8}) {
          if (g.K % (32 * S) != 0 || g.K / S < 256) continue;
          GraphSpecification s0 = stitched;
          s0.hip.profile_stages = true;
          s0.hip.barrier_timeout_ms = std::min(s0.hip.barrier_timeout_ms, kTrialBarrierTimeoutMs);
          s0.codegen_allow_list.clear();
          for (auto& n : c.nodes) s0.gemm_spec_list.erase(n);
          for (auto& n : base_consumers) {
            s0.cluster_reduce_spec.erase(n);
            s0.cluster_elewise_spec.erase(n);
          }
          graph::GemmDesc part = g;
          part.K = g.K / S;
          codegen::LaunchShape shape;
          shape.block_size = cx.block;
          for (auto& in : instrs) {
            apply_gemm(s0, in, codegen::default_gemm_tuning(part, shape, props.compute_units), part.K);
            s0.gemm_spec_list[in].split_k = S;
          }
          // first pass without an allow list: learns whether the split is legal here and the new node names
          std::vector<std::string> allow, consumers;
          try {
            GraphSpecification probe_spec = s0;
            MonoNNModule probe(params.hlo_text, probe_spec.to_json().dump(0), "mononn_probe");
            probe.generate_code();
            // an epilogue that cannot move into the consumer becomes a stage of its own: not a candidate
            if (probe.hip_program().num_barriers > base_barriers) continue;
            names_and_consumers(probe.program(), instr_set, &allow, &consumers);
          } catch (const Error& e) {
            if (verbose) std::fprintf(stderr, "[mononn tuner] split_k=%d not applicable to %s: %s\n", S, instrs[0].c_str(), e.what());
            continue;
          }
          std::vector<std::string> both = allow;
          both.insert(both.end(), consumers.begin(), consumers.end());
          std::vector<codegen::GemmTuning> tiles = gemm_candidates(part, cx.block / 64, std::max(budget, 1));
          size_t seed_tile = tiles.size();
          if (seed) {
            auto it = seed->gemm_spec_list.find(instrs[0]);
            if (it != seed->gemm_spec_list.end() && it->second.split_k == S) {
              codegen::GemmTuning st;
              st.bm = it->second.tb_m;
              st.bn = it->second.tb_n;
              st.wm = it->second.wave_m;
              st.wn = it->second.wave_n;
              st.wk = it->second.wave_k;
              tiles.push_back(st);
            }
          }
          for (size_t ti = 0; ti < tiles.size(); ++ti) {
            const codegen::GemmTuning& t = tiles[ti];
            GraphSpecification s = s0;
            for (auto& in : instrs) {
              apply_gemm(s, in, t, part.K);
              s.gemm_spec_list[in].split_k = S;
            }
            if (have_knobs)
              for (auto& n : consumers) {
                spec::ClusterReduceSpec r = consumer_knobs;
                r.name = n;
                s.cluster_reduce_spec[n] = r;
              }
            s.codegen_allow_list = both;
            Trial tr;
            char lbl[112];
            std::snprintf(lbl, sizeof lbl, "split%d_%stile%dx%d_waves%dx%dx%d", S, ti == seed_tile ? "seed_" : "", t.bm, t.bn, t.wm, t.wn, t.wk);
            if (ti == seed_tile)
              for (auto& n : consumers) {
                auto it = seed->cluster_reduce_spec.find(n);
                if (it != seed->cluster_reduce_spec.end()) s.cluster_reduce_spec[n] = it->second;
              }
            tr.label = lbl;
            tr.spec = std::move(s);
            cand.push_back(std::move(tr));
          }
        }
        if (cand.size() < 2) continue;
        const size_t first = trials.size();
        for (auto& t : cand) trials.push_back(std::move(t));
        parallel_for(cand.size(), threads, [&](size_t j) {
          Trial& t = trials[first + j];
          try {
            t.mod = std::make_unique<MonoNNModule>(params.hlo_text, t.spec.to_json().dump(0), "mononn_tune_" + std::to_string(first + j));
            t.mod->generate_code();
          } catch (const Error& e) {
            t.error = e.what();
            t.mod.reset();
          }
        });
        std::vector<size_t> live;
        for (size_t i = first; i < trials.size(); ++i)
          if (trials[i].mod) live.push_back(i);
        if (live.empty() || live[0] != first) {
          for (size_t i = first; i < trials.size(); ++i) trials[i].mod.reset();
          continue;
        }
        size_t best_i = first;
        try {
          measure(live);
          for (size_t i : live)
            if (trials[i].total_us > 0 && trials[first].total_us > 0 && trials[i].total_us < trials[best_i].total_us) best_i = i;
        } catch (const Error& e) {
          log << "  [" << ctx_str << "] split-K candidates of " << instrs[0] << " failed: " << e.what() << "\n";
        }
        const double per = static_cast<double>(instrs.size());
        log << "  [" << ctx_str << "] split-K x" << instrs.size() << " (" << instrs[0] << "), GEMM + consumer stages per GEMM: best " << trials[best_i].label
            << " " << trials[best_i].total_us / per << " us;";
        for (size_t i : live)
          if (trials[i].total_us > 0) log << " " << trials[i].label << "=" << trials[i].total_us / per;
        log << "\n";
        if (verbose)
          std::fprintf(stderr, "[mononn tuner] %s split-K x%zu (%s): %zu candidates, unsplit %.2f us, best %s %.2f us\n", ctx_str.c_str(), instrs.size(),
                       instrs[0].c_str(), live.size(), trials[first].total_us / per, trials[best_i].label.c_str(), trials[best_i].total_us / per);
        // The stage clocks leave out barrier skew and cache effects between stages, so the best few candidates
        // are built into the whole kernel and one is adopted only when that kernel is faster than without.
        // Candidates: per split factor the best one or two by the stage clocks, as long as they are not far behind
        // the unsplit pair of stages (what a split saves is partly hidden in the clocks of the isolated stages).
        std::vector<size_t> order;
        {
          std::map<std::string, std::vector<size_t>> by_factor;   // "split4" -> trials
          for (size_t i : live)
            if (i != first && trials[i].total_us > 0 && trials[first].total_us > 0 && trials[i].total_us < 1.2 * trials[first].total_us)
              by_factor[trials[i].label.substr(0, trials[i].label.find('_'))].push_back(i);
          for (auto& bf : by_factor) {
            std::sort(bf.second.begin(), bf.second.end(), [&](size_t a, size_t b) { return trials[a].total_us < trials[b].total_us; });
            for (size_t k = 0; k < bf.second.size() && k < (budget == 0 ? 3u : 1u); ++k) order.push_back(bf.second[k]);
          }
          for (size_t i : live)
            if (i != first && trials[i].total_us > 0 && trials[i].label.find("_seed_") != std::string::npos &&
                std::find(order.begin(), order.end(), i) == order.end())
              order.push_back(i);
        }
        if (!order.empty()) {
          if (stitched_us < 0) stitched_us = whole_kernel_us(stitched);
          double best_with = -1;
          GraphSpecification best_spec;
          size_t best_split = first;
          log << "    whole kernel: " << stitched_us << " us without;";
          for (size_t i : order) {
            GraphSpecification adopted = trials[i].spec;
            drop_unknown(adopted, trials[i].mod->program());
            const double with_split = whole_kernel_us(adopted);
            log << timed(trials[i].label, with_split);
            if (with_split > 0 && (best_with < 0 || with_split < best_with)) {
              best_with = with_split;
              best_spec = std::move(adopted);
              best_split = i;
            }
          }
          log << "\n";
          if (verbose) std::fprintf(stderr, "[mononn tuner] %s   whole kernel %.2f us without, %.2f us with %s\n", ctx_str.c_str(), stitched_us, best_with, trials[best_split].label.c_str());
          if (best_with > 0 && stitched_us > 0 && best_with < 0.995 * stitched_us) {
            for (auto& in : instrs) report << ctx_str << "," << in << "," << trials[best_split].total_us / per << "\n";
            stitched = std::move(best_spec);
            stitched_us = best_with;
            split_adopted = true;
            // the row programs that now add up the partial sums do more loading than before: their knobs again
            std::vector<std::string> allow, consumers;
            names_and_consumers(trials[best_split].mod->program(), instr_set, &allow, &consumers);
            std::string line;
            GraphSpecification best_knobs;
            double best_knobs_us = -1;
            for (int tier : {1, 2})
              for (int ilp : {1, 2, 4}) {
                GraphSpecification s = stitched;
                bool changed = false;
                for (auto& n : consumers) {
                  auto it = s.cluster_reduce_spec.find(n);
                  if (it == s.cluster_reduce_spec.end()) continue;
                  changed = changed || it->second.locality_tier != tier || it->second.ilp_factor != ilp;
                  it->second.locality_tier = tier;
                  it->second.ilp_factor = ilp;
                }
                if (!changed) continue;
                const double us = whole_kernel_us(s);
                char buf[64];
                std::snprintf(buf, sizeof buf, "tier%d_ilp%d", tier, ilp);
                line += timed(buf, us);
                if (us > 0 && (best_knobs_us < 0 || us < best_knobs_us)) {
                  best_knobs_us = us;
                  best_knobs = std::move(s);
                }
              }
            log << "    consumers of the split GEMM, whole kernel: now " << stitched_us << " us;" << line << "\n";
            if (best_knobs_us > 0 && best_knobs_us < 0.997 * stitched_us) {
              stitched = std::move(best_knobs);
              stitched_us = best_knobs_us;
            }
          }
        }
        for (size_t i = first; i < trials.size(); ++i) trials[i].mod.reset();
      }
    }
    // the classes that kept their node names once more, now against the split GEMMs and their consumers
    if (split_adopted) refine(budget == 0 ? 2 : 1);
    // ---- stages made of several GEMM calls: a tile per call ---------------------------------------------
    // The GEMMs of one stage (the Q, K and V projections) have been tuned as one class, with one tile.  Their calls
    // occupy consecutive ranges of workgroups, and the workgroups differ: those that had a unit in the stage before
    // ask for their weights later than those that were idle, and some may have no unit at all.  Giving every call
    // position its own tile, under the condition that the stage still fits the grid in one round, lets the late
    // workgroups take the small tiles.  Judged on the whole kernel.
    if (promising && budget <= 1 && !env::is_true("MONONN_TUNER_NO_REFINEMENT")) {
      MonoNNModule probe(params.hlo_text, [&] {
        GraphSpecification s = stitched;
        s.codegen_allow_list.clear();
        s.hip.profile_stages = false;
        return s.to_json().dump(0);
      }(), "mononn_probe");
      bool ok = true;
      try {
        probe.generate_code();
      } catch (const Error&) {
        ok = false;
      }
      if (ok) {
        const codegen::HipProgram& php = probe.hip_program();
        std::map<std::string, const codegen::NodeReport*> report_of;
        for (auto& r : php.nodes) report_of[r.name] = &r;
        std::map<std::string, const graph::Node*> node_of;
        for (auto& n : probe.program().nodes) node_of[n.name] = &n;
        // (function of the class under this specification, position in the stage) -> nodes; stage totals
        std::map<std::pair<std::string, int>, std::vector<std::string>> groups;
        std::map<std::string, int64_t> stage_total_of;   // node -> units of its whole stage
        for (auto& st : php.stage_nodes) {
          int gemms = 0;
          int64_t total = 0;
          for (auto& n : st) {
            auto it = report_of.find(n);
            if (it == report_of.end()) continue;
            total += it->second->units;
            gemms += it->second->kind == "gemm";
          }
          if (gemms < 2) continue;
          for (size_t pos = 0; pos < st.size(); ++pos) {
            auto it = report_of.find(st[pos]);
            if (it == report_of.end() || it->second->kind != "gemm") continue;
            auto nd = node_of.find(st[pos]);
            if (nd == node_of.end() || !nd->second->prologue.empty() || nd->second->gemm.split_k > 1 || !codegen::gemm_uses_mfma(nd->second->gemm)) continue;
            groups[{nd->second->gemm.problem_hash(), static_cast<int>(pos)}].push_back(st[pos]);
            stage_total_of[st[pos]] = total;
          }
        }
        if (stitched_us < 0) stitched_us = whole_kernel_us(stitched);
        // the calls of one problem shape, in stage order; a candidate tile is given to the first p of them (the
        // workgroups with the lowest numbers are the ones that were busy in the stage before), p = 1 .. all
        std::map<std::string, std::vector<int>> positions_of;
        for (auto& gr : groups) positions_of[gr.first.first].push_back(gr.first.second);
        for (auto& fam : positions_of) {
          std::vector<int>& pos = fam.second;
          std::sort(pos.begin(), pos.end());
          const std::vector<std::string>& first_names = groups.at({fam.first, pos[0]});
          const graph::GemmDesc& g = node_of.at(first_names[0])->gemm;
          const int64_t total = stage_total_of.at(first_names[0]);
          const int64_t grid = php.grid;
          std::string line;
          double best_us2 = -1;
          GraphSpecification best_spec2;
          for (size_t p = 1; p <= pos.size(); ++p) {
            int64_t cur = 0;
            for (size_t i = 0; i < p; ++i) cur += report_of.at(groups.at({fam.first, pos[i]})[0])->units;
            struct Cand {
              codegen::GemmTuning t;
              int64_t units;
            };
            std::vector<Cand> cands;
            for (auto& t : gemm_candidates(g, cx.block / 64, 1)) {
              const int64_t u = ((g.M + t.bm - 1) / t.bm) * ((g.N + t.bn - 1) / t.bn) * g.batch;
              const int64_t new_total = total - cur + static_cast<int64_t>(p) * u;
              if (static_cast<int64_t>(p) * u == cur || new_total > grid || 8 * new_total < 7 * grid || t.wk != cx.block / 64) continue;
              cands.push_back({t, u});
            }
            // fullest grid first; a handful is enough
            std::sort(cands.begin(), cands.end(), [&](const Cand& a, const Cand& b) { return a.units > b.units; });
            if (cands.size() > 4) cands.resize(4);
            for (auto& cd : cands) {
              GraphSpecification s2 = stitched;
              for (size_t i = 0; i < p; ++i)
                for (auto& n : groups.at({fam.first, pos[i]})) apply_gemm(s2, n, cd.t, g.K);
              const double us2 = whole_kernel_us(s2);
              char buf[112];
              std::snprintf(buf, sizeof buf, "first%zu:tile%dx%d_waves%dx%dx%d(%lld units each)", p, cd.t.bm, cd.t.bn, cd.t.wm, cd.t.wn, cd.t.wk,
                            static_cast<long long>(cd.units));
              line += timed(buf, us2);
              if (us2 > 0 && (best_us2 < 0 || us2 < best_us2)) {
                best_us2 = us2;
                best_spec2 = std::move(s2);
              }
            }
          }
          if (line.empty()) continue;
          log << "  [" << ctx_str << "] tiles per call in the stages of " << first_names[0] << " (x" << first_names.size() << ", " << pos.size() << " calls, " << total
              << " units): now " << stitched_us << " us;" << line << "\n";
          if (verbose) std::fprintf(stderr, "[mononn tuner] %s tiles per call (%s): now %.2f us;%s\n", ctx_str.c_str(), first_names[0].c_str(), stitched_us, line.c_str());
          if (best_us2 > 0 && best_us2 < 0.997 * stitched_us) {
            stitched = std::move(best_spec2);
            stitched_us = best_us2;
          }
        }
      }
    }
    // ---- stage-fusion decisions ------------------------------------------------------------------------
    // Which stages exist is a tuning decision like any tile (the reference's per-node implementation alternatives,
    // tuning_space_generator.cc:139-307, and its pass switches, config.cc:82-86): with the tiles settled, every decision
    // of the specification's mononn_hip section that changes the stage list or the barrier tiers is tried on the whole
    // kernel and kept when that kernel is faster.  A decision that merges nodes renames them: the new nodes start from
    // the tile of the GEMM instruction they contain, and the GEMMs that changed get a short tile search of their own.
    if (promising && !env::is_true("MONONN_TUNER_NO_FUSION_SEARCH") && !env::is_true("MONONN_TUNER_NO_REFINEMENT")) {
      struct Decision {
        const char* name;
        void (*set)(spec::HipOptions&);
        bool (*is_on)(const spec::HipOptions&);
      };
      const Decision decisions[] = {
          {"regional_synchronization", [](spec::HipOptions& h) { h.regional_synchronization = true; }, [](const spec::HipOptions& h) { return h.regional_synchronization; }},
          {"attention_out_proj_fusion", [](spec::HipOptions& h) { h.attention_out_proj_fusion = true; }, [](const spec::HipOptions& h) { return h.attention_out_proj_fusion; }},
          {"layer_norm_folding", [](spec::HipOptions& h) { h.gemm_prologue_fusion = h.layer_norm_folding = true; }, [](const spec::HipOptions& h) { return h.layer_norm_folding; }},
          {"gemm_prologue_fusion", [](spec::HipOptions& h) { h.gemm_prologue_fusion = true; }, [](const spec::HipOptions& h) { return h.gemm_prologue_fusion; }},
      };
      auto plain = [](GraphSpecification s) {
        s.codegen_allow_list.clear();
        s.hip.profile_stages = false;
        return s;
      };
      // node name -> name of the GEMM instruction inside, and the nodes of a specification's graph
      auto gemm_instr_of = [&](const GraphSpecification& s, std::map<std::string, std::string>* instr_of, std::map<std::string, graph::GemmDesc>* desc_of,
                               std::set<std::string>* all_nodes, std::map<std::string, bool>* has_prologue) {
        MonoNNModule probe(params.hlo_text, plain(s).to_json().dump(0), "mononn_probe");
        probe.generate_code();
        for (auto& n : probe.program().nodes) {
          all_nodes->insert(n.name);
          if (n.kind != graph::NodeKind::kGemm) continue;
          (*instr_of)[n.name] = n.members[0]->name;
          (*desc_of)[n.name] = n.gemm;
          (*has_prologue)[n.name] = !n.prologue.empty();
        }
      };
      if (stitched_us < 0) stitched_us = whole_kernel_us(stitched);
      for (const Decision& d : decisions) {
        if (d.is_on(stitched.hip) || stitched_us < 0) continue;
        // The out-projection inside attention is searched only on request: at GPT-2 / BERT-large size a kernel of this
        // search ended in a GPU memory fault whose cause has not been shown, and a faulted device ends the whole search.
        // The option itself stays valid in a specification.
        if (std::string(d.name) == "attention_out_proj_fusion" && !env::is_true("MONONN_TUNER_TRY_OUT_PROJ_FUSION")) {
          log << "  [" << ctx_str << "] fusion decision " << d.name << ", whole kernel: now " << stitched_us
              << " us; not tried [searched only with MONONN_TUNER_TRY_OUT_PROJ_FUSION=1]  -> not adopted\n";
          continue;
        }
        GraphSpecification s = stitched;
        d.set(s.hip);
        std::string line;
        double best_d = -1;
        GraphSpecification best_spec_d;
        try {
          std::map<std::string, std::string> old_instr, new_instr;
          std::map<std::string, graph::GemmDesc> old_desc, new_desc;
          std::map<std::string, bool> old_pro, new_pro;
          std::set<std::string> old_nodes, new_nodes;
          gemm_instr_of(stitched, &old_instr, &old_desc, &old_nodes, &old_pro);
          // the graph under the decision: entries of nodes that no longer exist would be refused, so only the k splits
          // stay (a split GEMM goes by the name of its instruction and shapes the nodes around it); where the decision
          // takes such a GEMM away (a projection absorbed by its attention node), its split goes with it
          GraphSpecification bare = s;
          bare.cluster_reduce_spec.clear();
          bare.cluster_elewise_spec.clear();
          for (auto it = bare.gemm_spec_list.begin(); it != bare.gemm_spec_list.end();) it = it->second.split_k > 1 ? std::next(it) : bare.gemm_spec_list.erase(it);
          for (;;) {
            try {
              gemm_instr_of(bare, &new_instr, &new_desc, &new_nodes, &new_pro);
              break;
            } catch (const Error&) {
              if (bare.gemm_spec_list.empty()) throw;
              new_instr.clear(), new_desc.clear(), new_nodes.clear(), new_pro.clear();
              bare.gemm_spec_list.erase(bare.gemm_spec_list.begin());
            }
          }
          auto drop = [&](auto& m) {
            for (auto it = m.begin(); it != m.end();) it = new_nodes.count(it->first) ? std::next(it) : m.erase(it);
          };
          drop(s.gemm_spec_list);
          drop(s.cluster_reduce_spec);
          drop(s.cluster_elewise_spec);
          std::map<std::string, std::string> entry_of_instr;   // GEMM instruction -> node that held it before
          for (auto& kv : old_instr) entry_of_instr[kv.second] = kv.first;
          std::vector<std::string> renamed;
          for (auto& kv : new_instr) {
            if (s.gemm_spec_list.count(kv.first)) continue;
            renamed.push_back(kv.first);
            auto from = entry_of_instr.find(kv.second);
            if (from == entry_of_instr.end() || !stitched.gemm_spec_list.count(from->second)) continue;
            // the tile moves with the instruction when the generator takes it for the new node
            GraphSpecification with = s;
            with.gemm_spec_list[kv.first] = stitched.gemm_spec_list.at(from->second);
            try {
              MonoNNModule probe(params.hlo_text, plain(with).to_json().dump(0), "mononn_probe");
              probe.generate_code();
              s = std::move(with);
            } catch (const Error&) {
            }
          }
          double us = whole_kernel_us(s);
          line += timed("as_is", us);
          if (us > 0) best_d = us, best_spec_d = s;
          // the GEMMs whose node changed, by problem: a few tiles each, on the whole kernel
          if (us > 0 && us < 1.15 * stitched_us && !renamed.empty()) {
            std::map<std::string, std::vector<std::string>> families;
            for (auto& n : renamed) families[new_desc.at(n).problem_hash() + (new_pro.at(n) ? "_pro" : "")].push_back(n);
            for (auto& fam : families) {
              const graph::GemmDesc& g = new_desc.at(fam.second[0]);
              if (!codegen::gemm_uses_mfma(g)) continue;
              std::vector<codegen::GemmTuning> tiles = gemm_candidates(g, cx.block / 64, std::max(budget, 1));
              // nearest to the grid first: the tiles whose unit count fills the workgroups once
              const int64_t grid = base.runtime.grid_dim.x;
              std::stable_sort(tiles.begin(), tiles.end(), [&](const codegen::GemmTuning& a, const codegen::GemmTuning& b) {
                auto units = [&](const codegen::GemmTuning& t) { return ((g.M + t.bm - 1) / t.bm) * ((g.N + t.bn - 1) / t.bn) * g.batch * std::max(1, g.split_k); };
                auto badness = [&](int64_t u) { return u > grid ? (u - grid) * 4 : grid - u; };
                return badness(units(a)) < badness(units(b));
              });
              if (tiles.size() > 6) tiles.resize(6);
              for (auto& t : tiles) {
                GraphSpecification s2 = best_spec_d;
                for (auto& n : fam.second) {
                  const int split = s2.gemm_spec_list.count(n) ? s2.gemm_spec_list.at(n).split_k : 1;
                  apply_gemm(s2, n, t, g.K / std::max(1, g.split_k));
                  s2.gemm_spec_list[n].split_k = split;
                }
                const double us2 = whole_kernel_us(s2);
                char lbl[96];
                std::snprintf(lbl, sizeof lbl, "%s:tile%dx%d_waves%dx%dx%d%s", fam.first.c_str(), t.bm, t.bn, t.wm, t.wn, t.wk, t.stages >= 2 ? "_lds" : "");
                line += timed(lbl, us2);
                if (us2 > 0 && us2 < best_d) best_d = us2, best_spec_d = std::move(s2);
              }
            }
          }
        } catch (const Error& e) {
          line += std::string(" not applicable [") + e.what() + "]";
        }
        log << "  [" << ctx_str << "] fusion decision " << d.name << ", whole kernel: now " << stitched_us << " us;" << line
            << (best_d > 0 && best_d < 0.997 * stitched_us ? "  -> adopted" : "  -> not adopted") << "\n";
        if (verbose) std::fprintf(stderr, "[mononn tuner] %s fusion decision %s: now %.2f us;%s\n", ctx_str.c_str(), d.name, stitched_us, line.c_str());
        if (best_d > 0 && best_d < 0.997 * stitched_us) {
          stitched = std::move(best_spec_d);
          stitched_us = best_d;
        }
      }
    }
    // ---- whole kernel of this context --------------------------------------------------------------
    stitched.codegen_allow_list.clear();
    stitched.hip.profile_stages = false;
    auto full = std::make_unique<MonoNNModule>(params.hlo_text, stitched.to_json().dump(0), params.kernel_name);
    double us = -1;
    try {
      full->generate_code();
      full->build_assembly();
      bufs.ensure_temp(static_cast<size_t>(full->hip_program().temp_bytes));
      us = time_module(*full, params.device, bufs, 5, 30);
    } catch (const Error& e) {
      log << ctx_str << " failed: " << e.what() << "\n";
      continue;
    }
    log << ctx_str << " " << us / 1000.0 << " ms\n";
    if (!params.dump_dir.empty()) full->dump_candidate(params.dump_dir);
    if (best_us < 0 || us < best_us) {
      best_us = us;
      // hand back an unloaded module: the caller uploads constants and loads it where it wants
      best = std::make_unique<MonoNNModule>(params.hlo_text, stitched.to_json().dump(0), params.kernel_name);
      best->generate_code();
      best->set_code_object(full->code_object());
    }
  }
  MONONN_CHECK(best != nullptr, kRuntimeError) << "no launch context could be tuned:\n" << log.str();
  if (!params.dump_dir.empty()) {
    best->dump_best(params.dump_dir);
    std::string dir = best->cluster_dir(params.dump_dir);
    module::write_file(dir + "/tuning_log.log", log.str());
    module::write_file(dir + "/performance_report.csv", report.str());
  }
  return best;
}

}  // namespace tuner
}  // namespace mononn
