// Tuning-space search on the target GPU.
//
// Reference: MonoNNModuleTuner::tune (mononn_engine/module/mononn_module_tuner.cc:620-991) with
// TuningSpaceGenerator (mononn_engine/tuning/tuning_space_generator.cc:52-310): per launch context
// (grid, block) every node gets its candidates timed alone, GEMMs de-duplicated by problem hash
// (:386-408), the best per-node choices are stitched into one specification per context, each
// context's whole kernel is timed and the fastest wins (final_tuning, :450-618).
#pragma once
#include <memory>
#include <string>

#include "module/mononn_module.h"

namespace mononn {
namespace tuner {

struct TuneParams {
  std::string hlo_text;
  std::string kernel_name;
  int device = 0;
  std::string dump_dir;   // empty = no dump
  int budget = 0;         // 0 full, 1 faster, 2 fastest
};

class MonoNNModuleTuner {
 public:
  static std::unique_ptr<module::MonoNNModule> tune(const TuneParams& params);
};

}  // namespace tuner
}  // namespace mononn
