#include "tuner/tuner.h"

#include "common/status.h"

namespace mononn {
namespace tuner {

std::unique_ptr<module::MonoNNModule> MonoNNModuleTuner::tune(const TuneParams& params) {
  (void)params;
  MONONN_FAIL(kUnsupported) << "tuner not built yet";
}

}  // namespace tuner
}  // namespace mononn
