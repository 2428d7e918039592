// model.hip — fused whole-model decode / prefill entry points (placeholder until the pipeline lands).
#include "runtime_internal.h"

namespace oxb {
void shutdown_models() {}
}  // namespace oxb
