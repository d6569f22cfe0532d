// Kernel variant "duo256_prof" of the evaluator (two positions per workgroup, phase profile), compiled as its own translation unit.
#include "bf_duo.hip.h"

namespace bf {
hipError_t launch_duo256_prof(const KArgs& k, hipStream_t stream) { return duo::launch_duo<false, false, true>(k, stream); }
}  // namespace bf
