// Kernel variant "duo256_fp8_prof" of the evaluator (two positions per workgroup, e4m3, with the phase profile), compiled as its own translation unit.
#include "bf_duo.hip.h"

namespace bf {
hipError_t launch_duo256_fp8_prof(const KArgs& k, hipStream_t stream) { return duo::launch_duo<false, true, true>(k, stream); }
}  // namespace bf
