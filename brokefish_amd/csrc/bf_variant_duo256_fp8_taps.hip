// Kernel variant "duo256_fp8_taps" of the evaluator (two positions per workgroup), compiled as its own translation unit.
#include "bf_duo.hip.h"

namespace bf {
hipError_t launch_duo256_fp8_taps(const KArgs& k, hipStream_t stream) { return duo::launch_duo<true,true>(k, stream); }
}  // namespace bf
