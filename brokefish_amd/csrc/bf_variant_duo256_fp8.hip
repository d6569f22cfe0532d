// Kernel variant "duo256_fp8" of the evaluator (two positions per workgroup), compiled as its own translation unit.
#include "bf_duo.hip.h"

namespace bf {
hipError_t launch_duo256_fp8(const KArgs& k, hipStream_t stream) { return duo::launch_duo<false,true>(k, stream); }
}  // namespace bf
