// Kernel variant "duo256" of the evaluator (two positions per workgroup), compiled as its own translation unit.
#include "bf_duo.hip.h"

namespace bf {
hipError_t launch_duo256(const KArgs& k, hipStream_t stream) { return duo::launch_duo<false,false>(k, stream); }
}  // namespace bf
