// Kernel variant "prof" of the evaluator, compiled as its own translation unit.
#include "bf_kernel.hip.h"

namespace bf {
hipError_t launch_prof(const KArgs& k, int grid, hipStream_t stream) { return launch_variant<false, true, false>(k, grid, stream); }
}  // namespace bf
