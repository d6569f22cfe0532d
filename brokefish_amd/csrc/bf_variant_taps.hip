// Kernel variant "taps" of the evaluator, compiled as its own translation unit.
#include "bf_kernel.hip.h"

namespace bf {
hipError_t launch_taps(const KArgs& k, int grid, hipStream_t stream) { return launch_variant<true, false, false>(k, grid, stream); }
}  // namespace bf
