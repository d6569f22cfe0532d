// Kernel variant "taps_fp8" of the evaluator, compiled as its own translation unit.
#include "bf_kernel.hip.h"

namespace bf {
hipError_t launch_taps_fp8(const KArgs& k, int grid, hipStream_t stream) { return launch_variant<true, false, true>(k, grid, stream); }
}  // namespace bf
