// Kernel variant "prof_fp8" of the evaluator (four positions per workgroup, e4m3, with the phase profile), compiled as its own translation unit.
#include "bf_kernel.hip.h"

namespace bf {
hipError_t launch_prof_fp8(const KArgs& k, int grid, hipStream_t stream) { return launch_variant<false, true, true>(k, grid, stream); }
}  // namespace bf
