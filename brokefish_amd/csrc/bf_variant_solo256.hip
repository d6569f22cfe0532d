// Kernel variant "solo256" of the evaluator (one position per workgroup of eight wavefronts, products issued under the previous epilogue), compiled as its own translation unit.
#include "bf_duo.hip.h"

namespace bf {
hipError_t launch_solo256(const KArgs& k, hipStream_t stream) { return duo::launch_duo<false, false, false, 1>(k, stream); }
}  // namespace bf
