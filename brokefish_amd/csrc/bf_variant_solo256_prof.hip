// Kernel variant "solo256_prof" of the evaluator (one position per workgroup of eight wavefronts, products issued under the previous epilogue), compiled as its own translation unit.
#include "bf_duo.hip.h"

namespace bf {
hipError_t launch_solo256_prof(const KArgs& k, hipStream_t stream) { return duo::launch_duo<false, false, true, 1>(k, stream); }
}  // namespace bf
