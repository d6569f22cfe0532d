// Kernel variant "twin256_fp8_prof" of the evaluator (one position per workgroup, two workgroups per compute unit, e4m3, with the phase profile), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_twin256_fp8_prof(const KArgs& k, hipStream_t stream) { return board::launch_board<256, false, true, true, false, true>(k, stream); }
}  // namespace bf
