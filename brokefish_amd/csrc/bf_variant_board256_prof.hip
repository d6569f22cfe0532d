// Kernel variant "board256_prof" of the evaluator (one position per workgroup, one workgroup per compute unit, int8, with the phase profile), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_board256_prof(const KArgs& k, hipStream_t stream) { return board::launch_board<256, false, false, false, false, true>(k, stream); }
}  // namespace bf
