// Kernel variant "twin256_prof" of the evaluator (one position per workgroup, with the phase profile), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_twin256_prof(const KArgs& k, hipStream_t stream) { return board::launch_board<256, false, true, false, false, true>(k, stream); }
}  // namespace bf
