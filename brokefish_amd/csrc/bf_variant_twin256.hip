// Kernel variant "twin256" of the evaluator (one position per workgroup), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_twin256(const KArgs& k, hipStream_t stream) { return board::launch_board<256, false, true>(k, stream); }
}  // namespace bf
