// Kernel variant "twin256_taps" of the evaluator (one position per workgroup), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_twin256_taps(const KArgs& k, hipStream_t stream) { return board::launch_board<256, true, true>(k, stream); }
}  // namespace bf
