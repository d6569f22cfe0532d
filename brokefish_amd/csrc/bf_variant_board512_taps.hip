// Kernel variant "board512_taps" of the evaluator (one position per workgroup), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_board512_taps(const KArgs& k, hipStream_t stream) { return board::launch_board<512, true, false>(k, stream); }
}  // namespace bf
