// Kernel variant "octo512_prof" of the evaluator (one position per workgroup, with the phase profile), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_octo512_prof(const KArgs& k, hipStream_t stream) { return board::launch_board<512, false, true, false, true, true>(k, stream); }
}  // namespace bf
