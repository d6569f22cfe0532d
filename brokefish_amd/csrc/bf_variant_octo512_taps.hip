// Kernel variant "octo512_taps" of the evaluator (one position per workgroup of eight wavefronts, 512-wide network), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_octo512_taps(const KArgs& k, hipStream_t stream) { return board::launch_board<512, true, true, false, true>(k, stream); }
}  // namespace bf
