// Kernel variant "octo512" of the evaluator (one position per workgroup of eight wavefronts, 512-wide network), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_octo512(const KArgs& k, hipStream_t stream) { return board::launch_board<512, false, true, false, true>(k, stream); }
}  // namespace bf
