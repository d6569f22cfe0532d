// Kernel variant "octo256" of the evaluator (one position per workgroup of eight wavefronts), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_octo256(const KArgs& k, hipStream_t stream) { return board::launch_board<256, false, true, false, true>(k, stream); }
}  // namespace bf
