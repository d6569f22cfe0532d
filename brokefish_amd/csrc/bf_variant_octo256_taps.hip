// Kernel variant "octo256_taps" of the evaluator (one position per workgroup of eight wavefronts), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_octo256_taps(const KArgs& k, hipStream_t stream) { return board::launch_board<256, true, true, false, true>(k, stream); }
}  // namespace bf
