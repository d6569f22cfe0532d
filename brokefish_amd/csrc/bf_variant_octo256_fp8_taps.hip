// Kernel variant "octo256_fp8_taps" of the evaluator (one position per workgroup of eight wavefronts, e4m3), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_octo256_fp8_taps(const KArgs& k, hipStream_t stream) { return board::launch_board<256, true, true, true, true>(k, stream); }
}  // namespace bf
