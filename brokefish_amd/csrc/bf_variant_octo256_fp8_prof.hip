// Kernel variant "octo256_fp8_prof" of the evaluator (eight wavefronts per position, e4m3, with the phase profile), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_octo256_fp8_prof(const KArgs& k, hipStream_t stream) { return board::launch_board<256, false, true, true, true, true>(k, stream); }
}  // namespace bf
