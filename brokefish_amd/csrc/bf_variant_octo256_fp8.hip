// Kernel variant "octo256_fp8" of the evaluator (one position per workgroup of eight wavefronts, e4m3), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_octo256_fp8(const KArgs& k, hipStream_t stream) { return board::launch_board<256, false, true, true, true>(k, stream); }
}  // namespace bf
