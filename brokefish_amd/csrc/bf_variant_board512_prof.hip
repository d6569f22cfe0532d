// Kernel variant "board512_prof" of the evaluator (the 512-wide network, four wavefronts per position, int8, with the phase profile), compiled as its own translation unit.
#include "bf_board.hip.h"

namespace bf {
hipError_t launch_board512_prof(const KArgs& k, hipStream_t stream) { return board::launch_board<512, false, false, false, false, true>(k, stream); }
}  // namespace bf
