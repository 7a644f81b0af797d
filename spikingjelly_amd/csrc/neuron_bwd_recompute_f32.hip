// Recompute-backward kernels for storage dtype float.
#include "neuron_bwd_recompute_launch.h"

namespace sjhip {
template int launch_recompute_dtype<float>(const FwdArgs &, const BwdArgs &, bool, int, int, unsigned, int64_t, hipStream_t, const PieceArgs *);
}  // namespace sjhip
