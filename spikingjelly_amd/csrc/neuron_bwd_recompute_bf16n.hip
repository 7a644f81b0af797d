// Recompute-backward kernels for storage dtype bf16n_t (8-byte accesses, fp32 state).
#include "neuron_bwd_recompute_launch.h"

namespace sjhip {
template int launch_recompute_dtype<bf16n_t>(const FwdArgs &, const BwdArgs &, bool, int, int, unsigned, int64_t, hipStream_t, const PieceArgs *);
}  // namespace sjhip
