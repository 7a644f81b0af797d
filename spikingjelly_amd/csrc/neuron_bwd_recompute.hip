// Host launcher of the recompute backward (see neuron_bwd_recompute.h).
#include "neuron_bwd_recompute.h"

// the kernels of each storage dtype are compiled in their own translation unit


namespace sjhip {

extern template int launch_recompute_dtype<float>(const FwdArgs &, const BwdArgs &, bool, int, int, unsigned, int64_t, hipStream_t, const PieceArgs *);
extern template int launch_recompute_dtype<f16_t>(const FwdArgs &, const BwdArgs &, bool, int, int, unsigned, int64_t, hipStream_t, const PieceArgs *);
extern template int launch_recompute_dtype<bf16_t>(const FwdArgs &, const BwdArgs &, bool, int, int, unsigned, int64_t, hipStream_t, const PieceArgs *);
extern template int launch_recompute_dtype<f16n_t>(const FwdArgs &, const BwdArgs &, bool, int, int, unsigned, int64_t, hipStream_t, const PieceArgs *);
extern template int launch_recompute_dtype<bf16n_t>(const FwdArgs &, const BwdArgs &, bool, int, int, unsigned, int64_t, hipStream_t, const PieceArgs *);

namespace {

constexpr unsigned kMaxLds = 159u * 1024u;  // LDS per compute unit on gfx950 minus 1 KiB for static words

// LDS bytes one work-item needs per step for h, the same in every mode: its 4 fp32 neurons (fp32 storage, and 16-bit
// storage with fp32 state, which runs four neurons per work-item through 8-byte accesses) or its 8 neurons as 16-bit
// patterns (16-bit storage, every op rounded)
constexpr int64_t kHBytesPerItem = 16;

}  // namespace

// Largest block (128 or 64 lanes) whose h buffer fits in LDS; 0 if none.
int recompute_block(int dtype, int64_t T, bool round_each) {
  for (int block : {128, 64}) {
    if (block > SJHIP_MAX_BLOCK) continue;
    if (T * block * kHBytesPerItem <= (int64_t)kMaxLds) return block;
  }
  return 0;
}

bool recompute_supported(int dtype, int64_t T, int64_t N) {
  const int64_t V = dtype == SJHIP_F32 ? 4 : 8;
  return N % V == 0 && recompute_block(dtype, T, false) != 0;
}

bool recompute_preferred(int dtype, int64_t T, int64_t N, bool round_each) {
  // the replay needs T * 64 lanes * h_bytes of LDS per wavefront; below four resident wavefronts per compute unit
  // it is slower than reading a saved h_seq (measured: T = 32 still wins, T = 64 loses, fp32)
  if (!recompute_supported(dtype, T, N)) return false;
  return 4 * T * 64 * kHBytesPerItem <= (int64_t)kMaxLds;
}

namespace {

// One launch over the whole sequence (chunk == 0: T steps of h in LDS) or over pieces of `chunk` steps.
int launch_replay(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N, int64_t chunk,
                  const void *x_seq, const void *v_init, const float *k_device, const void *checkpoints,
                  const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                  void *grad_x_seq, void *grad_v_init, float *grad_rtau, float *workspace,
                  hipStream_t stream) {
  const int64_t lds_steps = chunk > 0 ? chunk : T;
  if (!recompute_supported(dtype, lds_steps, N))
    return fail(SJHIP_ERR_UNSUPPORTED, "backward(recompute): T=%lld N=%lld does not fit (N %% %d != 0 or T too large for LDS)",
                (long long)T, (long long)N, dtype == SJHIP_F32 ? 4 : 8);
  const bool broadcast = (p.flags & SJHIP_FLAG_V_INIT_BROADCAST) != 0;
  if (!aligned16(x_seq) || (!broadcast && !aligned16(v_init)) || !aligned16(grad_spike_seq) || !aligned16(grad_x_seq) ||
      (grad_v_init && !aligned16(grad_v_init)) || (grad_v_seq && !aligned16(grad_v_seq)) ||
      (grad_v_last && !aligned16(grad_v_last)))
    return fail(SJHIP_ERR_INVALID, "backward(recompute): every tensor must be 16-byte aligned");

  FwdArgs f;
  bool round_each = false;
  // spike/v/h outputs of the replayed forward are never written: the kernel only uses x, v_init and scalars
  int rc = build_fwd_args(f, round_each, neuron, dtype, p, T, N, x_seq, v_init, k_device, nullptr, nullptr, nullptr, nullptr);
  if (rc != SJHIP_OK) return rc;
  BwdArgs b;
  rc = build_bwd_args(b, neuron, dtype, p, T, N, grad_spike_seq, grad_v_seq, grad_v_last, nullptr, v_init, k_device,
                      grad_x_seq, grad_v_init, grad_rtau, workspace);
  if (rc != SJHIP_OK) return rc;

  const bool narrow = dtype != SJHIP_F32 && !round_each;  // 16-bit storage, fp32 state: four neurons per work-item
  const int V = (dtype == SJHIP_F32 || narrow) ? 4 : 8;
  // The walk over several pieces measured faster with each XCD on a contiguous eighth of the columns at every row
  // stride tried (T = 128: 1.65 against 1.88 ms at N = 2^22, and likewise at seven other strides; T = 64: equal or
  // better), unlike the single-piece kernel, which keeps the stride rule of column_spread().  In that order 256
  // work-items per block are 2 to 4 % faster than 128 when two such blocks still fit a compute unit's LDS
  // (T = 128: 1.604 -> 1.543 ms; one piece of 16 steps at N = 2^25 + 1024: 1.466 -> 1.455).
  // A single piece at a resonant stride takes the order and the block size column_spread() and spread_block() give.
  const bool auto_order = tuning().column_spread == 2;
  const bool several = chunk > 0 && T > chunk;
  if (several && auto_order) b.spread = 1;
  int block = recompute_block(dtype, lds_steps, round_each);
  if ((several || b.spread > 1) && auto_order) {
    const int want = several ? kSpreadBlock : spread_block(N * (dtype == SJHIP_F32 ? 4 : 2));
    if (want > block && want <= SJHIP_MAX_BLOCK && 2 * lds_steps * want * kHBytesPerItem <= (int64_t)kMaxLds) block = want;
  }
  const int64_t items = N / V;
  const int64_t blocks = (items + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "backward(recompute): N=%lld", (long long)N);
  unsigned lds = (unsigned)(lds_steps * block * kHBytesPerItem);
  const unsigned cap = occupancy_cap_lds(tuning().replay_blocks_per_cu);
  if (cap > lds) lds = cap;
  const bool plif = neuron == SJHIP_NEURON_PLIF;
  const int mode = plif ? BWD_PLIF : ((neuron == SJHIP_NEURON_QIF || neuron == SJHIP_NEURON_EIF) ? BWD_QIF : BWD_PLAIN);
  PieceArgs piece_args;
  piece_args.checkpoints = const_cast<void *>(checkpoints); piece_args.chunk = chunk;
  piece_args.checkpoints_f32 = checkpoints_are_f32(dtype, p.flags) ? 1 : 0;
  piece_args.pieces = chunk > 0 ? (T + chunk - 1) / chunk : 1;
  const PieceArgs *pieces = chunk > 0 ? &piece_args : nullptr;
  {
    ProfileScope prof(KC_BACKWARD, stream);
    switch (dtype) {
      case SJHIP_F32: rc = launch_recompute_dtype<float>(f, b, false, mode, block, lds, blocks, stream, pieces); break;
      case SJHIP_F16:
        rc = narrow ? launch_recompute_dtype<f16n_t>(f, b, false, mode, block, lds, blocks, stream, pieces)
                    : launch_recompute_dtype<f16_t>(f, b, round_each, mode, block, lds, blocks, stream, pieces);
        break;
      case SJHIP_BF16:
        rc = narrow ? launch_recompute_dtype<bf16n_t>(f, b, false, mode, block, lds, blocks, stream, pieces)
                    : launch_recompute_dtype<bf16_t>(f, b, round_each, mode, block, lds, blocks, stream, pieces);
        break;
      default: return fail(SJHIP_ERR_INVALID, "backward(recompute): dtype %d", dtype);
    }
    if (rc != SJHIP_OK) return rc;
  }
  if (plif && !b.atomic_reduce) return launch_plif_reduce(b, blocks, grad_rtau, stream);
  return SJHIP_OK;
}

}  // namespace

int launch_backward_recompute(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                              const void *x_seq, const void *v_init, const float *k_device,
                              const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                              void *grad_x_seq, void *grad_v_init, float *grad_rtau, float *workspace,
                              hipStream_t stream) {
  return launch_replay(neuron, dtype, p, T, N, 0, x_seq, v_init, k_device, nullptr, grad_spike_seq, grad_v_seq, grad_v_last,
                       grad_x_seq, grad_v_init, grad_rtau, workspace, stream);
}

int launch_backward_recompute_pieces(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N, int64_t chunk,
                                     const void *x_seq, const void *v_init, const float *k_device, const void *checkpoints,
                                     const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                                     void *grad_x_seq, void *grad_v_init, float *grad_rtau, float *workspace,
                                     hipStream_t stream) {
  if (chunk < 1 || (T > chunk && checkpoints == nullptr) || !aligned16(checkpoints))
    return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): chunk=%lld needs 16-byte aligned checkpoints", (long long)chunk);
  return launch_replay(neuron, dtype, p, T, N, chunk, x_seq, v_init, k_device, checkpoints, grad_spike_seq, grad_v_seq,
                       grad_v_last, grad_x_seq, grad_v_init, grad_rtau, workspace, stream);
}

}  // namespace sjhip
