// Host launcher of the multi-step forward kernels.
#include "neuron_fwd.h"

#include <cmath>

namespace sjhip {

namespace {

#ifndef SJHIP_FWD_STREAM_X_FP32
#define SJHIP_FWD_STREAM_X_FP32 0
#endif
template <typename S, bool ROUND_EACH>
constexpr bool kStreamX = (sizeof(S) == 2 && !ROUND_EACH) || (sizeof(S) == 4 && SJHIP_FWD_STREAM_X_FP32 != 0);

template <typename S, bool ROUND_EACH, bool PACKED = false>
int launch_typed(const FwdArgs &a, bool vector, hipStream_t stream) {
  int block = tuning().fwd_block;
  // (the block size changes only with the runs that answer a resonant row stride, not with the contiguous eighths)
  if (a.spread > 1 && tuning().column_spread == 2) block = spread_block(a.N * (int64_t)sizeof(S));
  const int V = vector ? Acc<S, true, true>::V : 1;
  const int64_t items = (a.N + V - 1) / V;
  const int64_t blocks = (items + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "forward: N=%lld needs %lld blocks", (long long)a.N, (long long)blocks);
  // the residency cap pays for fp32 storage writing two or three [T, N] tensors (spikes plus v_seq and / or h_seq);
  // with spikes only, and with 16-bit storage (more wavefronts hide its conversions), uncapped is faster (measured)
  // A short sequence has few rows in flight per work-item and needs more resident blocks instead: twice the cap
  // below 16 steps, none below 4 (measured at T = 1, 2, 4, 8, 16).  ILIF's step is a longer dependent chain (a
  // quotient, a clamp and a rounding on top of the charge): with two resident blocks that latency shows, with four
  // it is hidden (measured 1.47 -> 1.24 ms at T = 16, N = 33.5 M).  The same holds for EIF's exp().
  const bool several_outputs = a.v_seq != nullptr || a.h != nullptr;
  int cap = tuning().fwd_blocks_per_cu;
  if (a.T < 4) cap = 0;
  else if (a.T < 16 || a.soft_reset == RESET_COUNT || a.charge == CH_EIF_DIV || a.charge == CH_EIF_MUL) cap *= 2;
  const unsigned lds = (sizeof(S) == 4 && several_outputs) ? occupancy_cap_lds(cap) : 0u;
  ProfileScope prof(KC_FORWARD, stream);
  const dim3 grid((unsigned)blocks), threads(block);
  if constexpr (PACKED) {
    if (vector) hipLaunchKernelGGL((forward_kernel<S, true, ROUND_EACH, FWD_OUT_PACKED>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((forward_kernel<S, false, ROUND_EACH, FWD_OUT_PACKED>), grid, threads, lds, stream, a);
  } else if (kStreamX<S, ROUND_EACH> && several_outputs && a.T > 1) {
    // 16-bit storage with fp32 state writing spikes plus v_seq / h_seq: see FwdOut
    if constexpr (kStreamX<S, ROUND_EACH>) {
      if (vector) hipLaunchKernelGGL((forward_kernel<S, true, ROUND_EACH, FWD_OUT_DENSE_STREAM_X>), grid, threads, lds, stream, a);
      else hipLaunchKernelGGL((forward_kernel<S, false, ROUND_EACH, FWD_OUT_DENSE_STREAM_X>), grid, threads, lds, stream, a);
    }
  } else if (a.T == 1) {
    if (vector) hipLaunchKernelGGL((forward_kernel<S, true, ROUND_EACH, FWD_OUT_DENSE | FWD_OUT_SHORT>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((forward_kernel<S, false, ROUND_EACH, FWD_OUT_DENSE | FWD_OUT_SHORT>), grid, threads, lds, stream, a);
  } else {
    if (vector) hipLaunchKernelGGL((forward_kernel<S, true, ROUND_EACH, FWD_OUT_DENSE>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((forward_kernel<S, false, ROUND_EACH, FWD_OUT_DENSE>), grid, threads, lds, stream, a);
  }
  return check_launch(PACKED ? "forward_packed" : "forward");
}

template <typename S, bool ROUND_EACH> int launch_pieces_typed(const FwdArgs &a, hipStream_t stream) {
  // From 64 steps on, one wavefront per block: the steady-state loop keeps a block's next rows in flight while it
  // computes, so half the resident work-items still fill the memory pipeline, and with a fixed number of neuron-steps
  // a longer sequence means fewer, longer blocks, whose last round leaves less of the chip idle when they are small
  // (2^29 neuron-steps, fp32, T = 64 / 128 / 512: 1.198 / 1.234 / 1.327 ms against 1.231 / 1.283 / 1.398 with 128
  // lanes; T = 48: 1.304 against 1.283).
  const int block = a.T >= 64 && tuning().fwd_block > 64 ? 64 : tuning().fwd_block;
  const int64_t items = a.N / Acc<S, true, true>::V;
  const int64_t blocks = (items + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "forward(pieces): N=%lld", (long long)a.N);
  const unsigned lds = (sizeof(S) == 4 && a.v_seq != nullptr) ? occupancy_cap_lds(tuning().fwd_blocks_per_cu) : 0u;
  ProfileScope prof(KC_FORWARD, stream);
  hipLaunchKernelGGL((forward_pieces_kernel<S, ROUND_EACH>), dim3((unsigned)blocks), dim3(block), lds, stream, a);
  return check_launch("forward(pieces)");
}

}  // namespace

int launch_forward_pieces(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N, int64_t chunk,
                          const void *x_seq, const void *v_init, const float *k_device, void *spike_seq, void *v_seq,
                          void *v_last, void *checkpoints, hipStream_t stream) {
  FwdArgs a;
  bool round_each = false;
  int rc = build_fwd_args(a, round_each, neuron, dtype, p, T, N, x_seq, v_init, k_device, spike_seq, v_seq, v_last, nullptr);
  if (rc != SJHIP_OK) return rc;
  const int V = dtype == SJHIP_F32 ? 4 : 8;
  if (N % V != 0 || !aligned16(x_seq) || !(a.v_init_broadcast || aligned16(v_init)) || !aligned16(spike_seq) || !aligned16(v_seq) ||
      !aligned16(v_last) || !aligned16(checkpoints))
    return fail(SJHIP_ERR_UNSUPPORTED, "forward(pieces): N=%lld must be a multiple of %d and every tensor 16-byte aligned", (long long)N, V);
  a.checkpoints = checkpoints; a.chunk = chunk;
  switch (dtype) {
    case SJHIP_F32: return launch_pieces_typed<float, false>(a, stream);
    case SJHIP_F16: return round_each ? launch_pieces_typed<f16_t, true>(a, stream) : launch_pieces_typed<f16_t, false>(a, stream);
    case SJHIP_BF16: return round_each ? launch_pieces_typed<bf16_t, true>(a, stream) : launch_pieces_typed<bf16_t, false>(a, stream);
    default: return fail(SJHIP_ERR_INVALID, "forward(pieces): dtype %d", dtype);
  }
}

int launch_forward_packed(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                          const void *x_seq, const void *v_init, const float *k_device, uint8_t *spike_bits,
                          void *v_seq, void *v_last, hipStream_t stream) {
  if (N % 8 != 0)
    return fail(SJHIP_ERR_UNSUPPORTED, "forward_packed: N=%lld is not a multiple of 8 (rows must start on a byte)", (long long)N);
  FwdArgs a;
  bool round_each = false;
  int rc = build_fwd_args(a, round_each, neuron, dtype, p, T, N, x_seq, v_init, k_device, spike_bits, v_seq, v_last, nullptr);
  if (rc != SJHIP_OK) return rc;
  const bool vector = aligned16(x_seq) && (a.v_init_broadcast || aligned16(v_init)) && (v_seq == nullptr || aligned16(v_seq)) &&
                      (v_last == nullptr || aligned16(v_last));
  switch (dtype) {
    case SJHIP_F32: return launch_typed<float, false, true>(a, vector, stream);
    case SJHIP_F16: return round_each ? launch_typed<f16_t, true, true>(a, vector, stream) : launch_typed<f16_t, false, true>(a, vector, stream);
    case SJHIP_BF16: return round_each ? launch_typed<bf16_t, true, true>(a, vector, stream) : launch_typed<bf16_t, false, true>(a, vector, stream);
    default: return fail(SJHIP_ERR_INVALID, "forward_packed: dtype %d", dtype);
  }
}

int launch_forward(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                   const void *x_seq, const void *v_init, const float *k_device, void *spike_seq,
                   void *v_seq, void *v_last, void *h_seq, hipStream_t stream) {
  FwdArgs a;
  bool round_each = false;
  int rc = build_fwd_args(a, round_each, neuron, dtype, p, T, N, x_seq, v_init, k_device, spike_seq, v_seq, v_last, h_seq);
  if (rc != SJHIP_OK) return rc;

  const int esize = dtype == SJHIP_F32 ? 4 : 2;
  const int V = 16 / esize;
  const bool vector = (N % V == 0) && aligned16(x_seq) && (a.v_init_broadcast || aligned16(v_init)) && aligned16(spike_seq) &&
                      (v_seq == nullptr || aligned16(v_seq)) && (v_last == nullptr || aligned16(v_last)) &&
                      (h_seq == nullptr || aligned16(h_seq));

  switch (dtype) {
    case SJHIP_F32: return launch_typed<float, false>(a, vector, stream);
    case SJHIP_F16: return round_each ? launch_typed<f16_t, true>(a, vector, stream) : launch_typed<f16_t, false>(a, vector, stream);
    case SJHIP_BF16: return round_each ? launch_typed<bf16_t, true>(a, vector, stream) : launch_typed<bf16_t, false>(a, vector, stream);
    default: return fail(SJHIP_ERR_INVALID, "forward: dtype %d", dtype);
  }
}

}  // namespace sjhip
