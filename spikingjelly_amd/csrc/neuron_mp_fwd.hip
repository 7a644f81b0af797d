// Forward kernels of the 8-bit-storage mixed-precision neurons (see neuron_mp.h).
#include "neuron_mp.h"

#ifndef SJHIP_MP_FWD_NT
#define SJHIP_MP_FWD_NT 0
#endif
#ifndef SJHIP_MP_FWD_X_NT
#define SJHIP_MP_FWD_X_NT 0
#endif

namespace sjhip {

template <typename ST, typename SP, int CH, int RS>
__device__ __forceinline__ void mp_forward_walk(const FwdArgs &a, const MpLane &l) {
  typedef Tile16<ST, SJHIP_MP_FWD_NT != 0> RX;  // streaming policy as measured for the fp32 forward: default wins
  typedef Tile16<ST, (SJHIP_MP_FWD_NT != 0) || (SJHIP_MP_FWD_X_NT != 0)> RXL;  // the x loads alone
  typedef Tile16<SP, SJHIP_MP_FWD_NT != 0> RSP;
  constexpr int V = 16, PF = SJHIP_MP_PF;
  const int64_t N = a.N, T = a.T;
  const float tau = a.k_device ? *a.k_device : a.tau;

  typename RXL::raw_t ahead[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) ahead[i] = (i < T) ? RXL::load(a.x, (int64_t)i * N, l) : RXL::zero();
  float v[V];
  if (a.v_init_broadcast) {
    const float v0 = Codec<ST>::dec(*(const uint8_t *)a.v_init);
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] = v0;
  } else {
    RX::unpack(RX::load(a.v_init, 0, l), v);
  }
  for (int64_t t0 = 0; t0 < T; t0 += PF) {
    typename RXL::raw_t now[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) now[i] = ahead[i];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 + PF + i;
      if (tn < T) ahead[i] = RXL::load(a.x, tn * N, l);
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 + i;
      if (t < T) {
        float x[V], h[V], s[V];
        RXL::unpack(now[i], x);
#pragma unroll
        for (int j = 0; j < V; ++j) neuron_step<float, CH, RS>(x[j], v[j], h[j], s[j], tau, a);
        RSP::store(a.spike, t * N, l, s);
        if (a.v_seq) RX::store(a.v_seq, t * N, l, v);
        if (a.h) RX::store(a.h, t * N, l, h);
      }
    }
  }
  if (a.v_last) RX::store(a.v_last, 0, l, v);
}

template <typename ST, typename SP, int CH>
__device__ __forceinline__ void mp_forward_reset(const FwdArgs &a, const MpLane &l) {
  if (a.soft_reset) mp_forward_walk<ST, SP, CH, RESET_SOFT>(a, l);
  else mp_forward_walk<ST, SP, CH, RESET_HARD>(a, l);
}

template <typename ST, typename SP>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) mp_forward_kernel(const FwdArgs a) {
  const MpLane l = mp_lane(a.N);
  if (l.groups == 0) return;
  switch (a.charge) {
    case CH_IF: mp_forward_reset<ST, SP, CH_IF>(a, l); break;
    case CH_DECAY_INPUT_DIV: mp_forward_reset<ST, SP, CH_DECAY_INPUT_DIV>(a, l); break;
    case CH_DECAY_INPUT_MUL: mp_forward_reset<ST, SP, CH_DECAY_INPUT_MUL>(a, l); break;
    case CH_PLAIN_INPUT_DIV: mp_forward_reset<ST, SP, CH_PLAIN_INPUT_DIV>(a, l); break;
    default: mp_forward_reset<ST, SP, CH_PLAIN_INPUT_MUL>(a, l); break;
  }
}

namespace {

template <typename ST>
int launch_fwd_storage(int spike_dtype, const FwdArgs &a, dim3 grid, dim3 threads, hipStream_t stream) {
  // measured at T = 16, N = 33.5 M (blocks of 128): 6 resident blocks per compute unit 0.526 ms, uncapped 0.550, 1-3 0.57
  const unsigned lds = occupancy_cap_lds(6);
  switch (spike_dtype) {
    case SJHIP_F32: hipLaunchKernelGGL((mp_forward_kernel<ST, float>), grid, threads, lds, stream, a); break;
    case SJHIP_F16: hipLaunchKernelGGL((mp_forward_kernel<ST, f16_t>), grid, threads, lds, stream, a); break;
    case SJHIP_BF16: hipLaunchKernelGGL((mp_forward_kernel<ST, bf16_t>), grid, threads, lds, stream, a); break;
    default: return fail(SJHIP_ERR_INVALID, "forward(mp): spike dtype %d", spike_dtype);
  }
  return check_launch("forward(mp)");
}

}  // namespace

int launch_forward_mp(int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                      const void *x_seq, const void *v_init, const float *k_device, void *spike_seq, void *v_seq,
                      void *v_last, void *h_seq, hipStream_t stream) {
  if (N % 4 != 0) return fail(SJHIP_ERR_UNSUPPORTED, "forward(mp): N=%lld must be a multiple of 4", (long long)N);
  FwdArgs a;
  bool round_each = false;
  // scalars as for fp32 storage: the recurrence is the fp32 one
  int rc = build_fwd_args(a, round_each, neuron, SJHIP_F32, p, T, N, x_seq, v_init, k_device, spike_seq, v_seq, v_last, h_seq);
  if (rc != SJHIP_OK) return rc;
  if (!mp_aligned({x_seq, spike_seq, v_seq, v_last, h_seq}) || (!a.v_init_broadcast && !aligned16(v_init)))
    return fail(SJHIP_ERR_INVALID, "forward(mp): every tensor must be 16-byte aligned");
  const int block = tuning().fwd_block;
  const int64_t blocks = mp_blocks(N, block);
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "forward(mp): N=%lld", (long long)N);
  ProfileScope prof(KC_FORWARD, stream);
  if (storage_dtype == SJHIP_F8E4M3) return launch_fwd_storage<f8e4m3_t>(spike_dtype, a, dim3((unsigned)blocks), dim3(block), stream);
  if (storage_dtype == SJHIP_F8E5M2) return launch_fwd_storage<f8e5m2_t>(spike_dtype, a, dim3((unsigned)blocks), dim3(block), stream);
  return fail(SJHIP_ERR_INVALID, "forward(mp): storage dtype %d is not an 8-bit float", storage_dtype);
}

}  // namespace sjhip
