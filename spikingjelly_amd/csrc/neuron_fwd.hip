// Host launcher of the multi-step forward kernels.
#include "neuron_fwd.h"

#include <cmath>

namespace sjhip {

namespace {

template <typename S, bool ROUND_EACH>
int launch_typed(const FwdArgs &a, bool vector, hipStream_t stream) {
  const int block = tuning().fwd_block;
  const int V = vector ? Acc<S, true, true>::V : 1;
  const int64_t items = (a.N + V - 1) / V;
  const int64_t blocks = (items + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "forward: N=%lld needs %lld blocks", (long long)a.N, (long long)blocks);
  const unsigned lds = occupancy_cap_lds(tuning().fwd_blocks_per_cu);
  ProfileScope prof(KC_FORWARD, stream);
  if (vector)
    hipLaunchKernelGGL((forward_kernel<S, true, ROUND_EACH>), dim3((unsigned)blocks), dim3(block), lds, stream, a);
  else
    hipLaunchKernelGGL((forward_kernel<S, false, ROUND_EACH>), dim3((unsigned)blocks), dim3(block), lds, stream, a);
  return check_launch("forward");
}

bool is_power_of_two(float f) {
  int e;
  return std::isfinite(f) && f > 0.0f && std::frexp(f, &e) == 0.5f;
}

}  // namespace

int launch_forward(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                   const void *x_seq, const void *v_init, const float *k_device, void *spike_seq,
                   void *v_seq, void *v_last, void *h_seq, hipStream_t stream) {
  FwdArgs a;
  a.x = x_seq; a.v_init = v_init; a.spike = spike_seq; a.v_seq = v_seq; a.v_last = v_last; a.h = h_seq;
  a.k_device = nullptr;
  a.T = T; a.N = N;
  a.soft_reset = (p.flags & SJHIP_FLAG_SOFT_RESET) ? 1 : 0;
  const bool decay_input = (p.flags & SJHIP_FLAG_DECAY_INPUT) != 0;
  const bool round_each = dtype != SJHIP_F32 && !(p.flags & SJHIP_FLAG_FP32_STATE);

  a.tau = p.tau;
  if (neuron == SJHIP_NEURON_IF) {
    a.charge = CH_IF;
  } else if (neuron == SJHIP_NEURON_PLIF) {
    a.charge = decay_input ? CH_DECAY_INPUT_MUL : CH_PLAIN_INPUT_MUL;
    a.k_device = k_device;
  } else {
    if (!(p.tau > 0.0f) || !std::isfinite(p.tau)) return fail(SJHIP_ERR_INVALID, "forward: tau=%g", (double)p.tau);
    if (p.flags & SJHIP_FLAG_RECIPROCAL_TAU) {
      // fl(1/tau) from the double quotient, as the reference kernels receive it (multi_step/lif.py:338)
      a.tau = (float)(1.0 / (double)p.tau);
      a.charge = decay_input ? CH_DECAY_INPUT_MUL : CH_PLAIN_INPUT_MUL;
    } else if (is_power_of_two(p.tau) && p.tau <= 0x1p100f && p.tau >= 0x1p-100f) {
      // x / 2^e == x * 2^-e bit for bit (both are exact scalings, subnormal results round identically)
      a.tau = 1.0f / p.tau;
      a.charge = decay_input ? CH_DECAY_INPUT_MUL : CH_PLAIN_INPUT_MUL;
    } else {
      a.charge = decay_input ? CH_DECAY_INPUT_DIV : CH_PLAIN_INPUT_DIV;
    }
  }

  // The torch CPU backend rounds a Python scalar to the tensor dtype before add/sub and keeps it in
  // fp32 for mul/div; mirror that when every op is rounded to a 16-bit storage dtype.
  a.vr_mul = p.v_reset;
  a.vth_mul = p.v_threshold;
  a.vr_add = p.v_reset;
  a.vth_sub = p.v_threshold;
  if (round_each) {
    if (dtype == SJHIP_F16) { a.vr_add = Cvt<f16_t>::round(p.v_reset); a.vth_sub = Cvt<f16_t>::round(p.v_threshold); }
    else { a.vr_add = Cvt<bf16_t>::round(p.v_reset); a.vth_sub = Cvt<bf16_t>::round(p.v_threshold); }
  }

  const int esize = dtype == SJHIP_F32 ? 4 : 2;
  const int V = 16 / esize;
  const bool vector = (N % V == 0) && aligned16(x_seq) && aligned16(v_init) && aligned16(spike_seq) &&
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
