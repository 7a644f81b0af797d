// Host launcher of the multi-step backward kernels and of the PLIF dL/dk reduction.
#include "neuron_bwd.h"

#include <cmath>

namespace sjhip {

namespace {

template <typename S>
int launch_typed(BwdArgs &a, bool vector, bool plif, float *grad_k_out, hipStream_t stream) {
  const int block = tuning().bwd_block;
  const int V = vector ? Acc<S, true, true>::V : 1;
  const int64_t items = (a.N + V - 1) / V;
  const int64_t blocks = (items + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "backward: N=%lld needs %lld blocks", (long long)a.N, (long long)blocks);
  const dim3 grid((unsigned)blocks), threads(block);
  const unsigned lds = occupancy_cap_lds(tuning().bwd_blocks_per_cu);
  {
    ProfileScope prof(KC_BACKWARD, stream);
    if (plif) {
      if (vector) hipLaunchKernelGGL((backward_kernel<S, true, true>), grid, threads, lds, stream, a);
      else hipLaunchKernelGGL((backward_kernel<S, false, true>), grid, threads, lds, stream, a);
    } else {
      if (vector) hipLaunchKernelGGL((backward_kernel<S, true, false>), grid, threads, lds, stream, a);
      else hipLaunchKernelGGL((backward_kernel<S, false, false>), grid, threads, lds, stream, a);
    }
    int rc = check_launch("backward");
    if (rc != SJHIP_OK) return rc;
  }
  if (plif && !a.atomic_reduce) {
    ProfileScope prof(KC_PLIF_REDUCE, stream);
    hipLaunchKernelGGL(plif_reduce_kernel, dim3(1), dim3(1024), 0, stream, (const float *)a.partials, blocks,
                       a.k_device, a.k, a.decay_input, grad_k_out);
    return check_launch("plif_reduce");
  }
  return SJHIP_OK;
}

}  // namespace

int64_t plif_blocks(int dtype, int64_t N) {
  (void)dtype;
  // upper bound for every block size (>= 64 lanes) and access width the launcher may pick
  return (N + 63) / 64;
}

int launch_backward(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                    const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                    const void *h_seq, const void *v_init,
                    const float *k_device, void *grad_x_seq, void *grad_v_init, float *grad_rtau,
                    float *workspace, hipStream_t stream) {
  BwdArgs a;
  a.grad_spike = grad_spike_seq; a.grad_v_seq = grad_v_seq; a.grad_v_last = grad_v_last; a.h = h_seq; a.v_init = v_init;
  a.k_device = nullptr;
  a.grad_x = grad_x_seq; a.grad_v_init = grad_v_init;
  a.partials = workspace; a.grad_k = grad_rtau;
  a.T = T; a.N = N;
  a.v_th = p.v_threshold; a.v_reset = p.v_reset; a.alpha = p.sg_alpha;
  a.sg = p.sg_id;
  a.soft_reset = (p.flags & SJHIP_FLAG_SOFT_RESET) ? 1 : 0;
  a.decay_input = (p.flags & SJHIP_FLAG_DECAY_INPUT) ? 1 : 0;
  a.is_if = neuron == SJHIP_NEURON_IF;
  a.atomic_reduce = (p.flags & SJHIP_FLAG_ATOMIC_REDUCE) ? 1 : 0;
  const bool detach = (p.flags & SJHIP_FLAG_DETACH_RESET) != 0;
  if (a.soft_reset) { a.cB = 0.0f; a.cC = detach ? 0.0f : -p.v_threshold; a.cD = 0.0f; }
  else { a.cB = 1.0f; a.cC = detach ? 0.0f : p.v_reset; a.cD = detach ? 0.0f : 1.0f; }

  const bool plif = neuron == SJHIP_NEURON_PLIF;
  if (neuron == SJHIP_NEURON_IF) {
    a.k = 0.0f;
  } else if (plif) {
    a.k = p.tau;
    a.k_device = k_device;
  } else {
    if (!(p.tau > 0.0f) || !std::isfinite(p.tau)) return fail(SJHIP_ERR_INVALID, "backward: tau=%g", (double)p.tau);
    a.k = (float)(1.0 / (double)p.tau);
  }

  const int esize = dtype == SJHIP_F32 ? 4 : 2;
  const int V = 16 / esize;
  const bool vector = (N % V == 0) && aligned16(grad_spike_seq) && aligned16(h_seq) && aligned16(grad_x_seq) &&
                      aligned16(grad_v_init) && (grad_v_seq == nullptr || aligned16(grad_v_seq)) &&
                      (grad_v_last == nullptr || aligned16(grad_v_last)) &&
                      (v_init == nullptr || aligned16(v_init));

  switch (dtype) {
    case SJHIP_F32: return launch_typed<float>(a, vector, plif, grad_rtau, stream);
    case SJHIP_F16: return launch_typed<f16_t>(a, vector, plif, grad_rtau, stream);
    case SJHIP_BF16: return launch_typed<bf16_t>(a, vector, plif, grad_rtau, stream);
    default: return fail(SJHIP_ERR_INVALID, "backward: dtype %d", dtype);
  }
}

}  // namespace sjhip
