// Backward kernels of the 8-bit-storage mixed-precision neurons (see neuron_mp.h).
#include "neuron_mp.h"

namespace sjhip {

// BPTT over the stored (8-bit) h_seq; the recurrence and the PLIF sum are those of neuron_bwd.h.  grad_spike_seq is in
// the spike dtype, grad_v_seq / grad_v_last in the storage dtype; the results leave in GO: fp32, or the storage dtype
// (rounded once from the fp32 value, what a cast of the fp32 result gives; 5 instead of 8 bytes per neuron-step).
template <typename ST, typename SP, typename GO, int SG, bool PLIF>
__device__ __forceinline__ float mp_backward_walk(const BwdArgs &a, const MpLane &l, float k) {
  typedef Tile16<ST> RH;
  typedef Tile16<SP> RG;
  typedef Tile16<GO> RO;
  constexpr int V = 16, PF = SJHIP_MP_BWD_PF;
  const int64_t N = a.N, T = a.T;
  const float km = a.is_if ? 1.0f : 1.0f - k;
  const float kx = a.is_if ? 1.0f : (a.decay_input ? k : 1.0f);

  typename RG::raw_t ahead_gs[PF];
  typename RH::raw_t ahead_h[PF], ahead_gv[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) {
    const int64_t t = T - 1 - i;
    ahead_gs[i] = (t >= 0) ? RG::load(a.grad_spike, t * N, l) : RG::zero();
    ahead_h[i] = (t >= 0) ? RH::load(a.h, t * N, l) : RH::zero();
    if (a.grad_v_seq) ahead_gv[i] = (t >= 0) ? RH::load(a.grad_v_seq, t * N, l) : RH::zero();
  }
  float carry[V], acc[V], g_next[V], h_next[V];
#pragma unroll
  for (int j = 0; j < V; ++j) { carry[j] = 0.0f; acc[j] = 0.0f; g_next[j] = 0.0f; h_next[j] = 0.0f; }
  if (a.grad_v_last) RH::unpack(RH::load(a.grad_v_last, 0, l), carry);

  for (int64_t t0 = T - 1; t0 >= 0; t0 -= PF) {
    typename RG::raw_t cur_gs[PF];
    typename RH::raw_t cur_h[PF], cur_gv[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      cur_gs[i] = ahead_gs[i]; cur_h[i] = ahead_h[i];
      if (a.grad_v_seq) cur_gv[i] = ahead_gv[i];
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 - PF - i;
      if (tn >= 0) {
        ahead_gs[i] = RG::load(a.grad_spike, tn * N, l);
        ahead_h[i] = RH::load(a.h, tn * N, l);
        if (a.grad_v_seq) ahead_gv[i] = RH::load(a.grad_v_seq, tn * N, l);
      }
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 - i;
      if (t >= 0) {
        float gs[V], h[V], gv[V], gx[V];
        RG::unpack(cur_gs[i], gs);
        RH::unpack(cur_h[i], h);
#pragma unroll
        for (int j = 0; j < V; ++j) gv[j] = 0.0f;
        if (a.grad_v_seq) RH::unpack(cur_gv[i], gv);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float over = h[j] - a.v_th;
          const float s = (over >= 0.0f) ? 1.0f : 0.0f;
          const float sg = surrogate_grad<SG, false>(over, a.alpha);
          if (PLIF) {
            const float v_t = reset_as_forward(h[j], s, a);
            const float dh_dk = a.decay_input ? (h_next[j] - v_t) : (a.v_reset - v_t);
            acc[j] += g_next[j] * dh_dk;  // g_next is 0 on the first processed step
          }
          const float dvdh = (1.0f - s * a.cB) + (a.cC - h[j] * a.cD) * sg;
          const float G = (carry[j] + gv[j]) * dvdh + gs[j] * sg;
          gx[j] = G * kx;
          carry[j] = G * km;
          if (PLIF) { g_next[j] = G; h_next[j] = h[j]; }
        }
        RO::store(a.grad_x, t * N, l, gx);
      }
    }
  }
  if (a.grad_v_init) RO::store(a.grad_v_init, 0, l, carry);
  float total = 0.0f;
  if (PLIF) {
    float v0[V];
    if (a.v_init_broadcast) {
      const float b = Codec<ST>::dec(*(const uint8_t *)a.v_init);
#pragma unroll
      for (int j = 0; j < V; ++j) v0[j] = b;
    } else {
      RH::unpack(RH::load(a.v_init, 0, l), v0);
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float dh_dk = a.decay_input ? (h_next[j] - v0[j]) : (a.v_reset - v0[j]);
      acc[j] += g_next[j] * dh_dk;
      total += acc[j];
    }
  }
  return total;
}

template <typename ST, typename SP, typename GO, bool PLIF>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) mp_backward_kernel(const BwdArgs a) {
  const MpLane l = mp_lane(a.N);
  const float k = a.k_device ? *a.k_device : a.k;
  float part = 0.0f;
  if (l.groups != 0) {
    switch (a.sg) {
      case SJHIP_SG_SIGMOID: part = mp_backward_walk<ST, SP, GO, SJHIP_SG_SIGMOID, PLIF>(a, l, k); break;
      case SJHIP_SG_ATAN: part = mp_backward_walk<ST, SP, GO, SJHIP_SG_ATAN, PLIF>(a, l, k); break;
      case SJHIP_SG_PIECEWISE_QUADRATIC: part = mp_backward_walk<ST, SP, GO, SJHIP_SG_PIECEWISE_QUADRATIC, PLIF>(a, l, k); break;
      case SJHIP_SG_PIECEWISE_EXP: part = mp_backward_walk<ST, SP, GO, SJHIP_SG_PIECEWISE_EXP, PLIF>(a, l, k); break;
      case SJHIP_SG_SOFT_SIGN: part = mp_backward_walk<ST, SP, GO, SJHIP_SG_SOFT_SIGN, PLIF>(a, l, k); break;
      case SJHIP_SG_SUPER_SPIKE: part = mp_backward_walk<ST, SP, GO, SJHIP_SG_SUPER_SPIKE, PLIF>(a, l, k); break;
      default: part = mp_backward_walk<ST, SP, GO, SJHIP_SG_ERF, PLIF>(a, l, k); break;
    }
  }
  if (PLIF) plif_block_reduce(a, part, k);
}

namespace {

template <typename ST, typename GO, bool PLIF>
int launch_bwd_storage(int spike_dtype, const BwdArgs &a, dim3 grid, dim3 threads, hipStream_t stream) {
  // resident blocks per compute unit, measured at T = 16, N = 33.5 M (blocks of 128).  fp32 gradients: 6 blocks 0.810 ms,
  // no cap 0.845, 1-3 1.30; 8-bit gradients (less to write, closer to the arithmetic): 4 blocks 0.722, 6 0.631, 8 0.585,
  // no cap 0.583
  const unsigned lds = occupancy_cap_lds(sizeof(GO) == 4 ? 6 : 0);
  switch (spike_dtype) {
    case SJHIP_F32: hipLaunchKernelGGL((mp_backward_kernel<ST, float, GO, PLIF>), grid, threads, lds, stream, a); break;
    case SJHIP_F16: hipLaunchKernelGGL((mp_backward_kernel<ST, f16_t, GO, PLIF>), grid, threads, lds, stream, a); break;
    case SJHIP_BF16: hipLaunchKernelGGL((mp_backward_kernel<ST, bf16_t, GO, PLIF>), grid, threads, lds, stream, a); break;
    default: return fail(SJHIP_ERR_INVALID, "backward(mp): spike dtype %d", spike_dtype);
  }
  return check_launch("backward(mp)");
}

template <typename ST>
int launch_bwd_outputs(int spike_dtype, bool plif, bool grads_in_storage, const BwdArgs &a, dim3 grid, dim3 threads,
                       hipStream_t stream) {
  if (grads_in_storage)
    return plif ? launch_bwd_storage<ST, ST, true>(spike_dtype, a, grid, threads, stream)
                : launch_bwd_storage<ST, ST, false>(spike_dtype, a, grid, threads, stream);
  return plif ? launch_bwd_storage<ST, float, true>(spike_dtype, a, grid, threads, stream)
              : launch_bwd_storage<ST, float, false>(spike_dtype, a, grid, threads, stream);
}

}  // namespace

int launch_backward_mp(int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                       const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last, const void *h_seq,
                       const void *v_init, const float *k_device, void *grad_x_seq, void *grad_v_init,
                       float *grad_rtau, float *workspace, hipStream_t stream) {
  if (N % 4 != 0) return fail(SJHIP_ERR_UNSUPPORTED, "backward(mp): N=%lld must be a multiple of 4", (long long)N);
  BwdArgs a;
  int rc = build_bwd_args(a, neuron, SJHIP_F32, p, T, N, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, v_init, k_device,
                          grad_x_seq, grad_v_init, grad_rtau, workspace);
  if (rc != SJHIP_OK) return rc;
  const bool plif = neuron == SJHIP_NEURON_PLIF;
  if (!mp_aligned({grad_spike_seq, grad_v_seq, grad_v_last, h_seq, grad_x_seq, grad_v_init}) ||
      (plif && !a.v_init_broadcast && !aligned16(v_init)))
    return fail(SJHIP_ERR_INVALID, "backward(mp): every tensor must be 16-byte aligned");
  const int block = tuning().bwd_block;
  const int64_t blocks = mp_blocks(N, block);
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "backward(mp): N=%lld", (long long)N);
  const dim3 grid((unsigned)blocks), threads(block);
  {
    ProfileScope prof(KC_BACKWARD, stream);
    const bool grads_in_storage = (p.flags & SJHIP_FLAG_GRAD_STORAGE) != 0;
    if (storage_dtype == SJHIP_F8E4M3)
      rc = launch_bwd_outputs<f8e4m3_t>(spike_dtype, plif, grads_in_storage, a, grid, threads, stream);
    else if (storage_dtype == SJHIP_F8E5M2)
      rc = launch_bwd_outputs<f8e5m2_t>(spike_dtype, plif, grads_in_storage, a, grid, threads, stream);
    else
      return fail(SJHIP_ERR_INVALID, "backward(mp): storage dtype %d is not an 8-bit float", storage_dtype);
    if (rc != SJHIP_OK) return rc;
  }
  if (plif && !a.atomic_reduce) return launch_plif_reduce(a, blocks, grad_rtau, stream);
  return SJHIP_OK;
}

}  // namespace sjhip
