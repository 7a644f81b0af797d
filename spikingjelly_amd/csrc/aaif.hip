// Activation-aware IF: an IF neuron with a per-channel (or scalar) firing threshold and membrane offset, inference only.
//
// Reference: functional/neuron.py:577-584 (activation_aware_if_step, the torch backend) and
// triton_kernel/neuron_kernel/activation_aware_if.py:44-93 (multi-step kernel).  Per step
//     h = v + x            s = [(h + offset_c) - threshold_c >= 0]
//     v = h - s * threshold_c   (soft reset)    or    s * v_reset + (1 - s) * h   (hard reset)
// where c = (n / inner_size) % channel_size is the channel of neuron n of the flattened time step.
//
// Same ownership as the neuron forward: one work-item owns V consecutive neurons, looks up their channels once, and
// walks the T rows with v in registers while rows of x are requested ahead of their use.  Thresholds and offsets are
// read from device memory as fp32 and rounded to the storage dtype first, like `.to(x)` in the reference.
#include "sjhip_common.h"

#ifndef SJHIP_AAIF_PF
#define SJHIP_AAIF_PF 8
#endif

#ifndef SJHIP_AAIF_NT
#define SJHIP_AAIF_NT 1
#endif

namespace sjhip {

struct AaifArgs {
  const void *x;
  const void *v_init;
  const float *threshold, *offset;  // device; one element or channel_size elements each
  void *spike;
  void *v_seq;   // may be null
  void *v_last;  // may be null
  int64_t T, N, channel_size, inner_size;
  float v_reset;
  int threshold_scalar, offset_scalar, soft_reset, v_init_broadcast;
};

template <typename S, bool VECTOR, bool ROUND_EACH>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) aaif_forward_kernel(const AaifArgs a) {
  typedef Acc<S, VECTOR, SJHIP_AAIF_NT != 0> A;  // one read and one write per element, nothing is reused: streaming policy
  typedef typename A::elem_t E;
  typedef typename std::conditional<ROUND_EACH, S, float>::type R;
  constexpr int V = A::V;
  constexpr int PF = sizeof(S) == 2 ? SJHIP_AAIF_PF / 2 : SJHIP_AAIF_PF;

  const int64_t N = a.N, T = a.T;
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (col >= N) return;

  const E *xp = (const E *)a.x + col;
  E *sp = (E *)a.spike + col;
  E *vp = a.v_seq ? (E *)a.v_seq + col : nullptr;

  typename A::raw_t ahead[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) ahead[i] = (i < T) ? A::load(xp + (int64_t)i * N) : A::zero();

  // Channel of the first neuron with one division pair (32-bit when N allows: a 64-bit division is a software loop
  // of more instructions than the whole walk over T); the neighbours follow by counting.
  float thr[V], off[V];
  int64_t within, c;
  if (N <= 0xffffffffLL) {
    const uint32_t inner = (uint32_t)a.inner_size, q = (uint32_t)col / inner;
    within = (uint32_t)col - q * inner;
    c = q % (uint32_t)a.channel_size;
  } else {
    const int64_t q = col / a.inner_size;
    within = col - q * a.inner_size;
    c = q % a.channel_size;
  }
#pragma unroll
  for (int j = 0; j < V; ++j) {
    thr[j] = Cvt<S>::round(a.threshold[a.threshold_scalar ? 0 : c]);
    off[j] = Cvt<S>::round(a.offset[a.offset_scalar ? 0 : c]);
    if (++within == a.inner_size) {
      within = 0;
      if (++c == a.channel_size) c = 0;
    }
  }
  const float reset_mul = a.v_reset;  // a Python scalar in torch: fp32 as a factor

  float v[V];
  load_state<S, VECTOR, SJHIP_AAIF_NT != 0>(a.v_init, col, a.v_init_broadcast != 0, v);

  for (int64_t t0 = 0; t0 < T; t0 += PF) {
    typename A::raw_t now[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) now[i] = ahead[i];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 + PF + i;
      if (tn < T) ahead[i] = A::load(xp + tn * N);
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 + i;
      if (t < T) {
        float x[V], s[V];
        A::unpack(now[i], x);
#pragma unroll
        for (int j = 0; j < V; ++j) {
#pragma clang fp contract(off)
          const float h = Cvt<R>::round(v[j] + x[j]);
          const float over = Cvt<R>::round(Cvt<R>::round(h + off[j]) - thr[j]);
          s[j] = (over >= 0.0f) ? 1.0f : 0.0f;
          if (a.soft_reset) {
            v[j] = Cvt<R>::round(h - Cvt<R>::round(s[j] * thr[j]));
          } else {
            const float m = Cvt<R>::round(s[j] * reset_mul);
            const float n = Cvt<R>::round(1.0f - s[j]);
            v[j] = Cvt<R>::round(m + Cvt<R>::round(n * h));
          }
        }
        A::store_spikes(sp + t * N, s);
        if (vp) A::store(vp + t * N, v);
      }
    }
  }
  if (a.v_last) A::store((E *)a.v_last + col, v);
}

namespace {

template <typename S>
int launch_typed(const AaifArgs &a, bool vector, bool round_each, hipStream_t stream) {
  const int block = tuning().fwd_block;
  const int V = vector ? Acc<S, true, false>::V : 1;
  const int64_t items = (a.N + V - 1) / V;
  const int64_t blocks = (items + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "aaif_forward: N=%lld needs %lld blocks", (long long)a.N, (long long)blocks);
  const dim3 grid((unsigned)blocks), threads(block);
  // the residency rule measured for the other one-read-one-write walk of this library (the ST-BIF kernel): four
  // resident blocks per compute unit at T >= 16, more for shorter sequences
  const unsigned lds = occupancy_cap_lds(a.T < 4 ? 0 : (a.T < 16 ? 8 : 4));
  ProfileScope prof(KC_FORWARD, stream);
  if (vector) {
    if (round_each) hipLaunchKernelGGL((aaif_forward_kernel<S, true, true>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((aaif_forward_kernel<S, true, false>), grid, threads, lds, stream, a);
  } else {
    if (round_each) hipLaunchKernelGGL((aaif_forward_kernel<S, false, true>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((aaif_forward_kernel<S, false, false>), grid, threads, lds, stream, a);
  }
  return check_launch("aaif_forward");
}

}  // namespace

int launch_aaif_forward(int dtype, uint32_t flags, int64_t T, int64_t N, const void *x_seq, const void *v_init,
                        const float *v_threshold, int64_t threshold_count, const float *v_offset, int64_t offset_count,
                        int64_t channel_size, int64_t inner_size, float v_reset, void *spike_seq, void *v_seq,
                        void *v_last, hipStream_t stream) {
  AaifArgs a;
  a.x = x_seq; a.v_init = v_init; a.threshold = v_threshold; a.offset = v_offset;
  a.spike = spike_seq; a.v_seq = v_seq; a.v_last = v_last;
  a.T = T; a.N = N; a.channel_size = channel_size; a.inner_size = inner_size;
  a.v_reset = v_reset;
  a.threshold_scalar = threshold_count == 1 ? 1 : 0;
  a.offset_scalar = offset_count == 1 ? 1 : 0;
  a.soft_reset = (flags & SJHIP_FLAG_SOFT_RESET) ? 1 : 0;
  a.v_init_broadcast = (flags & SJHIP_FLAG_V_INIT_BROADCAST) ? 1 : 0;
  const bool round_each = dtype != SJHIP_F32 && !(flags & SJHIP_FLAG_FP32_STATE);
  const int V = dtype == SJHIP_F32 ? 4 : 8;
  const bool vector = (N % V == 0) && aligned16(x_seq) && aligned16(spike_seq) && (v_seq == nullptr || aligned16(v_seq)) &&
                      (v_last == nullptr || aligned16(v_last)) && (a.v_init_broadcast || aligned16(v_init));
  switch (dtype) {
    case SJHIP_F32: return launch_typed<float>(a, vector, false, stream);
    case SJHIP_F16: return launch_typed<f16_t>(a, vector, round_each, stream);
    case SJHIP_BF16: return launch_typed<bf16_t>(a, vector, round_each, stream);
    default: return fail(SJHIP_ERR_INVALID, "aaif_forward: dtype %d", dtype);
  }
}

}  // namespace sjhip
