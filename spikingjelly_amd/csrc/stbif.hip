// ST-BIF: the signed ternary integrate-and-fire neuron of SpikeZIP (QANN -> SNN conversion), inference only.
//
// Reference: functional/neuron.py:3234-3247 (stbif_step, the torch backend) and
// triton_kernel/neuron_kernel/stbif.py:94-137 (multi-step kernel).  Per step, with the quantiser scale s and the
// accumulator bounds [neg_min, pos_max]:
//     n   = x / s                       q = q + n                acc = round(acc)
//     pos = (q - 1 >= 0) & (acc < pos_max)        neg = (q < 0) & (acc > neg_min)
//     cur = pos - neg                    acc = acc + cur
//     q   = pos ? q - 1 : q              q = neg ? q + 1 : q      out = cur * s
// q carries the quantisation residual (it starts from 0.5, which makes the released total round to nearest), acc the
// integer released so far; out is -s, 0 or +s.  The work flag is set when any input or any output of the call is
// non-zero (the module's `is_work`, neuron/spikezip.py:311, 345).
//
// Same ownership as the neuron forward: one work-item owns V consecutive neurons, walks the T rows with q, acc and
// cur in registers and requests rows of x ahead of their use.  Per neuron-step it reads x and writes out: 2 x
// sizeof(dtype) bytes.  The scale and the bounds are read from device memory (one fp32 each), so a module whose
// buffers live on the device needs no host synchronisation to launch (the reference's Triton path calls .item() on
// each of them, stbif.py:360-362).
//
// Arithmetic: every op in torch's order with contraction off.  With 16-bit storage either every op result is rounded
// to the storage dtype (torch backend on half tensors: the three scalars are rounded to it first, x / s and cur * s
// are fp32 operations on the rounded values, rounded once more) or, with SJHIP_FLAG_FP32_STATE, the scalars are
// rounded to the storage dtype and everything else stays fp32 until it is stored (the Triton kernel).
#include "sjhip_common.h"

#ifndef SJHIP_STBIF_PF
#define SJHIP_STBIF_PF 8
#endif

#ifndef SJHIP_STBIF_NT
#define SJHIP_STBIF_NT 1
#endif

namespace sjhip {

struct StbifArgs {
  const void *x;
  const void *q_init;
  const void *acc_init;
  const float *scale, *pos_max, *neg_min;  // device, one fp32 each
  void *out;
  void *q_final;
  void *acc_final;
  void *cur;
  int32_t *work_flag;  // may be null
  int64_t T, N;
  int q_broadcast, acc_broadcast;
};

template <typename S, bool VECTOR, bool ROUND_EACH>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) stbif_forward_kernel(const StbifArgs a) {
  typedef Acc<S, VECTOR, SJHIP_STBIF_NT != 0> A;  // one read and one write per element, nothing is reused: streaming policy
  typedef typename A::elem_t E;
  typedef typename std::conditional<ROUND_EACH, S, float>::type R;
  constexpr int V = A::V;
  constexpr int PF = SJHIP_STBIF_PF;

  const int64_t N = a.N, T = a.T;
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  bool work = false;
  if (col < N) {
    const E *xp = (const E *)a.x + col;
    E *op = (E *)a.out + col;
    // `.to(x)` of the three scalars
    const float s = Cvt<S>::round(*a.scale), pmax = Cvt<S>::round(*a.pos_max), nmin = Cvt<S>::round(*a.neg_min);

    typename A::raw_t ahead[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) ahead[i] = (i < T) ? A::load(xp + (int64_t)i * N) : A::zero();

    float q[V], acc[V], cur[V];
    load_state<S, VECTOR, SJHIP_STBIF_NT != 0>(a.q_init, col, a.q_broadcast != 0, q);
    load_state<S, VECTOR, SJHIP_STBIF_NT != 0>(a.acc_init, col, a.acc_broadcast != 0, acc);
#pragma unroll
    for (int j = 0; j < V; ++j) cur[j] = 0.0f;

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
          float x[V], out[V];
          A::unpack(now[i], x);
#pragma unroll
          for (int j = 0; j < V; ++j) {
#pragma clang fp contract(off)
            const float n = Cvt<R>::round(x[j] / s);
            float qn = Cvt<R>::round(q[j] + n);
            float an = rintf(acc[j]);
            const float less = Cvt<R>::round(qn - 1.0f);
            const bool pos = (less >= 0.0f) && (an < pmax);
            const bool neg = (qn < 0.0f) && (an > nmin);
            cur[j] = (pos ? 1.0f : 0.0f) - (neg ? 1.0f : 0.0f);
            an = Cvt<R>::round(an + cur[j]);
            qn = pos ? less : qn;
            qn = neg ? Cvt<R>::round(qn + 1.0f) : qn;
            out[j] = Cvt<R>::round(cur[j] * s);
            work = work || (x[j] != 0.0f) || (out[j] != 0.0f);
            q[j] = qn;
            acc[j] = an;
          }
          A::store(op + t * N, out);
        }
      }
    }
    A::store((E *)a.q_final + col, q);
    A::store((E *)a.acc_final + col, acc);
    A::store((E *)a.cur + col, cur);
  }
  // one (vector) store per wavefront that saw work; the caller cleared the flag, every writer writes 1
  if (a.work_flag != nullptr && __ballot(work) != 0ull && (threadIdx.x & 63) == 0) *a.work_flag = 1;
}

namespace {

constexpr int kStbifBlocksPerCu = 4;

template <typename S>
int launch_typed(const StbifArgs &a, bool vector, bool round_each, hipStream_t stream) {
  const int block = tuning().fwd_block;
  const int V = vector ? Acc<S, true, false>::V : 1;
  const int64_t items = (a.N + V - 1) / V;
  const int64_t blocks = (items + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "stbif_forward: N=%lld needs %lld blocks", (long long)a.N, (long long)blocks);
  const dim3 grid((unsigned)blocks), threads(block);
  // Measured at T = 16, N = 33.5 M fp32 (block 128): four resident blocks per compute unit, i.e. two wavefronts per
  // SIMD, 0.80 ms; uncapped 0.86 ms; two blocks 1.19 ms.  Short sequences have fewer rows in flight per work-item
  // and get more blocks, as in the neuron forward.
  const int cap = a.T < 4 ? 0 : (a.T < 16 ? 2 * kStbifBlocksPerCu : kStbifBlocksPerCu);
  const unsigned lds = occupancy_cap_lds(cap);
  ProfileScope prof(KC_FORWARD, stream);
  if (vector) {
    if (round_each) hipLaunchKernelGGL((stbif_forward_kernel<S, true, true>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((stbif_forward_kernel<S, true, false>), grid, threads, lds, stream, a);
  } else {
    if (round_each) hipLaunchKernelGGL((stbif_forward_kernel<S, false, true>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((stbif_forward_kernel<S, false, false>), grid, threads, lds, stream, a);
  }
  return check_launch("stbif_forward");
}

}  // namespace

int launch_stbif_forward(int dtype, uint32_t flags, int64_t T, int64_t N, const void *x_seq, const void *q_init,
                         const void *acc_q_init, const float *q_threshold, const float *pos_max, const float *neg_min,
                         void *out_seq, void *q_final, void *acc_q_final, void *cur_output, int32_t *work_flag,
                         hipStream_t stream) {
  StbifArgs a;
  a.x = x_seq; a.q_init = q_init; a.acc_init = acc_q_init;
  a.scale = q_threshold; a.pos_max = pos_max; a.neg_min = neg_min;
  a.out = out_seq; a.q_final = q_final; a.acc_final = acc_q_final; a.cur = cur_output; a.work_flag = work_flag;
  a.T = T; a.N = N;
  a.q_broadcast = (flags & SJHIP_FLAG_Q_BROADCAST) ? 1 : 0;
  a.acc_broadcast = (flags & SJHIP_FLAG_ACC_BROADCAST) ? 1 : 0;
  const bool round_each = dtype != SJHIP_F32 && !(flags & SJHIP_FLAG_FP32_STATE);
  const int V = dtype == SJHIP_F32 ? 4 : 8;
  const bool vector = (N % V == 0) && aligned16(x_seq) && aligned16(out_seq) && aligned16(q_final) &&
                      aligned16(acc_q_final) && aligned16(cur_output) && (a.q_broadcast || aligned16(q_init)) &&
                      (a.acc_broadcast || aligned16(acc_q_init));
  switch (dtype) {
    case SJHIP_F32: return launch_typed<float>(a, vector, false, stream);
    case SJHIP_F16: return launch_typed<f16_t>(a, vector, round_each, stream);
    case SJHIP_BF16: return launch_typed<bf16_t>(a, vector, round_each, stream);
    default: return fail(SJHIP_ERR_INVALID, "stbif_forward: dtype %d", dtype);
  }
}

}  // namespace sjhip
