// Multi-step backward (BPTT) for IF / LIF / PLIF / QIF / ILIF with the surrogate gradient inlined.
//
// Same ownership as the forward: one work-item owns V consecutive neurons and walks the rows from
// t = T-1 down to 0 with the running gradient in registers.  Per step it reads grad_spike[t], h[t]
// (and grad_v_seq[t] when given) and writes grad_x[t]; spikes are recomputed from h.  Rows are requested
// SJHIP_BWD_PF steps before their use.
//
// Recurrence (reference: cuda_kernel/neuron_kernel/multi_step/base.py:293-409, lif.py:89-102,
// plif.py:143-203; equal to autograd through functional/neuron.py:225-228, 849-852, 1290-1297):
//   sg_t   = surrogate'(h_t - v_th)            s_t = [h_t >= v_th]
//   dvdh_t = hard: (1 - s_t) + [!detach] (v_reset - h_t) sg_t       soft: 1 - [!detach] v_th sg_t
//   G_t    = (carry_{t+1} + grad_v_seq[t]) dvdh_t + grad_spike[t] sg_t      carry_T = grad_v_last
//   grad_x[t] = G_t * (decay_input ? k : 1)      carry_t = G_t (1 - k)      grad_v_init = carry_0
// with k = 1/tau (LIF), sigmoid(w) (PLIF), and k = 0 / factor 1 for IF.
// PLIF adds dL/dk = sum_{t,n} G_t * dh_t/dk, dh_t/dk = (h_t - v_{t-1})/k (decay_input) or
// (v_reset - v_{t-1}); v_{t-1} is re-derived from h_{t-1} by the forward's own reset arithmetic, so
// no v_seq has to be stored or read.  The sum is reduced by wavefront shuffles, then through LDS,
// then either one fp32 partial per block (summed in a fixed order by plif_reduce_kernel, in fp64)
// or one atomicAdd per block.
// QIF (h_t = v_{t-1} + k (x_t + a0 (v_{t-1} - v_rest)(v_{t-1} - v_c)), cuda_kernel/neuron_kernel/multi_step/
// qif.py:138-277) has a state-dependent dh_{t+1}/dv_t = 1 + k a0 ((v_t - v_c) + (v_t - v_rest)); the carry then
// holds G_{t+1} itself and is scaled when step t has re-derived v_t from h_t; grad_v_init needs v_init.
// ILIF (triton_kernel/neuron_kernel/ilif.py:300-326, equal to autograd through functional/neuron.py:1097-1099 and
// quantize.py:594-598): z_t = h_t / v_th, w_t = [grad_min <= z_t <= grad_max], the count's derivative is w_t / v_th and
// its soft reset by c_t v_th gives dv_t/dh_t = 1 - [!detach] w_t, so
//   G_t = (carry_{t+1} + grad_v_seq[t]) (1 - [!detach] w_t) + grad_spike[t] w_t / v_th,   grad_x[t] = G_t.
// With every op rounded to a 16-bit storage dtype the window is tested on z_t rounded to it, as autograd does.
#pragma once

#include <cmath>

#include "sjhip_common.h"

#ifndef SJHIP_BWD_PF
#define SJHIP_BWD_PF 8
#endif
#ifndef SJHIP_BWD_PF16
#define SJHIP_BWD_PF16 4
#endif
#ifndef SJHIP_BWD_NT
#define SJHIP_BWD_NT 1
#endif
// policy of the grad_x stores alone (default: that of the loads)
#ifndef SJHIP_BWD_STORE_NT
#define SJHIP_BWD_STORE_NT SJHIP_BWD_NT
#endif
// policy of the x loads of the replay phase alone (default: that of the other loads)
#ifndef SJHIP_REPLAY_X_NT
#define SJHIP_REPLAY_X_NT SJHIP_BWD_NT
#endif

namespace sjhip {

struct BwdArgs {
  const void *grad_spike;
  const void *grad_v_seq;   // [T,N] or null
  const void *grad_v_last;  // [N] or null
  const void *h;
  const void *v_init;  // PLIF only
  const float *k_device;
  void *grad_x;
  void *grad_v_init;
  float *partials;     // PLIF, deterministic reduction: one float per block
  float *grad_k;       // PLIF, atomic reduction target
  int64_t T, N;
  float k;             // 1/tau, sigmoid(w) or 0
  float v_th, v_reset, alpha;
  // dvdh = (1 - s*cB) + (cC - h*cD) * sg : hard reset cB=1,cC=v_reset,cD=1; soft cB=0,cC=-v_th,cD=0;
  // detach_reset zeroes cC and cD.
  float cB, cC, cD;
  int sg;
  int soft_reset;
  int decay_input;
  int is_if;
  int atomic_reduce;
  int v_init_broadcast;  // v_init holds one element for all neurons
  float q_rest, q_c, q_a0;  // QIF, EIF
  int exponential;          // the state-dependent mode is EIF's, not QIF's
  float grad_min, grad_max; // ILIF: gradient window on h / v_th
  float vth_inv;            // ILIF: 1 / v_threshold when that is an exact power of two, else 0 (as in FwdArgs)
  float vth_rcp;            // ILIF: fl(1 / v_threshold), the factor of the count's gradient
  int detach_reset;
  int round_each;           // 16-bit storage with every op rounded
  int spread;               // block-to-column order, see column_block()
};

// Which extra terms the BPTT walk carries.
enum BwdMode { BWD_PLAIN = 0, BWD_PLIF = 1, BWD_QIF = 2 };
// Added to a BwdMode for short sequences: two rows in flight per work-item instead of eight.  The deep prefetch costs
// registers, i.e. resident wavefronts, and a wavefront with T rows has only T to ask for: at T <= 4 the bytes in flight
// per compute unit fall below what the memory latency needs (measured, replaying backward, fp32, GB/s of actual
// traffic with 8 / 2 rows: T = 1: 1.6 / 5.5, T = 2: 2.9 / 6.5, T = 4: 4.7 / 6.2, T = 8: 5.9 / 6.2 without and 6.2 / 6.0 with
// grad_v_seq; bf16 PLIF with fp32 state at T = 8, N = 8.4 M: 124 -> 110 us; at T = 16 four rows were already 2.5 % slower
// than eight).
constexpr int BWD_SHORT = 4;
#ifndef SJHIP_SHORT_ROWS
#define SJHIP_SHORT_ROWS 2
#endif
constexpr int kShortRows = SJHIP_SHORT_ROWS;
// sequences up to this length run the BWD_SHORT kernels
#ifndef SJHIP_SHORT_SEQUENCE
#define SJHIP_SHORT_SEQUENCE 8
#endif
constexpr int64_t kShortSequence = SJHIP_SHORT_SEQUENCE;
template <int MODE> struct BwdModeOf {
  static constexpr int BASE = MODE & 3;
  static constexpr bool SHORT = (MODE & BWD_SHORT) != 0;
};

// FAST (16-bit storage, where the result is rounded to 8 or 11 significant bits anyway) uses the hardware
// exp2 / reciprocal approximations (about 1 ulp each) in place of the correctly rounded library exp and IEEE
// division; fp32 storage keeps the latter.
template <bool FAST> __device__ __forceinline__ float sg_exp(float x) { return FAST ? __expf(x) : expf(x); }
template <bool FAST> __device__ __forceinline__ float sg_div(float a, float b) {
  return FAST ? a * __builtin_amdgcn_rcpf(b) : a / b;
}

template <int SG, bool FAST> __device__ __forceinline__ float surrogate_grad(float x, float alpha) {
#pragma clang fp contract(fast)
  if (SG == SJHIP_SG_SIGMOID) {
    // surrogate.py:769-771:  s = sigmoid(alpha x);  (1 - s) s alpha
    float s = sg_div<FAST>(1.0f, 1.0f + sg_exp<FAST>(-alpha * x));
    return (1.0f - s) * s * alpha;
  } else if (SG == SJHIP_SG_ATAN) {
    // surrogate.py:1247-1250:  a = alpha/2;  a / (1 + (pi a x)^2)
    float a = 0.5f * alpha;
    float ax = 3.14159265358979323846f * a * x;
    return __fdividef(a, 1.0f + ax * ax);
  } else if (SG == SJHIP_SG_PIECEWISE_QUADRATIC) {
    // surrogate.py:401-407:  0 where |x| > 1/alpha else alpha - alpha^2 |x|
    float ax = fabsf(x);
    return (ax > 1.0f / alpha) ? 0.0f : (alpha - alpha * alpha * ax);
  } else if (SG == SJHIP_SG_PIECEWISE_EXP) {
    // surrogate.py:595-596:  alpha/2 exp(-alpha |x|)
    return 0.5f * alpha * sg_exp<FAST>(-alpha * fabsf(x));
  } else if (SG == SJHIP_SG_SOFT_SIGN) {
    // surrogate.py:936-937:  1 / (2 alpha (1/alpha + |x|)^2)
    float d = 1.0f / alpha + fabsf(x);
    return sg_div<FAST>(1.0f, 2.0f * alpha * d * d);
  } else if (SG == SJHIP_SG_SUPER_SPIKE) {
    // surrogate.py:1101-1102:  alpha / (|x| + 1)^2
    float d = fabsf(x) + 1.0f;
    return sg_div<FAST>(alpha, d * d);
  } else {
    // surrogate.py:1610-1613:  alpha/sqrt(pi) exp(-(alpha x)^2)
    float ax = x * alpha;
    return 0.56418958354775628695f * alpha * sg_exp<FAST>(-(ax * ax));
  }
}

// v_t from h_t exactly as the forward wrote it (no fused multiply-add)
__device__ __forceinline__ float reset_as_forward(float h, float s, const BwdArgs &a) {
#pragma clang fp contract(off)
  return a.soft_reset ? (h - s * a.v_th) : (s * a.v_reset + (1.0f - s) * h);
}

// QIF / EIF: d h_{t+1} / d v_t.  EIF (h = v + k (x + v_rest - v + dT exp((v - theta) / dT)), cuda_kernel/neuron_kernel/
// multi_step/eif.py): 1 + k (exp((v - theta) / dT) - 1), with theta in q_c and dT in q_a0.
__device__ __forceinline__ float qif_dh_dv(float v, float k, const BwdArgs &a) {
#pragma clang fp contract(fast)
  if (a.exponential) return 1.0f + k * (__expf((v - a.q_c) / a.q_a0) - 1.0f);
  return 1.0f + k * a.q_a0 * ((v - a.q_c) + (v - a.q_rest));
}

// HLDS != 0: h_t does not come from h_seq in global memory but from LDS, where the recompute kernel
// (neuron_bwd_recompute.h) has left it.  HLDS == 1: as fp32, V/4 float4 per work-item and step, laid out
// [step][quarter][lane] so a wavefront reads consecutive 16-byte words.  HLDS == 2 (16-bit storage with every
// op rounded, where h is exactly a storage-dtype value): as eight 16-bit patterns in one 16-byte word, laid out
// [step][lane], half the LDS footprint.
// First PF rows (t = T-1 downwards) of grad_spike and grad_v_seq, requested ahead of their use.
template <typename S, bool VECTOR, bool SHORT = false> struct BwdPrologue {
  typedef Acc<S, VECTOR, SJHIP_BWD_NT != 0> A;
  static constexpr int PF = SHORT ? kShortRows : ((sizeof(S) == 2 && A::V == 8) ? SJHIP_BWD_PF16 : SJHIP_BWD_PF);
  typename A::raw_t gs[PF], gv[PF];
  __device__ __forceinline__ void load(const BwdArgs &a, int64_t col) {
    typedef typename A::elem_t E;
    const E *gsp = (const E *)a.grad_spike + col;
    const E *gvp = (const E *)a.grad_v_seq + col;
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = a.T - 1 - i;
      gs[i] = (t >= 0 && a.grad_spike) ? A::load(gsp + t * a.N) : A::zero();  // no spike gradient: zeros, nothing read
      if (a.grad_v_seq) gv[i] = (t >= 0) ? A::load(gvp + t * a.N) : A::zero();
    }
  }
};

// How the gradient with respect to the state enters and leaves a walk.  Ordinarily through memory (grad_v_last in,
// grad_v_init out).  A kernel that walks a sequence piece by piece keeps it in registers from one piece to the one
// before it: `regs` holds the work-item's V values; `from_regs` / `to_regs` say which side of this walk uses them.
struct StateGradient {
  float *regs = nullptr;
  bool from_regs = false, to_regs = false;
};

template <typename S, bool VECTOR, int MODE, int SG, bool GVFULL, int HLDS = 0>
__device__ __forceinline__ float backward_body(const BwdArgs &a, bool active, int64_t col, float k,
                                               const f32x4 *lds_h = nullptr,
                                               const BwdPrologue<S, VECTOR, BwdModeOf<MODE>::SHORT> *pre = nullptr,
                                               const StateGradient sgr = StateGradient()) {
  typedef Acc<S, VECTOR, SJHIP_BWD_NT != 0> A;
  typedef typename A::elem_t E;
  constexpr int V = A::V;
  constexpr int PF = BwdPrologue<S, VECTOR, BwdModeOf<MODE>::SHORT>::PF;
  constexpr bool PLIF = BwdModeOf<MODE>::BASE == BWD_PLIF;
  constexpr bool QIF = BwdModeOf<MODE>::BASE == BWD_QIF;

  float acc_total = 0.0f;
  if (!active) return acc_total;

  const int64_t N = a.N, T = a.T;
  const bool has_gs = a.grad_spike != nullptr;  // a loss on the membrane potential alone sends no spike gradient
  const E *gsp = (const E *)a.grad_spike + col;
  const E *hp = HLDS ? nullptr : (const E *)a.h + col;
  const E *gvp = GVFULL ? (const E *)a.grad_v_seq + col : nullptr;
  E *gxp = (E *)a.grad_x + col;

  const float kx = a.is_if ? 1.0f : (a.decay_input ? k : 1.0f);
  const float km = a.is_if ? 1.0f : (1.0f - k);
  const float v_th = a.v_th, alpha = a.alpha, cB = a.cB, cC = a.cC, cD = a.cD;

  typename A::raw_t ahead_gs[PF], ahead_h[PF], ahead_gv[PF];
  if (HLDS) {
    // the replay kernel requested these rows before it started recomputing h
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      ahead_gs[i] = pre->gs[i];
      if (GVFULL) ahead_gv[i] = pre->gv[i];
    }
  } else {
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = T - 1 - i;
      ahead_gs[i] = (t >= 0 && has_gs) ? A::load(gsp + t * N) : A::zero();
      ahead_h[i] = (t >= 0) ? A::load(hp + t * N) : A::zero();
      if (GVFULL) ahead_gv[i] = (t >= 0) ? A::load(gvp + t * N) : A::zero();
    }
  }

  float carry[V];
  if (sgr.from_regs) {
#pragma unroll
    for (int j = 0; j < V; ++j) carry[j] = sgr.regs[j];
  } else if (a.grad_v_last) {
    A::unpack(A::load((const E *)a.grad_v_last + col), carry);
  } else {
#pragma unroll
    for (int j = 0; j < V; ++j) carry[j] = 0.0f;
  }
  // PLIF: G and h of the step processed just before (t+1), pending their v_t
  float g_next[V], h_next[V], acc[V];
#pragma unroll
  for (int j = 0; j < V; ++j) { g_next[j] = 0.0f; h_next[j] = 0.0f; acc[j] = 0.0f; }

  for (int64_t t0 = T - 1; t0 >= 0; t0 -= PF) {
    typename A::raw_t cur_gs[PF], cur_h[PF], cur_gv[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      cur_gs[i] = ahead_gs[i];
      if (!HLDS) cur_h[i] = ahead_h[i];
      if (GVFULL) cur_gv[i] = ahead_gv[i];
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 - PF - i;
      if (tn >= 0) {
        if (has_gs) ahead_gs[i] = A::load(gsp + tn * N);
        if (!HLDS) ahead_h[i] = A::load(hp + tn * N);
        if (GVFULL) ahead_gv[i] = A::load(gvp + tn * N);
      }
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 - i;
      if (t >= 0) {
        float gs[V], h[V], gv[V], gx[V];
        A::unpack(cur_gs[i], gs);
        if (HLDS == 2) {
          typedef Acc<S, true, false> AH;
          if constexpr (AH::V == V && sizeof(S) == 2)
            AH::unpack(reinterpret_cast<const typename AH::raw_t *>(lds_h)[(int)t * (int)blockDim.x + (int)threadIdx.x], h);
        } else if (HLDS) {
#pragma unroll
          for (int q = 0; q < V / 4; ++q) {
            const f32x4 w = lds_h[((int)t * (V / 4) + q) * (int)blockDim.x + (int)threadIdx.x];
            h[4 * q] = w.x; h[4 * q + 1] = w.y; h[4 * q + 2] = w.z; h[4 * q + 3] = w.w;
          }
        } else {
          A::unpack(cur_h[i], h);
        }
        if (GVFULL) A::unpack(cur_gv[i], gv);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          if constexpr (SG == SJHIP_SG_MULTI_LEVEL) {
            float z;
            {
#pragma clang fp contract(off)
              // the forward's own quotient, so both agree on which side of the window it lies
              z = a.vth_inv != 0.0f ? h[j] * a.vth_inv : h[j] / v_th;
            }
            if (a.round_each) z = Cvt<S>::round(z);
            const bool inside = z >= a.grad_min && z <= a.grad_max;
            const float gvt = GVFULL ? carry[j] + gv[j] : carry[j];
            const float G = ((inside && !a.detach_reset) ? 0.0f : gvt) + (inside ? gs[j] * a.vth_rcp : 0.0f);
            gx[j] = G;
            carry[j] = G * km;
            continue;
          }
          const float over = h[j] - v_th;
          const float s = (over >= 0.0f) ? 1.0f : 0.0f;
          float v_t = 0.0f;
          if (PLIF || QIF) v_t = reset_as_forward(h[j], s, a);
          {
            // gradients carry a tolerance, not bit-exactness: let multiply-adds fuse here
#pragma clang fp contract(fast)
            const float sg = surrogate_grad<SG, sizeof(S) == 2>(over, alpha);
            if (PLIF) {
              const float dh_dk = a.decay_input ? (h_next[j] - v_t) : (a.v_reset - v_t);
              acc[j] += g_next[j] * dh_dk;  // g_next is 0 on the first processed step
            }
            const float dvdh = (1.0f - s * cB) + (cC - h[j] * cD) * sg;
            // QIF: the carry is G_{t+1}; its factor depends on v_t, known only now (grad_v_last enters unscaled)
            const float cin = (QIF && t != T - 1) ? carry[j] * qif_dh_dv(v_t, k, a) : carry[j];
            const float gvt = GVFULL ? cin + gv[j] : cin;
            const float G = gvt * dvdh + gs[j] * sg;
            gx[j] = G * kx;
            carry[j] = QIF ? G : G * km;
            if (PLIF) { g_next[j] = G; h_next[j] = h[j]; }
          }
        }
        Acc<S, VECTOR, SJHIP_BWD_STORE_NT != 0>::store(gxp + t * N, gx);
      }
    }
  }
  if (QIF) {
    if (a.grad_v_init || sgr.to_regs) {
      float v0[V];
      load_state_from<S, VECTOR, SJHIP_BWD_NT != 0>(a.v_init, col, a.v_init_broadcast, v0);
#pragma unroll
      for (int j = 0; j < V; ++j) carry[j] *= qif_dh_dv(v0[j], k, a);
      if (!sgr.to_regs) A::store((E *)a.grad_v_init + col, carry);
    }
  } else if (a.grad_v_init && !sgr.to_regs) {
    A::store((E *)a.grad_v_init + col, carry);
  }
  if (sgr.to_regs) {
#pragma unroll
    for (int j = 0; j < V; ++j) sgr.regs[j] = carry[j];
  }
  if (PLIF) {
    float v0[V];
    load_state_from<S, VECTOR, SJHIP_BWD_NT != 0>(a.v_init, col, a.v_init_broadcast, v0);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float dh_dk = a.decay_input ? (h_next[j] - v0[j]) : (a.v_reset - v0[j]);
      acc[j] += g_next[j] * dh_dk;
      acc_total += acc[j];
    }
  }
  return acc_total;
}

template <typename S, bool VECTOR, int MODE, int SG, int HLDS = 0>
__device__ __forceinline__ float backward_gv_dispatch(const BwdArgs &a, bool active, int64_t col, float k,
                                                      const f32x4 *lds_h = nullptr,
                                                      const BwdPrologue<S, VECTOR, BwdModeOf<MODE>::SHORT> *pre = nullptr,
                                                      const StateGradient sgr = StateGradient()) {
  if (a.grad_v_seq) return backward_body<S, VECTOR, MODE, SG, true, HLDS>(a, active, col, k, lds_h, pre, sgr);
  return backward_body<S, VECTOR, MODE, SG, false, HLDS>(a, active, col, k, lds_h, pre, sgr);
}

template <typename S, bool VECTOR, int MODE, int HLDS>
__device__ __forceinline__ float backward_sg_dispatch(const BwdArgs &a, bool active, int64_t col, float k,
                                                      const f32x4 *lds_h,
                                                      const BwdPrologue<S, VECTOR, BwdModeOf<MODE>::SHORT> *pre = nullptr,
                                                      const StateGradient sgr = StateGradient()) {
  switch (a.sg) {
    case SJHIP_SG_SIGMOID: return backward_gv_dispatch<S, VECTOR, MODE, SJHIP_SG_SIGMOID, HLDS>(a, active, col, k, lds_h, pre, sgr);
    case SJHIP_SG_ATAN: return backward_gv_dispatch<S, VECTOR, MODE, SJHIP_SG_ATAN, HLDS>(a, active, col, k, lds_h, pre, sgr);
    case SJHIP_SG_PIECEWISE_QUADRATIC: return backward_gv_dispatch<S, VECTOR, MODE, SJHIP_SG_PIECEWISE_QUADRATIC, HLDS>(a, active, col, k, lds_h, pre, sgr);
    case SJHIP_SG_PIECEWISE_EXP: return backward_gv_dispatch<S, VECTOR, MODE, SJHIP_SG_PIECEWISE_EXP, HLDS>(a, active, col, k, lds_h, pre, sgr);
    case SJHIP_SG_SOFT_SIGN: return backward_gv_dispatch<S, VECTOR, MODE, SJHIP_SG_SOFT_SIGN, HLDS>(a, active, col, k, lds_h, pre, sgr);
    case SJHIP_SG_SUPER_SPIKE: return backward_gv_dispatch<S, VECTOR, MODE, SJHIP_SG_SUPER_SPIKE, HLDS>(a, active, col, k, lds_h, pre, sgr);
    case SJHIP_SG_MULTI_LEVEL:
      if constexpr (BwdModeOf<MODE>::BASE == BWD_PLAIN) return backward_gv_dispatch<S, VECTOR, MODE, SJHIP_SG_MULTI_LEVEL, HLDS>(a, active, col, k, lds_h, pre, sgr);
      return 0.0f;
    default: return backward_gv_dispatch<S, VECTOR, MODE, SJHIP_SG_ERF, HLDS>(a, active, col, k, lds_h, pre, sgr);
  }
}

// Block-level sum of `part` (PLIF dL/dk): wavefront shuffles, then LDS, then one partial or atomic.
__device__ __forceinline__ void plif_block_reduce(const BwdArgs &a, float part, float k) {
  __shared__ float wave_sum[SJHIP_MAX_BLOCK / 64];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) part += __shfl_down(part, off, 64);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) wave_sum[wave] = part;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.0f;
    const int nwaves = (blockDim.x + 63) >> 6;
    for (int w = 0; w < nwaves; ++w) total += wave_sum[w];
    if (a.atomic_reduce) {
      if (a.decay_input) total = total / k;
      atomicAdd(a.grad_k, total);
    } else {
      a.partials[blockIdx.x] = total;
    }
  }
}

template <typename S, bool VECTOR, int MODE>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) backward_kernel(const BwdArgs a) {
  constexpr int V = Acc<S, VECTOR, true>::V;
  const int64_t col = ((int64_t)column_block(a.spread) * blockDim.x + threadIdx.x) * V;
  const bool active = col < a.N;
  const float k = a.k_device ? *a.k_device : a.k;
  const float part = backward_sg_dispatch<S, VECTOR, MODE, 0>(a, active, col, k, nullptr);
  if (BwdModeOf<MODE>::BASE == BWD_PLIF) plif_block_reduce(a, part, k);
}

// ---- host side: turn the ABI parameters into kernel arguments ------------------------------------
inline int build_bwd_args(BwdArgs &a, int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                          const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                          const void *h_seq, const void *v_init, const float *k_device, void *grad_x_seq,
                          void *grad_v_init, float *grad_rtau, float *workspace) {
  a.grad_spike = grad_spike_seq; a.grad_v_seq = grad_v_seq; a.grad_v_last = grad_v_last; a.h = h_seq; a.v_init = v_init;
  a.k_device = nullptr;
  a.grad_x = grad_x_seq; a.grad_v_init = grad_v_init;
  a.partials = workspace; a.grad_k = grad_rtau;
  a.T = T; a.N = N;
  a.spread = column_spread(N * (dtype == SJHIP_F32 ? 4 : 2), T);
  a.v_th = p.v_threshold; a.v_reset = p.v_reset; a.alpha = p.sg_alpha;
  a.sg = p.sg_id;
  a.soft_reset = (p.flags & SJHIP_FLAG_SOFT_RESET) ? 1 : 0;
  a.decay_input = (p.flags & SJHIP_FLAG_DECAY_INPUT) ? 1 : 0;
  a.is_if = neuron == SJHIP_NEURON_IF;
  a.atomic_reduce = (p.flags & SJHIP_FLAG_ATOMIC_REDUCE) ? 1 : 0;
  a.v_init_broadcast = (p.flags & SJHIP_FLAG_V_INIT_BROADCAST) ? 1 : 0;
  const bool detach = (p.flags & SJHIP_FLAG_DETACH_RESET) != 0;
  a.detach_reset = detach ? 1 : 0;
  a.round_each = (dtype != SJHIP_F32 && !(p.flags & SJHIP_FLAG_FP32_STATE)) ? 1 : 0;
  a.grad_min = p.grad_min; a.grad_max = p.grad_max;
  a.vth_rcp = 1.0f / p.v_threshold;
  a.vth_inv = (neuron == SJHIP_NEURON_ILIF && exact_reciprocal(p.v_threshold)) ? a.vth_rcp : 0.0f;
  if (neuron == SJHIP_NEURON_ILIF) { a.soft_reset = 1; a.decay_input = 0; }
  if (a.soft_reset) { a.cB = 0.0f; a.cC = detach ? 0.0f : -p.v_threshold; a.cD = 0.0f; }
  else { a.cB = 1.0f; a.cC = detach ? 0.0f : p.v_reset; a.cD = detach ? 0.0f : 1.0f; }

  const bool plif = neuron == SJHIP_NEURON_PLIF;
  a.q_rest = p.v_rest; a.q_c = p.v_c; a.q_a0 = p.a0;
  a.exponential = neuron == SJHIP_NEURON_EIF ? 1 : 0;
  if (neuron == SJHIP_NEURON_QIF || neuron == SJHIP_NEURON_EIF) a.decay_input = 1;  // grad_x = G k
  if (neuron == SJHIP_NEURON_IF) {
    a.k = 0.0f;
  } else if (plif) {
    a.k = p.tau;
    a.k_device = k_device;
  } else {
    if (!(p.tau > 0.0f) || !std::isfinite(p.tau)) return fail(SJHIP_ERR_INVALID, "backward: tau=%g", (double)p.tau);
    a.k = (float)(1.0 / (double)p.tau);
  }

  return SJHIP_OK;
}

int launch_plif_reduce(const BwdArgs &a, int64_t blocks, float *grad_k_out, hipStream_t stream);

}  // namespace sjhip
