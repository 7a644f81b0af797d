// Multi-step backward (BPTT) for IF / LIF / PLIF with the surrogate gradient inlined.
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
#pragma once

#include "sjhip_common.h"

#ifndef SJHIP_BWD_PF
#define SJHIP_BWD_PF 8
#endif
#ifndef SJHIP_BWD_NT
#define SJHIP_BWD_NT 1
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
};

template <int SG> __device__ __forceinline__ float surrogate_grad(float x, float alpha) {
  if (SG == SJHIP_SG_SIGMOID) {
    // surrogate.py:769-771:  s = sigmoid(alpha x);  (1 - s) s alpha
    float s = 1.0f / (1.0f + expf(-alpha * x));
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
    return 0.5f * alpha * expf(-alpha * fabsf(x));
  } else if (SG == SJHIP_SG_SOFT_SIGN) {
    // surrogate.py:936-937:  1 / (2 alpha (1/alpha + |x|)^2)
    float d = 1.0f / alpha + fabsf(x);
    return 1.0f / (2.0f * alpha * d * d);
  } else if (SG == SJHIP_SG_SUPER_SPIKE) {
    // surrogate.py:1101-1102:  alpha / (|x| + 1)^2
    float d = fabsf(x) + 1.0f;
    return alpha / (d * d);
  } else {
    // surrogate.py:1610-1613:  alpha/sqrt(pi) exp(-(alpha x)^2)
    float ax = x * alpha;
    return 0.56418958354775628695f * alpha * expf(-(ax * ax));
  }
}

template <typename S, bool VECTOR, bool PLIF, int SG, bool GVFULL>
__device__ __forceinline__ float backward_body(const BwdArgs &a, bool active, int64_t col, float k) {
  typedef Acc<S, VECTOR, SJHIP_BWD_NT != 0> A;
  typedef typename A::elem_t E;
  constexpr int V = A::V;
  constexpr int PF = SJHIP_BWD_PF;

  float acc_total = 0.0f;
  if (!active) return acc_total;

  const int64_t N = a.N, T = a.T;
  const E *gsp = (const E *)a.grad_spike + col;
  const E *hp = (const E *)a.h + col;
  const E *gvp = GVFULL ? (const E *)a.grad_v_seq + col : nullptr;
  E *gxp = (E *)a.grad_x + col;

  const float kx = a.is_if ? 1.0f : (a.decay_input ? k : 1.0f);
  const float km = a.is_if ? 1.0f : (1.0f - k);
  const float v_th = a.v_th, alpha = a.alpha, cB = a.cB, cC = a.cC, cD = a.cD;

  typename A::raw_t ahead_gs[PF], ahead_h[PF], ahead_gv[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) {
    const int64_t t = T - 1 - i;
    ahead_gs[i] = (t >= 0) ? A::load(gsp + t * N) : A::zero();
    ahead_h[i] = (t >= 0) ? A::load(hp + t * N) : A::zero();
    if (GVFULL) ahead_gv[i] = (t >= 0) ? A::load(gvp + t * N) : A::zero();
  }

  float carry[V];
  if (a.grad_v_last) {
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
      cur_h[i] = ahead_h[i];
      if (GVFULL) cur_gv[i] = ahead_gv[i];
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 - PF - i;
      if (tn >= 0) {
        ahead_gs[i] = A::load(gsp + tn * N);
        ahead_h[i] = A::load(hp + tn * N);
        if (GVFULL) ahead_gv[i] = A::load(gvp + tn * N);
      }
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 - i;
      if (t >= 0) {
        float gs[V], h[V], gv[V], gx[V];
        A::unpack(cur_gs[i], gs);
        A::unpack(cur_h[i], h);
        if (GVFULL) A::unpack(cur_gv[i], gv);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float over = h[j] - v_th;
          const float sg = surrogate_grad<SG>(over, alpha);
          const float s = (over >= 0.0f) ? 1.0f : 0.0f;
          if (PLIF) {
            // v_t from h_t exactly as the forward wrote it
            const float v_t = a.soft_reset ? (h[j] - s * v_th) : (s * a.v_reset + (1.0f - s) * h[j]);
            const float dh_dk = a.decay_input ? (h_next[j] - v_t) : (a.v_reset - v_t);
            acc[j] += g_next[j] * dh_dk;  // g_next is 0 on the first processed step
          }
          const float dvdh = (1.0f - s * cB) + (cC - h[j] * cD) * sg;
          const float gvt = GVFULL ? carry[j] + gv[j] : carry[j];
          const float G = gvt * dvdh + gs[j] * sg;
          gx[j] = G * kx;
          carry[j] = G * km;
          if (PLIF) { g_next[j] = G; h_next[j] = h[j]; }
        }
        A::store(gxp + t * N, gx);
      }
    }
  }
  A::store((E *)a.grad_v_init + col, carry);
  if (PLIF) {
    float v0[V];
    A::unpack(A::load((const E *)a.v_init + col), v0);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const float dh_dk = a.decay_input ? (h_next[j] - v0[j]) : (a.v_reset - v0[j]);
      acc[j] += g_next[j] * dh_dk;
      acc_total += acc[j];
    }
  }
  return acc_total;
}

template <typename S, bool VECTOR, bool PLIF, int SG>
__device__ __forceinline__ float backward_gv_dispatch(const BwdArgs &a, bool active, int64_t col, float k) {
  if (a.grad_v_seq) return backward_body<S, VECTOR, PLIF, SG, true>(a, active, col, k);
  return backward_body<S, VECTOR, PLIF, SG, false>(a, active, col, k);
}

template <typename S, bool VECTOR, bool PLIF>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) backward_kernel(const BwdArgs a) {
  constexpr int V = Acc<S, VECTOR, true>::V;
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  const bool active = col < a.N;
  const float k = a.k_device ? *a.k_device : a.k;
  float part;
  switch (a.sg) {
    case SJHIP_SG_SIGMOID: part = backward_gv_dispatch<S, VECTOR, PLIF, SJHIP_SG_SIGMOID>(a, active, col, k); break;
    case SJHIP_SG_ATAN: part = backward_gv_dispatch<S, VECTOR, PLIF, SJHIP_SG_ATAN>(a, active, col, k); break;
    case SJHIP_SG_PIECEWISE_QUADRATIC: part = backward_gv_dispatch<S, VECTOR, PLIF, SJHIP_SG_PIECEWISE_QUADRATIC>(a, active, col, k); break;
    case SJHIP_SG_PIECEWISE_EXP: part = backward_gv_dispatch<S, VECTOR, PLIF, SJHIP_SG_PIECEWISE_EXP>(a, active, col, k); break;
    case SJHIP_SG_SOFT_SIGN: part = backward_gv_dispatch<S, VECTOR, PLIF, SJHIP_SG_SOFT_SIGN>(a, active, col, k); break;
    case SJHIP_SG_SUPER_SPIKE: part = backward_gv_dispatch<S, VECTOR, PLIF, SJHIP_SG_SUPER_SPIKE>(a, active, col, k); break;
    default: part = backward_gv_dispatch<S, VECTOR, PLIF, SJHIP_SG_ERF>(a, active, col, k); break;
  }
  if (PLIF) {
    // wavefront (64 lanes) shuffle reduction, then one value per wavefront through LDS
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
}

// Fixed-order final sum of the per-block partials: lane i adds partials[i], [i+1024], ... in fp64,
// then a binary tree over the 1024 lanes through LDS.  Same order on every run.
__global__ void __launch_bounds__(1024) plif_reduce_kernel(const float *partials, int64_t count,
                                                            const float *k_device, float k_host,
                                                            int decay_input, float *out) {
  __shared__ double tree[1024];
  double sum = 0.0;
  for (int64_t i = threadIdx.x; i < count; i += 1024) sum += (double)partials[i];
  tree[threadIdx.x] = sum;
  __syncthreads();
  for (int stride = 512; stride > 0; stride >>= 1) {
    if ((int)threadIdx.x < stride) tree[threadIdx.x] += tree[threadIdx.x + stride];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    double total = tree[0];
    if (decay_input) total /= (double)(k_device ? *k_device : k_host);
    out[0] = (float)total;
  }
}

}  // namespace sjhip
