// Izhikevich neuron: a quadratic integrate-and-fire membrane v coupled to an adaptation current w.
//
// Reference: functional/neuron.py:1514-1522 (izhikevich_step, the torch backend) and the CuPy kernels of
// cuda_kernel/neuron_kernel/multi_step/izhikevich.py.  Per step, in torch's op order (contraction off):
//     h   = v + (x + a0 (v - v_rest) (v - v_c) - w) / tau
//     u   = w + (a (h - v_rest) - w) / tau_w
//     s   = [h - v_th >= 0]
//     v'  = h - s v_th   (soft reset)    or    (1 - s) h + s v_reset   (hard reset)
//     w'  = u + b s
//
// Backward (BPTT over two coupled states), with k = 1/tau, kw = 1/tau_w, sg_t = surrogate'(h_t - v_th):
//     gv_t  = grad_v_seq[t] + Gh_{t+1} (1 + k a0 ((v_t - v_c) + (v_t - v_rest)))        (t = T-1: grad_v_last)
//     gw_t  = grad_w_seq[t] + Gh_{t+1} (-k) + gw_{t+1} (1 - kw)                          (t = T-1: grad_w_last)
//     dvdh  = soft: 1 - [!detach] v_th sg_t      hard: (1 - s_t) + sg_t (v_reset - [!detach] h_t)
//     Gh_t  = gv_t dvdh + (grad_spike[t] + b gw_t) sg_t + gw_t kw a
//     grad_x[t] = Gh_t k;   grad_v_init = Gh_0 (1 + k a0 ((v_init - v_c) + (v_init - v_rest)));   grad_w_init = Gh_0 (-k) + gw_0 (1 - kw)
// In the hard reset the reference multiplies v_reset by the undetached spike, so that term keeps its gradient under
// detach_reset.  v_t is re-derived from h_t by the forward's reset arithmetic; w never enters a derivative.
//
// Same ownership as the other neuron kernels: one work-item owns V consecutive neurons and walks the rows with its
// states (forward) or running gradients (backward) in registers, rows requested ahead of their use.
#include "neuron_bwd.h"

#include <initializer_list>

#ifndef SJHIP_IZH_PF
#define SJHIP_IZH_PF 4
#endif

namespace sjhip {

struct IzhFwdArgs {
  const void *x, *v_init, *w_init;
  void *spike, *v_seq, *w_seq, *v_last, *w_last, *h;  // v_seq, w_seq, h may be null
  int64_t T, N;
  float tau, tau_w;            // divisor, or multiplier when the matching *_mul flag is set
  int tau_mul, tau_w_mul;
  float rest_sub, c_sub;       // v_rest, v_c as subtrahends (rounded to the storage dtype when every op is rounded)
  float a0, a, b;              // factors: fp32
  float vth_sub, vth_mul, vr_mul;
  int soft_reset, v_broadcast, w_broadcast;
};

struct IzhBwdArgs {
  const void *grad_spike, *grad_v_seq, *grad_w_seq, *grad_v_last, *grad_w_last, *h, *v_init;
  void *grad_x, *grad_v_init, *grad_w_init;
  int64_t T, N;
  float k, kw, a0, a, b, v_rest, v_c, v_th, v_reset, alpha;
  int sg, soft_reset, detach_reset, v_broadcast;
};

template <typename S, bool VECTOR, bool ROUND_EACH>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) izhikevich_forward_kernel(const IzhFwdArgs a) {
  typedef Acc<S, VECTOR, false> A;
  typedef typename A::elem_t E;
  typedef typename std::conditional<ROUND_EACH, S, float>::type R;
  constexpr int V = A::V;
  constexpr int PF = SJHIP_IZH_PF;

  const int64_t N = a.N, T = a.T;
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (col >= N) return;
  const E *xp = (const E *)a.x + col;

  typename A::raw_t ahead[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) ahead[i] = (i < T) ? A::load(xp + (int64_t)i * N) : A::zero();
  float v[V], w[V];
  load_state<S, VECTOR, false>(a.v_init, col, a.v_broadcast != 0, v);
  load_state<S, VECTOR, false>(a.w_init, col, a.w_broadcast != 0, w);

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
        float x[V], h[V], s[V];
        A::unpack(now[i], x);
#pragma unroll
        for (int j = 0; j < V; ++j) {
#pragma clang fp contract(off)
          const float d1 = Cvt<R>::round(v[j] - a.rest_sub);
          const float m1 = scalar_product<R>(a.a0, d1);
          const float d2 = Cvt<R>::round(v[j] - a.c_sub);
          const float m2 = Cvt<R>::round(m1 * d2);
          const float e = Cvt<R>::round(Cvt<R>::round(x[j] + m2) - w[j]);
          const float f = a.tau_mul ? scalar_product<R>(a.tau, e) : Cvt<R>::round(e / a.tau);
          h[j] = Cvt<R>::round(v[j] + f);
          const float p = Cvt<R>::round(h[j] - a.rest_sub);
          const float r = Cvt<R>::round(scalar_product<R>(a.a, p) - w[j]);
          const float u = a.tau_w_mul ? scalar_product<R>(a.tau_w, r) : Cvt<R>::round(r / a.tau_w);
          const float wn = Cvt<R>::round(w[j] + u);
          const float over = Cvt<R>::round(h[j] - a.vth_sub);
          s[j] = (over >= 0.0f) ? 1.0f : 0.0f;
          if (a.soft_reset) {
            v[j] = Cvt<R>::round(h[j] - scalar_product<R>(a.vth_mul, s[j]));
          } else {
            const float keep = Cvt<R>::round(Cvt<R>::round(1.0f - s[j]) * h[j]);
            v[j] = Cvt<R>::round(keep + scalar_product<R>(a.vr_mul, s[j]));
          }
          w[j] = Cvt<R>::round(wn + scalar_product<R>(a.b, s[j]));
        }
        A::store_spikes((E *)a.spike + col + t * N, s);
        if (a.h) A::store((E *)a.h + col + t * N, h);
        if (a.v_seq) A::store((E *)a.v_seq + col + t * N, v);
        if (a.w_seq) A::store((E *)a.w_seq + col + t * N, w);
      }
    }
  }
  A::store((E *)a.v_last + col, v);
  A::store((E *)a.w_last + col, w);
}

__device__ __forceinline__ float surrogate_grad_any(int sg, float x, float alpha) {
  switch (sg) {
    case SJHIP_SG_SIGMOID: return surrogate_grad<SJHIP_SG_SIGMOID, false>(x, alpha);
    case SJHIP_SG_ATAN: return surrogate_grad<SJHIP_SG_ATAN, false>(x, alpha);
    case SJHIP_SG_PIECEWISE_QUADRATIC: return surrogate_grad<SJHIP_SG_PIECEWISE_QUADRATIC, false>(x, alpha);
    case SJHIP_SG_PIECEWISE_EXP: return surrogate_grad<SJHIP_SG_PIECEWISE_EXP, false>(x, alpha);
    case SJHIP_SG_SOFT_SIGN: return surrogate_grad<SJHIP_SG_SOFT_SIGN, false>(x, alpha);
    case SJHIP_SG_SUPER_SPIKE: return surrogate_grad<SJHIP_SG_SUPER_SPIKE, false>(x, alpha);
    default: return surrogate_grad<SJHIP_SG_ERF, false>(x, alpha);
  }
}

template <typename S, bool VECTOR>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) izhikevich_backward_kernel(const IzhBwdArgs a) {
  typedef Acc<S, VECTOR, true> A;
  typedef typename A::elem_t E;
  constexpr int V = A::V;
  constexpr int PF = SJHIP_IZH_PF;

  const int64_t N = a.N, T = a.T;
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (col >= N) return;
  const E *gsp = (const E *)a.grad_spike + col;
  const E *hp = (const E *)a.h + col;
  const E *gvp = a.grad_v_seq ? (const E *)a.grad_v_seq + col : nullptr;
  const E *gwp = a.grad_w_seq ? (const E *)a.grad_w_seq + col : nullptr;

  typename A::raw_t ahead_gs[PF], ahead_h[PF], ahead_gv[PF], ahead_gw[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) {
    const int64_t t = T - 1 - i;
    ahead_gs[i] = (t >= 0) ? A::load(gsp + t * N) : A::zero();
    ahead_h[i] = (t >= 0) ? A::load(hp + t * N) : A::zero();
    if (gvp) ahead_gv[i] = (t >= 0) ? A::load(gvp + t * N) : A::zero();
    if (gwp) ahead_gw[i] = (t >= 0) ? A::load(gwp + t * N) : A::zero();
  }

  float gh_next[V], cw_next[V], gv_last[V];
#pragma unroll
  for (int j = 0; j < V; ++j) { gh_next[j] = 0.0f; cw_next[j] = 0.0f; gv_last[j] = 0.0f; }
  if (a.grad_v_last) A::unpack(A::load((const E *)a.grad_v_last + col), gv_last);
  if (a.grad_w_last) A::unpack(A::load((const E *)a.grad_w_last + col), cw_next);

  const float k = a.k, kw = a.kw;
  for (int64_t t0 = T - 1; t0 >= 0; t0 -= PF) {
    typename A::raw_t cur_gs[PF], cur_h[PF], cur_gv[PF], cur_gw[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      cur_gs[i] = ahead_gs[i]; cur_h[i] = ahead_h[i];
      if (gvp) cur_gv[i] = ahead_gv[i];
      if (gwp) cur_gw[i] = ahead_gw[i];
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 - PF - i;
      if (tn >= 0) {
        ahead_gs[i] = A::load(gsp + tn * N);
        ahead_h[i] = A::load(hp + tn * N);
        if (gvp) ahead_gv[i] = A::load(gvp + tn * N);
        if (gwp) ahead_gw[i] = A::load(gwp + tn * N);
      }
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 - i;
      if (t >= 0) {
        float gs[V], h[V], gvs[V], gws[V], gx[V];
        A::unpack(cur_gs[i], gs);
        A::unpack(cur_h[i], h);
        if (gvp) A::unpack(cur_gv[i], gvs);
        if (gwp) A::unpack(cur_gw[i], gws);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float over = h[j] - a.v_th;
          const float s = (over >= 0.0f) ? 1.0f : 0.0f;
          float v_t;
          {
#pragma clang fp contract(off)
            v_t = a.soft_reset ? (h[j] - s * a.v_th) : ((1.0f - s) * h[j] + s * a.v_reset);
          }
          const float sg = surrogate_grad_any(a.sg, over, a.alpha);
          const float dhdv = 1.0f + k * a.a0 * ((v_t - a.v_c) + (v_t - a.v_rest));
          float gv = (t == T - 1) ? gv_last[j] : gh_next[j] * dhdv;
          if (gvp) gv += gvs[j];
          float gw = cw_next[j];  // grad_w_last at t = T-1
          if (gwp) gw += gws[j];
          const float live = a.detach_reset ? 0.0f : 1.0f;
          const float dvdh = a.soft_reset ? (1.0f - live * a.v_th * sg) : ((1.0f - s) + sg * (a.v_reset - live * h[j]));
          const float gh = gv * dvdh + (gs[j] + a.b * gw) * sg + gw * kw * a.a;
          gx[j] = gh * k;
          gh_next[j] = gh;
          cw_next[j] = gw * (1.0f - kw) - gh * k;
        }
        A::store((E *)a.grad_x + col + t * N, gx);
      }
    }
  }
  if (a.grad_v_init) {
    float v0[V];
    load_state<S, VECTOR, true>(a.v_init, col, a.v_broadcast != 0, v0);
#pragma unroll
    for (int j = 0; j < V; ++j) gh_next[j] *= 1.0f + k * a.a0 * ((v0[j] - a.v_c) + (v0[j] - a.v_rest));
    A::store((E *)a.grad_v_init + col, gh_next);
  }
  if (a.grad_w_init) A::store((E *)a.grad_w_init + col, cw_next);
}

namespace {

template <typename S>
int launch_fwd_typed(const IzhFwdArgs &a, bool vector, bool round_each, hipStream_t stream) {
  const int block = tuning().fwd_block;
  const int V = vector ? Acc<S, true, false>::V : 1;
  const int64_t blocks = ((a.N + V - 1) / V + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "izhikevich_forward: N=%lld", (long long)a.N);
  const dim3 grid((unsigned)blocks), threads(block);
  // write-dominated like the LIF forward that saves h_seq: the same residency cap (twice the tuned value, the step
  // being a longer dependent chain), scaled with T in the same way
  int cap = 2 * tuning().fwd_blocks_per_cu;
  if (a.T < 4) cap = 0; else if (a.T < 16) cap *= 2;
  const unsigned lds = sizeof(S) == 4 ? occupancy_cap_lds(cap) : 0u;
  ProfileScope prof(KC_FORWARD, stream);
  if (vector) {
    if (round_each) hipLaunchKernelGGL((izhikevich_forward_kernel<S, true, true>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((izhikevich_forward_kernel<S, true, false>), grid, threads, lds, stream, a);
  } else {
    if (round_each) hipLaunchKernelGGL((izhikevich_forward_kernel<S, false, true>), grid, threads, lds, stream, a);
    else hipLaunchKernelGGL((izhikevich_forward_kernel<S, false, false>), grid, threads, lds, stream, a);
  }
  return check_launch("izhikevich_forward");
}

template <typename S>
int launch_bwd_typed(const IzhBwdArgs &a, bool vector, hipStream_t stream) {
  const int block = tuning().bwd_block;
  const int V = vector ? Acc<S, true, true>::V : 1;
  const int64_t blocks = ((a.N + V - 1) / V + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "izhikevich_backward: N=%lld", (long long)a.N);
  ProfileScope prof(KC_BACKWARD, stream);
  if (vector) hipLaunchKernelGGL((izhikevich_backward_kernel<S, true>), dim3((unsigned)blocks), dim3(block), 0, stream, a);
  else hipLaunchKernelGGL((izhikevich_backward_kernel<S, false>), dim3((unsigned)blocks), dim3(block), 0, stream, a);
  return check_launch("izhikevich_backward");
}

float round_to(int dtype, float f) {
  return dtype == SJHIP_F16 ? Cvt<f16_t>::round(f) : dtype == SJHIP_BF16 ? Cvt<bf16_t>::round(f) : f;
}

bool all_aligned(std::initializer_list<const void *> ptrs) {
  for (const void *p : ptrs)
    if (p != nullptr && !aligned16(p)) return false;
  return true;
}

}  // namespace

int launch_izhikevich_forward(int dtype, const sjhip_izhikevich_params &p, int64_t T, int64_t N, const void *x_seq,
                              const void *v_init, const void *w_init, void *spike_seq, void *v_seq, void *w_seq,
                              void *v_last, void *w_last, void *h_seq, hipStream_t stream) {
  IzhFwdArgs a;
  a.x = x_seq; a.v_init = v_init; a.w_init = w_init;
  a.spike = spike_seq; a.v_seq = v_seq; a.w_seq = w_seq; a.v_last = v_last; a.w_last = w_last; a.h = h_seq;
  a.T = T; a.N = N;
  a.tau_mul = exact_reciprocal(p.tau) ? 1 : 0;
  a.tau = a.tau_mul ? 1.0f / p.tau : p.tau;
  a.tau_w_mul = exact_reciprocal(p.tau_w) ? 1 : 0;
  a.tau_w = a.tau_w_mul ? 1.0f / p.tau_w : p.tau_w;
  const bool round_each = dtype != SJHIP_F32 && !(p.flags & SJHIP_FLAG_FP32_STATE);
  // torch rounds a Python scalar to the tensor dtype before add / sub and keeps it in fp32 for mul / div
  a.rest_sub = round_each ? round_to(dtype, p.v_rest) : p.v_rest;
  a.c_sub = round_each ? round_to(dtype, p.v_c) : p.v_c;
  a.vth_sub = round_each ? round_to(dtype, p.v_threshold) : p.v_threshold;
  a.a0 = p.a0; a.a = p.a; a.b = p.b;
  a.vth_mul = p.v_threshold; a.vr_mul = p.v_reset;
  a.soft_reset = (p.flags & SJHIP_FLAG_SOFT_RESET) ? 1 : 0;
  a.v_broadcast = (p.flags & SJHIP_FLAG_V_INIT_BROADCAST) ? 1 : 0;
  a.w_broadcast = (p.flags & SJHIP_FLAG_W_INIT_BROADCAST) ? 1 : 0;
  const int V = dtype == SJHIP_F32 ? 4 : 8;
  const bool vector = (N % V == 0) && all_aligned({x_seq, spike_seq, v_seq, w_seq, v_last, w_last, h_seq}) &&
                      (a.v_broadcast || aligned16(v_init)) && (a.w_broadcast || aligned16(w_init));
  switch (dtype) {
    case SJHIP_F32: return launch_fwd_typed<float>(a, vector, false, stream);
    case SJHIP_F16: return launch_fwd_typed<f16_t>(a, vector, round_each, stream);
    case SJHIP_BF16: return launch_fwd_typed<bf16_t>(a, vector, round_each, stream);
    default: return fail(SJHIP_ERR_INVALID, "izhikevich_forward: dtype %d", dtype);
  }
}

int launch_izhikevich_backward(int dtype, const sjhip_izhikevich_params &p, int64_t T, int64_t N,
                               const void *grad_spike_seq, const void *grad_v_seq, const void *grad_w_seq,
                               const void *grad_v_last, const void *grad_w_last, const void *h_seq, const void *v_init,
                               void *grad_x_seq, void *grad_v_init, void *grad_w_init, hipStream_t stream) {
  IzhBwdArgs a;
  a.grad_spike = grad_spike_seq; a.grad_v_seq = grad_v_seq; a.grad_w_seq = grad_w_seq;
  a.grad_v_last = grad_v_last; a.grad_w_last = grad_w_last; a.h = h_seq; a.v_init = v_init;
  a.grad_x = grad_x_seq; a.grad_v_init = grad_v_init; a.grad_w_init = grad_w_init;
  a.T = T; a.N = N;
  a.k = (float)(1.0 / (double)p.tau); a.kw = (float)(1.0 / (double)p.tau_w);
  a.a0 = p.a0; a.a = p.a; a.b = p.b; a.v_rest = p.v_rest; a.v_c = p.v_c;
  a.v_th = p.v_threshold; a.v_reset = p.v_reset; a.alpha = p.sg_alpha; a.sg = p.sg_id;
  a.soft_reset = (p.flags & SJHIP_FLAG_SOFT_RESET) ? 1 : 0;
  a.detach_reset = (p.flags & SJHIP_FLAG_DETACH_RESET) ? 1 : 0;
  a.v_broadcast = (p.flags & SJHIP_FLAG_V_INIT_BROADCAST) ? 1 : 0;
  const int V = dtype == SJHIP_F32 ? 4 : 8;
  const bool vector = (N % V == 0) && all_aligned({grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last, h_seq,
                                                   grad_x_seq, grad_v_init, grad_w_init}) &&
                      (v_init == nullptr || a.v_broadcast || aligned16(v_init));
  switch (dtype) {
    case SJHIP_F32: return launch_bwd_typed<float>(a, vector, stream);
    case SJHIP_F16: return launch_bwd_typed<f16_t>(a, vector, stream);
    case SJHIP_BF16: return launch_bwd_typed<bf16_t>(a, vector, stream);
    default: return fail(SJHIP_ERR_INVALID, "izhikevich_backward: dtype %d", dtype);
  }
}

}  // namespace sjhip
