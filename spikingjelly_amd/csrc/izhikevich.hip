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

// The step is compiled once per combination of three launch-uniform choices, so that its body is straight-line code
// and the V neurons of a work-item interleave (a uniform branch inside the step would serialise them):
// bit 0: 1/tau is exact, multiply instead of divide; bit 1: the same for tau_w; bit 2: soft reset.
constexpr int IZH_TAU_MUL = 1, IZH_TAUW_MUL = 2, IZH_SOFT = 4, IZH_VARIANTS = 8;
__device__ __forceinline__ int izhikevich_variant(const IzhFwdArgs &a) {
  return (a.tau_mul ? IZH_TAU_MUL : 0) | (a.tau_w_mul ? IZH_TAUW_MUL : 0) | (a.soft_reset ? IZH_SOFT : 0);
}

// One step of one neuron in torch's op order; every result is rounded to R (the storage dtype when every op is
// rounded, fp32 otherwise).  The forward kernel and the replaying backward share it, so a replayed h_t has the
// forward's bits.
template <typename R, int VAR>
__device__ __forceinline__ void izhikevich_step(const IzhFwdArgs &a, float x, float &v, float &w, float &h, float &s) {
#pragma clang fp contract(off)
  const float d1 = Cvt<R>::round(v - a.rest_sub);
  const float m1 = scalar_product<R>(a.a0, d1);
  const float d2 = Cvt<R>::round(v - a.c_sub);
  const float m2 = Cvt<R>::round(m1 * d2);
  const float e = Cvt<R>::round(Cvt<R>::round(x + m2) - w);
  const float f = (VAR & IZH_TAU_MUL) ? scalar_product<R>(a.tau, e) : Cvt<R>::round(e / a.tau);
  h = Cvt<R>::round(v + f);
  const float p = Cvt<R>::round(h - a.rest_sub);
  const float r = Cvt<R>::round(scalar_product<R>(a.a, p) - w);
  const float u = (VAR & IZH_TAUW_MUL) ? scalar_product<R>(a.tau_w, r) : Cvt<R>::round(r / a.tau_w);
  const float wn = Cvt<R>::round(w + u);
  const float over = Cvt<R>::round(h - a.vth_sub);
  s = (over >= 0.0f) ? 1.0f : 0.0f;
  if constexpr ((VAR & IZH_SOFT) != 0) {
    v = Cvt<R>::round(h - scalar_product<R>(a.vth_mul, s));
  } else {
    const float keep = Cvt<R>::round(Cvt<R>::round(1.0f - s) * h);
    v = Cvt<R>::round(keep + scalar_product<R>(a.vr_mul, s));
  }
  w = Cvt<R>::round(wn + scalar_product<R>(a.b, s));
}

template <typename S, bool VECTOR, bool ROUND_EACH, int VAR>
__device__ __forceinline__ void izhikevich_forward_walk(const IzhFwdArgs &a, int64_t col) {
  typedef Acc<S, VECTOR, false> A;
  typedef typename A::elem_t E;
  typedef typename std::conditional<ROUND_EACH, S, float>::type R;
  constexpr int V = A::V;
  constexpr int PF = SJHIP_IZH_PF;

  const int64_t N = a.N, T = a.T;
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
        for (int j = 0; j < V; ++j) izhikevich_step<R, VAR>(a, x[j], v[j], w[j], h[j], s[j]);
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

template <typename S, bool VECTOR, bool ROUND_EACH>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) izhikevich_forward_kernel(const IzhFwdArgs a) {
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * Acc<S, VECTOR, false>::V;
  if (col >= a.N) return;
  switch (izhikevich_variant(a)) {
    case 0: izhikevich_forward_walk<S, VECTOR, ROUND_EACH, 0>(a, col); break;
    case 1: izhikevich_forward_walk<S, VECTOR, ROUND_EACH, 1>(a, col); break;
    case 2: izhikevich_forward_walk<S, VECTOR, ROUND_EACH, 2>(a, col); break;
    case 3: izhikevich_forward_walk<S, VECTOR, ROUND_EACH, 3>(a, col); break;
    case 4: izhikevich_forward_walk<S, VECTOR, ROUND_EACH, 4>(a, col); break;
    case 5: izhikevich_forward_walk<S, VECTOR, ROUND_EACH, 5>(a, col); break;
    case 6: izhikevich_forward_walk<S, VECTOR, ROUND_EACH, 6>(a, col); break;
    default: izhikevich_forward_walk<S, VECTOR, ROUND_EACH, 7>(a, col); break;
  }
}

// Replays the forward recurrence of one work-item (four neurons) from x_seq, v_init and w_init and parks h_t of every
// step in LDS as fp32; each work-item touches only its own LDS words, so no barrier is needed.
template <typename S, bool ROUND_EACH, int VAR, bool SHORT>
__device__ __forceinline__ void izhikevich_replay(const IzhFwdArgs &a, f32x4 *lds_h, int64_t col) {
  typedef Acc<S, true, true> A;
  typedef typename A::elem_t E;
  typedef typename std::conditional<ROUND_EACH, S, float>::type R;
  constexpr int V = A::V;
  static_assert(V == 4, "the replay parks one f32x4 per work-item and step");
  constexpr int PF = SHORT ? 2 : SJHIP_IZH_PF;

  const int64_t N = a.N, T = a.T;
  const E *xp = (const E *)a.x + col;
  typename A::raw_t ahead[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) ahead[i] = (i < T) ? A::load(xp + (int64_t)i * N) : A::zero();
  float v[V], w[V];
  load_state<S, true, true>(a.v_init, col, a.v_broadcast != 0, v);
  load_state<S, true, true>(a.w_init, col, a.w_broadcast != 0, w);
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
        for (int j = 0; j < V; ++j) izhikevich_step<R, VAR>(a, x[j], v[j], w[j], h[j], s[j]);
        f32x4 park; park.x = h[0]; park.y = h[1]; park.z = h[2]; park.w = h[3];
        lds_h[(int)t * (int)blockDim.x + (int)threadIdx.x] = park;
      }
    }
  }
}

// The first rows of the upstream gradients (and of a saved h_seq) of one work-item, requested before anything else so
// that they arrive while h is being replayed.
// RP: IZH_REPLAY (h_t comes from LDS) and / or IZH_SHORT (two rows in flight instead of SJHIP_IZH_PF: for sequences of up
// to eight steps the registers serve resident wavefronts better; replaying backward fp32, T = 4: 3.4 -> 5.2 TB/s,
// T = 16: 4.5 -> 4.4)
constexpr int IZH_REPLAY = 1, IZH_SHORT = 2;

template <typename S, bool VECTOR, int RP>
struct IzhPrologue {
  typedef Acc<S, VECTOR, true> A;
  typedef typename A::elem_t E;
  static constexpr bool REPLAY = (RP & IZH_REPLAY) != 0;
  static constexpr int V = A::V;
  static constexpr int PF = (RP & IZH_SHORT) ? 2 : SJHIP_IZH_PF;
  typename A::raw_t gs[PF], h[PF], gv[PF], gw[PF];
  float gv_last[V], gw_last[V];

  __device__ __forceinline__ void load(const IzhBwdArgs &a, int64_t col) {
    const int64_t N = a.N, T = a.T;
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = T - 1 - i;
      gs[i] = (t >= 0) ? A::load((const E *)a.grad_spike + col + t * N) : A::zero();
      if (!REPLAY) h[i] = (t >= 0) ? A::load((const E *)a.h + col + t * N) : A::zero();
      if (a.grad_v_seq) gv[i] = (t >= 0) ? A::load((const E *)a.grad_v_seq + col + t * N) : A::zero();
      if (a.grad_w_seq) gw[i] = (t >= 0) ? A::load((const E *)a.grad_w_seq + col + t * N) : A::zero();
    }
#pragma unroll
    for (int j = 0; j < V; ++j) { gv_last[j] = 0.0f; gw_last[j] = 0.0f; }
    if (a.grad_v_last) A::unpack(A::load((const E *)a.grad_v_last + col), gv_last);
    if (a.grad_w_last) A::unpack(A::load((const E *)a.grad_w_last + col), gw_last);
  }
};

// The BPTT walk of one work-item for surrogate SG.  REPLAY: h_t comes from LDS, otherwise from the saved h_seq.
// The two reset rules share one expression whose coefficients are chosen once per launch, so the per-neuron code has
// no branch:
//     v_t  = s ? fire_h h + fire_c : h            soft: h - v_th            hard: v_reset
//     dvdh = (1 - s hard) + sg (d_c + d_h h)      soft: 1 - live v_th sg    hard: (1 - s) + sg (v_reset - live h)
template <typename S, bool VECTOR, int RP, int SG>
__device__ __forceinline__ void izhikevich_bptt_walk(const IzhBwdArgs &a, const f32x4 *lds_h, int64_t col,
                                                     IzhPrologue<S, VECTOR, RP> &pre) {
  typedef Acc<S, VECTOR, true> A;
  typedef typename A::elem_t E;
  constexpr bool REPLAY = (RP & IZH_REPLAY) != 0;
  constexpr int V = A::V;
  constexpr int PF = IzhPrologue<S, VECTOR, RP>::PF;

  const int64_t N = a.N, T = a.T;
  const E *gsp = (const E *)a.grad_spike + col;
  const E *hp = REPLAY ? nullptr : (const E *)a.h + col;
  const E *gvp = a.grad_v_seq ? (const E *)a.grad_v_seq + col : nullptr;
  const E *gwp = a.grad_w_seq ? (const E *)a.grad_w_seq + col : nullptr;

  const float live = a.detach_reset ? 0.0f : 1.0f;
  const float hard = a.soft_reset ? 0.0f : 1.0f;
  const float fire_h = a.soft_reset ? 1.0f : 0.0f, fire_c = a.soft_reset ? -a.v_th : a.v_reset;
  const float d_c = a.soft_reset ? -live * a.v_th : a.v_reset, d_h = a.soft_reset ? 0.0f : -live;
  const float k = a.k, kw = a.kw, ka0 = a.k * a.a0, kwa = a.kw * a.a;

  float gh_next[V], cw_next[V];
#pragma unroll
  for (int j = 0; j < V; ++j) { gh_next[j] = 0.0f; cw_next[j] = pre.gw_last[j]; }

  for (int64_t t0 = T - 1; t0 >= 0; t0 -= PF) {
    typename A::raw_t cur_gs[PF], cur_h[PF], cur_gv[PF], cur_gw[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      cur_gs[i] = pre.gs[i];
      if (!REPLAY) cur_h[i] = pre.h[i];
      if (gvp) cur_gv[i] = pre.gv[i];
      if (gwp) cur_gw[i] = pre.gw[i];
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 - PF - i;
      if (tn >= 0) {
        pre.gs[i] = A::load(gsp + tn * N);
        if (!REPLAY) pre.h[i] = A::load(hp + tn * N);
        if (gvp) pre.gv[i] = A::load(gvp + tn * N);
        if (gwp) pre.gw[i] = A::load(gwp + tn * N);
      }
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 - i;
      if (t >= 0) {
        float gs[V], h[V], gvs[V], gws[V], gx[V];
        A::unpack(cur_gs[i], gs);
        if constexpr (REPLAY) {
          const f32x4 park = lds_h[(int)t * (int)blockDim.x + (int)threadIdx.x];
          h[0] = park.x; h[1] = park.y; h[2] = park.z; h[3] = park.w;
        } else {
          A::unpack(cur_h[i], h);
        }
#pragma unroll
        for (int j = 0; j < V; ++j) { gvs[j] = 0.0f; gws[j] = 0.0f; }
        if (gvp) A::unpack(cur_gv[i], gvs);
        if (gwp) A::unpack(cur_gw[i], gws);
        const bool last = t == T - 1;
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float over = h[j] - a.v_th;
          const bool fired = over >= 0.0f;
          const float s = fired ? 1.0f : 0.0f;
          float v_t;
          {
#pragma clang fp contract(off)
            v_t = fired ? (fire_h * h[j] + fire_c) : h[j];
          }
          const float sg = surrogate_grad<SG, false>(over, a.alpha);
          const float dhdv = 1.0f + ka0 * ((v_t - a.v_c) + (v_t - a.v_rest));
          const float gv = (last ? pre.gv_last[j] : gh_next[j] * dhdv) + gvs[j];
          const float gw = cw_next[j] + gws[j];  // cw_next starts from grad_w_last
          const float dvdh = (1.0f - s * hard) + sg * (d_c + d_h * h[j]);
          const float gh = gv * dvdh + (gs[j] + a.b * gw) * sg + gw * kwa;
          gx[j] = gh * k;
          gh_next[j] = gh;
          cw_next[j] = gw * (1.0f - kw) - gx[j];
        }
        A::store((E *)a.grad_x + col + t * N, gx);
      }
    }
  }
  if (a.grad_v_init) {
    float v0[V];
    load_state<S, VECTOR, true>(a.v_init, col, a.v_broadcast != 0, v0);
#pragma unroll
    for (int j = 0; j < V; ++j) gh_next[j] *= 1.0f + ka0 * ((v0[j] - a.v_c) + (v0[j] - a.v_rest));
    A::store((E *)a.grad_v_init + col, gh_next);
  }
  if (a.grad_w_init) A::store((E *)a.grad_w_init + col, cw_next);
}

template <typename S, bool VECTOR, int RP>
__device__ __forceinline__ void izhikevich_bptt(const IzhBwdArgs &a, const f32x4 *lds_h, int64_t col,
                                                IzhPrologue<S, VECTOR, RP> &pre) {
  switch (a.sg) {
    case SJHIP_SG_SIGMOID: izhikevich_bptt_walk<S, VECTOR, RP, SJHIP_SG_SIGMOID>(a, lds_h, col, pre); break;
    case SJHIP_SG_ATAN: izhikevich_bptt_walk<S, VECTOR, RP, SJHIP_SG_ATAN>(a, lds_h, col, pre); break;
    case SJHIP_SG_PIECEWISE_QUADRATIC: izhikevich_bptt_walk<S, VECTOR, RP, SJHIP_SG_PIECEWISE_QUADRATIC>(a, lds_h, col, pre); break;
    case SJHIP_SG_PIECEWISE_EXP: izhikevich_bptt_walk<S, VECTOR, RP, SJHIP_SG_PIECEWISE_EXP>(a, lds_h, col, pre); break;
    case SJHIP_SG_SOFT_SIGN: izhikevich_bptt_walk<S, VECTOR, RP, SJHIP_SG_SOFT_SIGN>(a, lds_h, col, pre); break;
    case SJHIP_SG_SUPER_SPIKE: izhikevich_bptt_walk<S, VECTOR, RP, SJHIP_SG_SUPER_SPIKE>(a, lds_h, col, pre); break;
    default: izhikevich_bptt_walk<S, VECTOR, RP, SJHIP_SG_ERF>(a, lds_h, col, pre); break;
  }
}

template <typename S, bool VECTOR, bool SHORT>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) izhikevich_backward_kernel(const IzhBwdArgs a) {
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * Acc<S, VECTOR, true>::V;
  if (col >= a.N) return;
  constexpr int RP = SHORT ? IZH_SHORT : 0;
  IzhPrologue<S, VECTOR, RP> pre;
  pre.load(a, col);
  izhikevich_bptt<S, VECTOR, RP>(a, nullptr, col, pre);
}

// Backward that recomputes h instead of reading a saved h_seq: the forward then never writes h_seq and this kernel
// reads x_seq in its place.  S is fp32 or a four-neurons-per-work-item 16-bit type; LDS holds T * blockDim * 16 bytes.
template <typename S, bool ROUND_EACH, bool SHORT>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) izhikevich_backward_replay_kernel(const IzhFwdArgs f, const IzhBwdArgs a) {
  extern __shared__ f32x4 izh_lds_h[];
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (col >= a.N) return;
  constexpr int RP = IZH_REPLAY | (SHORT ? IZH_SHORT : 0);
  IzhPrologue<S, true, RP> pre;
  pre.load(a, col);
  switch (izhikevich_variant(f)) {
    case 0: izhikevich_replay<S, ROUND_EACH, 0, SHORT>(f, izh_lds_h, col); break;
    case 1: izhikevich_replay<S, ROUND_EACH, 1, SHORT>(f, izh_lds_h, col); break;
    case 2: izhikevich_replay<S, ROUND_EACH, 2, SHORT>(f, izh_lds_h, col); break;
    case 3: izhikevich_replay<S, ROUND_EACH, 3, SHORT>(f, izh_lds_h, col); break;
    case 4: izhikevich_replay<S, ROUND_EACH, 4, SHORT>(f, izh_lds_h, col); break;
    case 5: izhikevich_replay<S, ROUND_EACH, 5, SHORT>(f, izh_lds_h, col); break;
    case 6: izhikevich_replay<S, ROUND_EACH, 6, SHORT>(f, izh_lds_h, col); break;
    default: izhikevich_replay<S, ROUND_EACH, 7, SHORT>(f, izh_lds_h, col); break;
  }
  izhikevich_bptt<S, true, RP>(a, izh_lds_h, col, pre);
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
  const dim3 grid((unsigned)blocks), threads(block);
  if (a.T <= kShortSequence) {
    if (vector) hipLaunchKernelGGL((izhikevich_backward_kernel<S, true, true>), grid, threads, 0, stream, a);
    else hipLaunchKernelGGL((izhikevich_backward_kernel<S, false, true>), grid, threads, 0, stream, a);
  } else {
    if (vector) hipLaunchKernelGGL((izhikevich_backward_kernel<S, true, false>), grid, threads, 0, stream, a);
    else hipLaunchKernelGGL((izhikevich_backward_kernel<S, false, false>), grid, threads, 0, stream, a);
  }
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

bool build_forward_args(IzhFwdArgs &a, int dtype, const sjhip_izhikevich_params &p, int64_t T, int64_t N,
                        const void *x_seq, const void *v_init, const void *w_init) {
  a.x = x_seq; a.v_init = v_init; a.w_init = w_init;
  a.spike = nullptr; a.v_seq = nullptr; a.w_seq = nullptr; a.v_last = nullptr; a.w_last = nullptr; a.h = nullptr;
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
  return round_each;
}

void build_backward_args(IzhBwdArgs &a, const sjhip_izhikevich_params &p, int64_t T, int64_t N, const void *grad_spike_seq,
                         const void *grad_v_seq, const void *grad_w_seq, const void *grad_v_last, const void *grad_w_last,
                         const void *h_seq, const void *v_init, void *grad_x_seq, void *grad_v_init, void *grad_w_init) {
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
}

}  // namespace

int launch_izhikevich_forward(int dtype, const sjhip_izhikevich_params &p, int64_t T, int64_t N, const void *x_seq,
                              const void *v_init, const void *w_init, void *spike_seq, void *v_seq, void *w_seq,
                              void *v_last, void *w_last, void *h_seq, hipStream_t stream) {
  IzhFwdArgs a;
  const bool round_each = build_forward_args(a, dtype, p, T, N, x_seq, v_init, w_init);
  a.spike = spike_seq; a.v_seq = v_seq; a.w_seq = w_seq; a.v_last = v_last; a.w_last = w_last; a.h = h_seq;
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
  build_backward_args(a, p, T, N, grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last, h_seq, v_init,
                      grad_x_seq, grad_v_init, grad_w_init);
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

namespace {

template <typename S>
void launch_replay_typed(const IzhFwdArgs &f, const IzhBwdArgs &b, bool round_each, int block, unsigned lds,
                         int64_t blocks, hipStream_t stream) {
  const dim3 grid((unsigned)blocks), threads(block);
  if (b.T <= kShortSequence) {
    if (round_each) hipLaunchKernelGGL((izhikevich_backward_replay_kernel<S, true, true>), grid, threads, lds, stream, f, b);
    else hipLaunchKernelGGL((izhikevich_backward_replay_kernel<S, false, true>), grid, threads, lds, stream, f, b);
  } else {
    if (round_each) hipLaunchKernelGGL((izhikevich_backward_replay_kernel<S, true, false>), grid, threads, lds, stream, f, b);
    else hipLaunchKernelGGL((izhikevich_backward_replay_kernel<S, false, false>), grid, threads, lds, stream, f, b);
  }
}

}  // namespace

int launch_izhikevich_backward_replay(int dtype, const sjhip_izhikevich_params &p, int64_t T, int64_t N,
                                      const void *x_seq, const void *v_init, const void *w_init,
                                      const void *grad_spike_seq, const void *grad_v_seq, const void *grad_w_seq,
                                      const void *grad_v_last, const void *grad_w_last, void *grad_x_seq,
                                      void *grad_v_init, void *grad_w_init, hipStream_t stream) {
  // same LDS footprint per work-item and step as the replay of the one-state neurons (one f32x4), so the same limits
  if (!recompute_supported(dtype, T, N))
    return fail(SJHIP_ERR_UNSUPPORTED, "izhikevich_backward(replay): T=%lld N=%lld does not fit (N %% %d != 0 or T too large for LDS)",
                (long long)T, (long long)N, dtype == SJHIP_F32 ? 4 : 8);
  IzhFwdArgs f;
  const bool round_each = build_forward_args(f, dtype, p, T, N, x_seq, v_init, w_init);
  if (!all_aligned({x_seq, grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last, grad_x_seq, grad_v_init, grad_w_init}) ||
      (!f.v_broadcast && !aligned16(v_init)) || (!f.w_broadcast && !aligned16(w_init)))
    return fail(SJHIP_ERR_INVALID, "izhikevich_backward(replay): every tensor must be 16-byte aligned");
  IzhBwdArgs b;
  build_backward_args(b, p, T, N, grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last, nullptr, v_init,
                      grad_x_seq, grad_v_init, grad_w_init);
  const int block = recompute_block(dtype, T, round_each);
  const int64_t blocks = (N / 4 + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "izhikevich_backward(replay): N=%lld", (long long)N);
  unsigned lds = (unsigned)(T * block * 16);
  const unsigned cap = occupancy_cap_lds(tuning().replay_blocks_per_cu);
  if (cap > lds) lds = cap;
  ProfileScope prof(KC_BACKWARD, stream);
  switch (dtype) {
    case SJHIP_F32: launch_replay_typed<float>(f, b, false, block, lds, blocks, stream); break;
    case SJHIP_F16: launch_replay_typed<f16n_t>(f, b, round_each, block, lds, blocks, stream); break;
    case SJHIP_BF16: launch_replay_typed<bf16n_t>(f, b, round_each, block, lds, blocks, stream); break;
    default: return fail(SJHIP_ERR_INVALID, "izhikevich_backward(replay): dtype %d", dtype);
  }
  return check_launch("izhikevich_backward(replay)");
}

}  // namespace sjhip
