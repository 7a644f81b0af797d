// Multi-step forward (charge -> fire -> reset over T steps) for IF / LIF / PLIF / QIF / ILIF.
//
// One work-item owns V consecutive neurons (one 128-bit access per row) and walks the T rows in
// order with the membrane potential in registers.  Rows of x are requested SJHIP_FWD_PF steps ahead
// of their use so several 128-bit loads per lane are always in flight; every tensor is touched
// exactly once (default cache policy: the write-dominated forward measured slower with
// non-temporal accesses, the read-dominated backward faster).
//
// The arithmetic restates the torch backend of the reference op for op and in its order
// (functional/neuron.py:225-228 voltage_reset, :310-312 if_step, :849-852 lif_charge, :1290-1297
// plif_step, surrogate.py:60 heaviside), with floating-point contraction off, so spikes, h and v are
// bit-identical to it in fp32.  For 16-bit storage either every op result is rounded to the storage
// dtype (the torch backend run on half tensors) or state and arithmetic stay fp32 and only stored
// values are rounded (the reference's mixed-precision kernels).
#pragma once

#include <cmath>
#include <type_traits>

#include "sjhip_common.h"

#ifndef SJHIP_FWD_PF
#define SJHIP_FWD_PF 8
#endif
// prefetch depth for 16-bit storage: a 16-byte access carries eight neurons there, so the per-lane state is
// twice as large and fewer rows in flight keep two wavefronts per SIMD resident
#ifndef SJHIP_FWD_PF16
#define SJHIP_FWD_PF16 4
#endif
#ifndef SJHIP_FWD_NT
#define SJHIP_FWD_NT 0
#endif
#ifndef SJHIP_FWD_PACKED_NT
#define SJHIP_FWD_PACKED_NT 1
#endif

namespace sjhip {

enum Charge {
  CH_IF = 0,
  CH_DECAY_INPUT_DIV = 1,  // v + (x - (v - vr)) / tau
  CH_DECAY_INPUT_MUL = 2,  // v + (x - (v - vr)) * k
  CH_PLAIN_INPUT_DIV = 3,  // v - (v - vr) / tau + x
  CH_PLAIN_INPUT_MUL = 4,  // v - (v - vr) * k + x
  CH_QIF_DIV = 5,          // v + (x + a0 * (v - v_rest) * (v - v_c)) / tau
  CH_QIF_MUL = 6,          // the same with * k
  CH_EIF_DIV = 7,          // v + (x + v_rest - v + dT * exp((v - theta) / dT)) / tau
  CH_EIF_MUL = 8           // the same with * k
};

struct FwdArgs {
  const void *x;
  const void *v_init;
  void *spike;           // dense spikes in the storage dtype, or the bit-packed byte array
  void *v_seq;           // may be null
  void *v_last;          // may be null
  void *h;               // may be null
  const float *k_device; // may be null: use `tau`
  int64_t T, N;
  float tau;     // divisor (DIV charges) or multiplier k (MUL charges)
  float vr_add;  // v_reset as an addend   (rounded to the storage dtype when every op is rounded)
  float vr_mul;  // v_reset as a factor    (fp32 always)
  float vth_sub; // v_threshold as a subtrahend
  float vth_mul; // v_threshold as a factor
  float q_rest_sub; // QIF: v_rest and v_c as subtrahends (rounded like vr_add), a0 as a factor
  float q_c_sub;    // EIF: v_rest as an addend, theta_rh as a subtrahend, delta_T as divisor and factor
  float q_a0_mul;
  float level_max;  // ILIF: largest spike count
  float vth_inv;    // ILIF: 1 / v_threshold when that is an exact power of two (h / v_th == h * vth_inv bit for bit), else 0
  int charge;
  int soft_reset;        // a Reset value
  int v_init_broadcast;  // v_init holds one element for all neurons
  int spread;            // block-to-column order, see column_block()
  void *checkpoints;     // forward_pieces_kernel only: [ceil(T / chunk) - 1][N] states after every chunk steps
  int64_t chunk;
};

// Fire-and-reset rule.  RESET_COUNT is ILIF (functional/neuron.py:1097-1099 with quantize.py:592): the neuron fires
// the count c = rint(clamp(h / v_th, 0, level_max)) and resets softly by c * v_th.
enum Reset { RESET_HARD = 0, RESET_SOFT = 1, RESET_COUNT = 2 };

// One neuron, one step.  R::round() is applied to the result of every arithmetic op.
template <typename R, int CH, int RS>
__device__ __forceinline__ void neuron_step(float x, float &v, float &h, float &s, float tau,
                                            const FwdArgs &a) {
#pragma clang fp contract(off)
  if (CH == CH_IF) {
    h = Cvt<R>::round(v + x);
  } else if (CH == CH_DECAY_INPUT_DIV || CH == CH_DECAY_INPUT_MUL) {
    float d = Cvt<R>::round(v - a.vr_add);
    float e = Cvt<R>::round(x - d);
    float f = (CH == CH_DECAY_INPUT_DIV) ? Cvt<R>::round(e / tau) : Cvt<R>::round(e * tau);
    h = Cvt<R>::round(v + f);
  } else if (CH == CH_QIF_DIV || CH == CH_QIF_MUL) {
    // functional/neuron.py:397, evaluated left to right: ((a0 * (v - v_rest)) * (v - v_c))
    float d1 = Cvt<R>::round(v - a.q_rest_sub);
    float m1 = Cvt<R>::round(a.q_a0_mul * d1);
    float d2 = Cvt<R>::round(v - a.q_c_sub);
    float m2 = Cvt<R>::round(m1 * d2);
    float e = Cvt<R>::round(x + m2);
    float f = (CH == CH_QIF_DIV) ? Cvt<R>::round(e / tau) : Cvt<R>::round(e * tau);
    h = Cvt<R>::round(v + f);
  } else if (CH == CH_EIF_DIV || CH == CH_EIF_MUL) {
    // functional/neuron.py:483-485, left to right: ((x + v_rest) - v) + delta_T * exp((v - theta_rh) / delta_T)
    float b = Cvt<R>::round(Cvt<R>::round(x + a.q_rest_sub) - v);
    float d = Cvt<R>::round(Cvt<R>::round(v - a.q_c_sub) / a.q_a0_mul);
    float e = Cvt<R>::round(expf(d));
    float g = Cvt<R>::round(b + Cvt<R>::round(a.q_a0_mul * e));
    float f = (CH == CH_EIF_DIV) ? Cvt<R>::round(g / tau) : Cvt<R>::round(g * tau);
    h = Cvt<R>::round(v + f);
  } else {
    float d = Cvt<R>::round(v - a.vr_add);
    float f = (CH == CH_PLAIN_INPUT_DIV) ? Cvt<R>::round(d / tau) : Cvt<R>::round(d * tau);
    float g = Cvt<R>::round(v - f);
    h = Cvt<R>::round(g + x);
  }
  if (RS == RESET_COUNT) {
    // written with comparisons so that a NaN stays a NaN, as in torch.clamp
    float z = Cvt<R>::round(a.vth_inv != 0.0f ? h * a.vth_inv : h / a.vth_mul);
    z = (z < 0.0f) ? 0.0f : ((z > a.level_max) ? a.level_max : z);
    s = rintf(z);
    float m = Cvt<R>::round(s * a.vth_mul);
    v = Cvt<R>::round(h - m);
    return;
  }
  float over = Cvt<R>::round(h - a.vth_sub);
  s = (over >= 0.0f) ? 1.0f : 0.0f;
  if (RS == RESET_SOFT) {
    float m = Cvt<R>::round(s * a.vth_mul);
    v = Cvt<R>::round(h - m);
  } else {
    // kept in the reference's arithmetic form (not a select): 0 * v_reset and 0 * h keep the
    // signed-zero / NaN behaviour of  s * v_reset + (1 - s) * h
    float m = Cvt<R>::round(s * a.vr_mul);
    float n = Cvt<R>::round(1.0f - s);
    float o = Cvt<R>::round(n * h);
    v = Cvt<R>::round(m + o);
  }
}

// fp16 storage with every op rounded: the same step in native half arithmetic.  For two fp16 operands an
// fp32 add / sub / mul followed by rounding to fp16 equals the correctly rounded fp16 operation (24 >= 2 * 11 + 2
// significand bits, so the double rounding is harmless; fp16 subnormals are kept), hence these results are
// bit-identical to neuron_step<f16_t> on floats while needing no conversions.  Python scalars that torch keeps
// in fp32 (the tau divisor / multiplier, v_threshold and v_reset as factors) still enter through an fp32 product
// rounded once.
// fp32 product rounded to fp32, then to fp16: the two roundings torch's CPU kernels perform for a half tensor
// times a Python scalar.  The product is pinned in a register because the compiler would otherwise fold the
// multiply and the conversion into v_fma_mixlo_f16, which rounds the exact product once and differs from the
// double rounding in about one result out of forty (measured).
__device__ __forceinline__ _Float16 scalar_product_f16(float scalar, _Float16 t) {
#pragma clang fp contract(off)
  float p = scalar * (float)t;
  asm volatile("" : "+v"(p));
  return (_Float16)p;
}

template <typename R, int CH, int RS>
__device__ __forceinline__ void neuron_step(_Float16 x, _Float16 &v, _Float16 &h, _Float16 &s, float tau,
                                            const FwdArgs &a) {
#pragma clang fp contract(off)
  typedef _Float16 H;
  const H vr_add = (H)a.vr_add, vth_sub = (H)a.vth_sub;  // rounded to fp16 by the host already
  if (CH == CH_IF) {
    h = v + x;
  } else if (CH == CH_DECAY_INPUT_DIV || CH == CH_DECAY_INPUT_MUL) {
    const H d = v - vr_add;
    const H e = x - d;
    const H f = (CH == CH_DECAY_INPUT_DIV) ? (H)((float)e / tau) : scalar_product_f16(tau, e);
    h = v + f;
  } else if (CH == CH_QIF_DIV || CH == CH_QIF_MUL) {
    const H d1 = v - (H)a.q_rest_sub;
    const H m1 = scalar_product_f16(a.q_a0_mul, d1);
    const H d2 = v - (H)a.q_c_sub;
    const H m2 = m1 * d2;
    const H e = x + m2;
    const H f = (CH == CH_QIF_DIV) ? (H)((float)e / tau) : scalar_product_f16(tau, e);
    h = v + f;
  } else if (CH == CH_EIF_DIV || CH == CH_EIF_MUL) {
    const H b = (x + (H)a.q_rest_sub) - v;
    const H d = (H)((float)(H)(v - (H)a.q_c_sub) / a.q_a0_mul);
    const H e = (H)expf((float)d);
    const H g = b + scalar_product_f16(a.q_a0_mul, e);
    const H f = (CH == CH_EIF_DIV) ? (H)((float)g / tau) : scalar_product_f16(tau, g);
    h = v + f;
  } else {
    const H d = v - vr_add;
    const H f = (CH == CH_PLAIN_INPUT_DIV) ? (H)((float)d / tau) : scalar_product_f16(tau, d);
    const H g = v - f;
    h = g + x;
  }
  if (RS == RESET_COUNT) {
    H z = a.vth_inv != 0.0f ? scalar_product_f16(a.vth_inv, h) : (H)((float)h / a.vth_mul);
    const H top = (H)a.level_max;
    z = (z < (H)0.0f) ? (H)0.0f : ((z > top) ? top : z);
    s = (H)rintf((float)z);
    const H m = scalar_product_f16(a.vth_mul, s);  // a count above 1 times v_th need not be exact
    v = h - m;
    return;
  }
  const H over = h - vth_sub;
  s = (over >= (H)0.0f) ? (H)1.0f : (H)0.0f;
  if (RS == RESET_SOFT) {
    const H m = (H)((float)s * a.vth_mul);  // s is 0 or 1: the product is exact, any rounding order agrees
    v = h - m;
  } else {
    const H m = (H)((float)s * a.vr_mul);
    const H n = (H)1.0f - s;
    const H o = n * h;
    v = m + o;
  }
}

// register type of x, v, h, s in the step loop
template <typename S, bool ROUND_EACH> struct StepNum { typedef float type; };
template <> struct StepNum<f16_t, true> { typedef _Float16 type; };

// Bit-packed spike output (PACKED): a.spike is a byte array holding the flattened [T, N] spikes LSB first,
// byte j bit i = element 8 j + i, the layout of bit_pack.  N % 8 == 0 makes every row start on a byte.  A
// work-item with eight neurons writes its byte; with four neurons two neighbouring lanes combine their
// nibbles; with one neuron a wavefront ballot yields eight bytes written by its first eight lanes.
template <int V, typename NUM>
__device__ __forceinline__ void store_spike_bits(uint8_t *row, int64_t col, int64_t N, const NUM (&s)[V]) {
  uint32_t bits = 0;
#pragma unroll
  for (int j = 0; j < V; ++j) bits |= (s[j] != (NUM)0.0f ? 1u : 0u) << j;
  if (V == 8) {
    row[col >> 3] = (uint8_t)bits;
  } else if (V == 4) {
    const uint32_t other = (uint32_t)__shfl_xor((int)bits, 1, 64);
    if ((threadIdx.x & 1) == 0) row[col >> 3] = (uint8_t)(bits | (other << 4));
  } else {
    const unsigned long long mask = __ballot(bits != 0);
    const int lane = threadIdx.x & 63;
    const int64_t col0 = col - lane;  // first neuron of this wavefront, a multiple of 64
    if (lane < 8 && col0 + 8 * lane < N) row[(col0 >> 3) + lane] = (uint8_t)(mask >> (8 * lane));
  }
}

// OUT: what leaves the kernel besides the state, and with it the cache policy of the x loads.  Measured on MI355X with
// both variants on one machine: bit-packed spikes (nothing but x moves) -> streaming everything (98.7 -> 94 us, fp16
// T = 32, N = 6.4 M); 16-bit storage with fp32 state writing spikes plus v_seq / h_seq -> streaming x loads (bf16 T = 8,
// N = 8.4 M: 88 -> 74 us); everything else -> default policy (fp32 with two outputs gained 4 % in a forward-only loop
// but lost 1.2 % inside the training step, forward and backward alternating, which is the case that counts; 16-bit
// with every op rounded lost 2 %).
enum FwdOut { FWD_OUT_DENSE = 0, FWD_OUT_PACKED = 1, FWD_OUT_DENSE_STREAM_X = 2 };
// Added to a FwdOut for a sequence of one step (what step_mode='s' runs): two rows in flight instead of eight; the
// registers the deep prefetch would hold go to resident wavefronts instead (T = 1, N = 134 M fp32: 3.7 -> 6.1 TB/s;
// at T = 2 and 4 the effect is mixed and the deep prefetch stays).
constexpr int FWD_OUT_SHORT = 4;

// CKPT: besides its outputs the walk leaves the state after every a.chunk steps (but not after the last step) in
// a.checkpoints, from where the replaying backward starts each piece of a long sequence.
template <typename S, bool VECTOR, bool ROUND_EACH, int CH, int RS, int OUT, bool CKPT = false>
__device__ __forceinline__ void forward_body(const FwdArgs &a) {
  constexpr bool PACKED = (OUT & 3) == FWD_OUT_PACKED;
  // with bit-packed spikes the kernel is read-dominated (x in, one bit out): streaming policy like the backward
  constexpr bool NT = (SJHIP_FWD_NT != 0) || (PACKED && SJHIP_FWD_PACKED_NT != 0);
  typedef Acc<S, VECTOR, NT> A;
  typedef Acc<S, VECTOR, NT || (OUT & 3) == FWD_OUT_DENSE_STREAM_X> AL;  // policy of the x loads alone
  typedef typename A::elem_t E;
  typedef typename std::conditional<ROUND_EACH, S, float>::type R;
  constexpr int V = A::V;
  // (eight 16-bit rows measured slower, packed too)
  constexpr int PF = (OUT & FWD_OUT_SHORT) ? 2 : (sizeof(S) == 2 ? SJHIP_FWD_PF16 : SJHIP_FWD_PF);

  const int64_t N = a.N, T = a.T;
  const int64_t col = ((int64_t)column_block(a.spread) * blockDim.x + threadIdx.x) * V;
  if (col >= N) return;

  const E *xp = (const E *)a.x + col;
  E *sp = (E *)a.spike + col;
  E *vp = a.v_seq ? (E *)a.v_seq + col : nullptr;
  E *hp = a.h ? (E *)a.h + col : nullptr;
  const float tau = a.k_device ? *a.k_device : a.tau;

  typename A::raw_t ahead[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) ahead[i] = (i < T) ? AL::load(xp + (int64_t)i * N) : A::zero();

  typedef typename StepNum<S, ROUND_EACH>::type NUM;
  NUM v[V];
  load_state<S, VECTOR, NT>(a.v_init, col, a.v_init_broadcast != 0, v);

  int64_t next_checkpoint = CKPT ? a.chunk : 0;  // the step count after which the next checkpoint is due
  E *cp = CKPT ? (E *)a.checkpoints + col : nullptr;
  // PF steps: requests the rows of the PF steps after them, then walks them.  STEADY: every one of those 2 * PF
  // rows exists, so no request stands under a condition; a request under a condition would make each later wait
  // a wait for everything outstanding, the rows just requested included.
  auto walk = [&](int64_t t0, auto steady) {
    constexpr bool STEADY = decltype(steady)::value;
    typename A::raw_t cur[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) cur[i] = ahead[i];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 + PF + i;
      if (STEADY || tn < T) ahead[i] = AL::load(xp + tn * N);
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 + i;
      if (STEADY || t < T) {
        NUM x[V], h[V], s[V];
        A::unpack(cur[i], x);
#pragma unroll
        for (int j = 0; j < V; ++j) neuron_step<R, CH, RS>(x[j], v[j], h[j], s[j], tau, a);
        if (PACKED) store_spike_bits<V>((uint8_t *)a.spike + t * (N >> 3), col, N, s);
        else if (RS == RESET_COUNT) A::store(sp + t * N, s);
        else A::store_spikes(sp + t * N, s);
        if (hp) A::store(hp + t * N, h);
        if (vp) A::store(vp + t * N, v);
        if (CKPT && t + 1 == next_checkpoint && t + 1 < T) {
          if constexpr (sizeof(S) == 2 && !ROUND_EACH) {
            // the state is kept in fp32 beside 16-bit storage: so is its checkpoint
            float *cpf = (float *)a.checkpoints + (next_checkpoint / a.chunk - 1) * N + col;
#pragma unroll
            for (int q = 0; q < V / 4; ++q) {
              f32x4 w; w.x = v[4 * q]; w.y = v[4 * q + 1]; w.z = v[4 * q + 2]; w.w = v[4 * q + 3];
              stream_store<NT>(reinterpret_cast<f32x4 *>(cpf) + q, w);
            }
          } else {
            A::store(cp, v);
            cp += N;
          }
          next_checkpoint += a.chunk;
        }
      }
    }
  };
  int64_t t0 = 0;
  if constexpr (CKPT) {  // long sequences only: the shorter ones gain nothing from the second copy of the loop
    for (; t0 + 2 * PF <= T; t0 += PF) walk(t0, std::true_type());
  }
  for (; t0 < T; t0 += PF) walk(t0, std::false_type());
  if (a.v_last) A::store((E *)a.v_last + col, v);
}

template <typename S, bool VECTOR, bool ROUND_EACH, int CH, int OUT, bool CKPT = false>
__device__ __forceinline__ void forward_reset_dispatch(const FwdArgs &a) {
  // counts exist for the charge ILIF uses (no input decay) and never bit-packed
  if constexpr ((CH == CH_PLAIN_INPUT_DIV || CH == CH_PLAIN_INPUT_MUL) && (OUT & 3) != FWD_OUT_PACKED) {
    if (a.soft_reset == RESET_COUNT) {
      forward_body<S, VECTOR, ROUND_EACH, CH, RESET_COUNT, OUT, CKPT>(a);
      return;
    }
  }
  if (a.soft_reset)
    forward_body<S, VECTOR, ROUND_EACH, CH, RESET_SOFT, OUT, CKPT>(a);
  else
    forward_body<S, VECTOR, ROUND_EACH, CH, RESET_HARD, OUT, CKPT>(a);
}

template <typename S, bool VECTOR, bool ROUND_EACH, int OUT = FWD_OUT_DENSE>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) forward_kernel(const FwdArgs a) {
  switch (a.charge) {
    case CH_IF: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_IF, OUT>(a); break;
    case CH_DECAY_INPUT_DIV: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_DECAY_INPUT_DIV, OUT>(a); break;
    case CH_DECAY_INPUT_MUL: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_DECAY_INPUT_MUL, OUT>(a); break;
    case CH_PLAIN_INPUT_DIV: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_PLAIN_INPUT_DIV, OUT>(a); break;
    case CH_QIF_DIV: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_QIF_DIV, OUT>(a); break;
    case CH_QIF_MUL: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_QIF_MUL, OUT>(a); break;
    case CH_EIF_DIV: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_EIF_DIV, OUT>(a); break;
    case CH_EIF_MUL: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_EIF_MUL, OUT>(a); break;
    default: forward_reset_dispatch<S, VECTOR, ROUND_EACH, CH_PLAIN_INPUT_MUL, OUT>(a); break;
  }
}

// The forward of a long sequence that the backward will replay in pieces: the ordinary walk over all T steps, which
// also leaves the state after every a.chunk steps in a.checkpoints.
template <typename S, bool ROUND_EACH>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) forward_pieces_kernel(const FwdArgs a) {
  switch (a.charge) {
    case CH_IF: forward_reset_dispatch<S, true, ROUND_EACH, CH_IF, FWD_OUT_DENSE, true>(a); break;
    case CH_DECAY_INPUT_DIV: forward_reset_dispatch<S, true, ROUND_EACH, CH_DECAY_INPUT_DIV, FWD_OUT_DENSE, true>(a); break;
    case CH_DECAY_INPUT_MUL: forward_reset_dispatch<S, true, ROUND_EACH, CH_DECAY_INPUT_MUL, FWD_OUT_DENSE, true>(a); break;
    case CH_PLAIN_INPUT_DIV: forward_reset_dispatch<S, true, ROUND_EACH, CH_PLAIN_INPUT_DIV, FWD_OUT_DENSE, true>(a); break;
    case CH_QIF_DIV: forward_reset_dispatch<S, true, ROUND_EACH, CH_QIF_DIV, FWD_OUT_DENSE, true>(a); break;
    case CH_QIF_MUL: forward_reset_dispatch<S, true, ROUND_EACH, CH_QIF_MUL, FWD_OUT_DENSE, true>(a); break;
    case CH_EIF_DIV: forward_reset_dispatch<S, true, ROUND_EACH, CH_EIF_DIV, FWD_OUT_DENSE, true>(a); break;
    case CH_EIF_MUL: forward_reset_dispatch<S, true, ROUND_EACH, CH_EIF_MUL, FWD_OUT_DENSE, true>(a); break;
    default: forward_reset_dispatch<S, true, ROUND_EACH, CH_PLAIN_INPUT_MUL, FWD_OUT_DENSE, true>(a); break;
  }
}

// ---- host side: turn the ABI parameters into kernel arguments ------------------------------------
inline int build_fwd_args(FwdArgs &a, bool &round_each, int neuron, int dtype, const sjhip_neuron_params &p,
                          int64_t T, int64_t N, const void *x_seq, const void *v_init, const float *k_device,
                          void *spike_seq, void *v_seq, void *v_last, void *h_seq) {
  a.x = x_seq; a.v_init = v_init; a.spike = spike_seq; a.v_seq = v_seq; a.v_last = v_last; a.h = h_seq;
  a.k_device = nullptr;
  a.checkpoints = nullptr; a.chunk = 0;
  a.T = T; a.N = N;
  a.spread = column_spread(N * (dtype == SJHIP_F32 ? 4 : 2), T);
  const bool ilif = neuron == SJHIP_NEURON_ILIF;
  a.soft_reset = ilif ? RESET_COUNT : ((p.flags & SJHIP_FLAG_SOFT_RESET) ? RESET_SOFT : RESET_HARD);
  a.level_max = p.level_max;
  a.vth_inv = (ilif && exact_reciprocal(p.v_threshold))
                  ? 1.0f / p.v_threshold : 0.0f;
  a.v_init_broadcast = (p.flags & SJHIP_FLAG_V_INIT_BROADCAST) ? 1 : 0;
  const bool decay_input = !ilif && (p.flags & SJHIP_FLAG_DECAY_INPUT) != 0;
  round_each = dtype != SJHIP_F32 && !(p.flags & SJHIP_FLAG_FP32_STATE);

  a.tau = p.tau;
  if (neuron == SJHIP_NEURON_IF) {
    a.charge = CH_IF;
  } else if (neuron == SJHIP_NEURON_PLIF) {
    a.charge = decay_input ? CH_DECAY_INPUT_MUL : CH_PLAIN_INPUT_MUL;
    a.k_device = k_device;
  } else {
    const bool qif = neuron == SJHIP_NEURON_QIF, eif = neuron == SJHIP_NEURON_EIF;
    if (!(p.tau > 0.0f) || !std::isfinite(p.tau)) return fail(SJHIP_ERR_INVALID, "forward: tau=%g", (double)p.tau);
    if (p.flags & SJHIP_FLAG_RECIPROCAL_TAU) {
      // fl(1/tau) from the double quotient, as the reference kernels receive it (multi_step/lif.py:338)
      a.tau = (float)(1.0 / (double)p.tau);
      a.charge = qif ? CH_QIF_MUL : eif ? CH_EIF_MUL : (decay_input ? CH_DECAY_INPUT_MUL : CH_PLAIN_INPUT_MUL);
    } else if (exact_reciprocal(p.tau)) {
      // x / 2^e == x * 2^-e bit for bit (both are exact scalings, subnormal results round identically)
      a.tau = 1.0f / p.tau;
      a.charge = qif ? CH_QIF_MUL : eif ? CH_EIF_MUL : (decay_input ? CH_DECAY_INPUT_MUL : CH_PLAIN_INPUT_MUL);
    } else {
      a.charge = qif ? CH_QIF_DIV : eif ? CH_EIF_DIV : (decay_input ? CH_DECAY_INPUT_DIV : CH_PLAIN_INPUT_DIV);
    }
  }

  // The torch CPU backend rounds a Python scalar to the tensor dtype before add/sub and keeps it in
  // fp32 for mul/div; mirror that when every op is rounded to a 16-bit storage dtype.
  a.vr_mul = p.v_reset;
  a.vth_mul = p.v_threshold;
  a.vr_add = ilif ? 0.0f : p.v_reset;  // ILIF charges with v_reset = None, i.e. the offset 0.0
  a.vth_sub = p.v_threshold;
  a.q_rest_sub = p.v_rest;
  a.q_c_sub = p.v_c;
  a.q_a0_mul = p.a0;
  if (round_each) {
    if (dtype == SJHIP_F16) {
      a.vr_add = Cvt<f16_t>::round(p.v_reset); a.vth_sub = Cvt<f16_t>::round(p.v_threshold);
      a.q_rest_sub = Cvt<f16_t>::round(p.v_rest); a.q_c_sub = Cvt<f16_t>::round(p.v_c);
    } else {
      a.vr_add = Cvt<bf16_t>::round(p.v_reset); a.vth_sub = Cvt<bf16_t>::round(p.v_threshold);
      a.q_rest_sub = Cvt<bf16_t>::round(p.v_rest); a.q_c_sub = Cvt<bf16_t>::round(p.v_c);
    }
  }

  return SJHIP_OK;
}

}  // namespace sjhip
