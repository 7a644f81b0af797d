/*
 * sj_oracle.c -- plain-C scalar restatement of the reference torch backend of SpikingJelly's
 * multi-step IF / LIF / PLIF neurons, their BPTT and the spike bit-packing.  TEST INFRASTRUCTURE
 * ONLY: built into oracle/_build/libsjoracle.so by oracle/Makefile and loaded by tests, the smoke
 * check and bench.py's cpu_baseline leg; no product code links or loads it.
 *
 * Compile with -O2 -ffp-contract=off -fno-fast-math (x86-64 SSE2: every float op is one IEEE
 * single-precision operation, no excess precision, no fused multiply-add).
 *
 * Reference lines restated (paths relative to spikingjelly/activation_based):
 *   charge     functional/neuron.py:310 (IF), :849-852 (LIF), :1290-1295 (PLIF)
 *   fire       surrogate.py:60   (x >= 0).to(x)   on   h - v_threshold
 *   reset      functional/neuron.py:225-228
 *   BPTT       cuda_kernel/neuron_kernel/multi_step/base.py:293-409, lif.py:89-102, plif.py:143-203
 *   surrogate' surrogate.py:769-771 (Sigmoid), :1247-1250 (ATan), :401-407, :595-596, :936-937,
 *              :1101-1102, :1610-1613
 *   bit-pack   triton_kernel/compress.py:19-44
 */
#define _USE_MATH_DEFINES
#define _GNU_SOURCE
#include <math.h>
#include <stddef.h>
#include <stdint.h>

enum { SJO_IF = 0, SJO_LIF = 1, SJO_PLIF = 2 };

/*
 * Forward.  x_seq [T,N], v_init [N]; outputs spike_seq, v_seq, h_seq [T,N] (each may be NULL).
 * tau: LIF divisor (IEEE division) ; PLIF multiplier k ; ignored for IF.
 * soft_reset != 0: v = h - s*v_th and the charge offset is 0 (v_reset=None in the reference).
 */
void sjo_forward_f32(int neuron, int64_t T, int64_t N, const float *x_seq, const float *v_init,
                     float *spike_seq, float *v_seq, float *h_seq, float *v_last,
                     float tau, int decay_input, float v_th, float v_reset, int soft_reset) {
  const float vr = soft_reset ? 0.0f : v_reset;
  for (int64_t n = 0; n < N; ++n) {
    float v = v_init[n];
    for (int64_t t = 0; t < T; ++t) {
      const float x = x_seq[t * N + n];
      float h;
      if (neuron == SJO_IF) {
        h = v + x;
      } else if (neuron == SJO_LIF) {
        if (decay_input) {
          float d = v - vr; float e = x - d; float f = e / tau; h = v + f;
        } else {
          float d = v - vr; float f = d / tau; float g = v - f; h = g + x;
        }
      } else {
        if (decay_input) {
          float d = v - vr; float e = x - d; float f = e * tau; h = v + f;
        } else {
          float d = v - vr; float f = d * tau; float g = v - f; h = g + x;
        }
      }
      const float over = h - v_th;
      const float s = (over >= 0.0f) ? 1.0f : 0.0f;
      if (soft_reset) {
        float m = s * v_th; v = h - m;
      } else {
        float m = s * v_reset; float q = 1.0f - s; float o = q * h; v = m + o;
      }
      if (spike_seq) spike_seq[t * N + n] = s;
      if (v_seq) v_seq[t * N + n] = v;
      if (h_seq) h_seq[t * N + n] = h;
    }
    if (v_last) v_last[n] = v;
  }
}

static double sg_prime(int sg_id, double x, double alpha) {
  switch (sg_id) {
    case 0: { double s = 1.0 / (1.0 + exp(-alpha * x)); return (1.0 - s) * s * alpha; }
    case 1: { double a = alpha / 2.0; double ax = M_PI * a * x; return a / (1.0 + ax * ax); }
    case 2: { double ax = fabs(x); return ax > 1.0 / alpha ? 0.0 : -(alpha * alpha) * ax + alpha; }
    case 3: return alpha / 2.0 * exp(-alpha * fabs(x));
    case 4: { double d = 1.0 / alpha + fabs(x); return 1.0 / (2.0 * alpha * d * d); }
    case 5: { double d = fabs(x) + 1.0; return alpha / (d * d); }
    default: { double ax = x * alpha; return exp(-(ax * ax)) * (alpha / sqrt(M_PI)); }
  }
}

/*
 * BPTT in double precision from fp32 inputs.  grad_v_seq / grad_v_last may be NULL.
 * k = 1/tau (LIF) or sigmoid(w) (PLIF).  For PLIF x_seq and v_prev (v_init followed by v_seq[0..T-2],
 * given as v_init + v_seq) are needed for dL/dk; grad_k may be NULL otherwise.
 */
void sjo_backward_f64(int neuron, int64_t T, int64_t N, const float *grad_spike_seq, const float *grad_v_seq,
                      const float *grad_v_last, const float *h_seq, const float *x_seq, const float *v_init,
                      const float *v_seq, double *grad_x_seq, double *grad_v_init, double *grad_k,
                      double k, int decay_input, double v_th, double v_reset, int soft_reset,
                      int detach_reset, int sg_id, double alpha) {
  const double kx = neuron == SJO_IF ? 1.0 : (decay_input ? k : 1.0);
  const double km = neuron == SJO_IF ? 1.0 : 1.0 - k;
  const double live = detach_reset ? 0.0 : 1.0;
  const double vr = soft_reset ? 0.0 : v_reset;
  double gk = 0.0;
  for (int64_t n = 0; n < N; ++n) {
    double carry = grad_v_last ? (double)grad_v_last[n] : 0.0;
    for (int64_t t = T - 1; t >= 0; --t) {
      const double h = h_seq[t * N + n];
      const double over = h - v_th;
      const double sg = sg_prime(sg_id, over, alpha);
      const double s = over >= 0.0 ? 1.0 : 0.0;
      const double dvdh = soft_reset ? 1.0 - live * v_th * sg : (1.0 - s) + live * (v_reset - h) * sg;
      const double gv = carry + (grad_v_seq ? (double)grad_v_seq[t * N + n] : 0.0);
      const double G = gv * dvdh + (double)grad_spike_seq[t * N + n] * sg;
      grad_x_seq[t * N + n] = G * kx;
      carry = G * km;
      if (neuron == SJO_PLIF && grad_k) {
        const double vp = t == 0 ? (double)v_init[n] : (double)v_seq[(t - 1) * N + n];
        gk += G * (decay_input ? ((double)x_seq[t * N + n] - (vp - vr)) : (vr - vp));
      }
    }
    grad_v_init[n] = carry;
  }
  if (grad_k) *grad_k = gk;
}

/* byte j bit i = (src[8j+i] != 0); pad bits 0.  esize = 4 (fp32), 2 (fp16/bf16 patterns), 1 (u8). */
void sjo_bit_pack(int esize, int64_t n, const void *src, uint8_t *dst) {
  const int64_t nbytes = (n + 7) / 8;
  for (int64_t j = 0; j < nbytes; ++j) {
    unsigned b = 0;
    for (int i = 0; i < 8; ++i) {
      const int64_t e = 8 * j + i;
      if (e >= n) break;
      int nz;
      if (esize == 4) nz = (((const uint32_t *)src)[e] & 0x7fffffffu) != 0;
      else if (esize == 2) nz = (((const uint16_t *)src)[e] & 0x7fffu) != 0;
      else nz = ((const uint8_t *)src)[e] != 0;
      if (nz) b |= 1u << i;
    }
    dst[j] = (uint8_t)b;
  }
}

void sjo_bit_unpack_u8(int64_t n, const uint8_t *src, uint8_t *dst) {
  for (int64_t e = 0; e < n; ++e) dst[e] = (src[e >> 3] >> (e & 7)) & 1u;
}
