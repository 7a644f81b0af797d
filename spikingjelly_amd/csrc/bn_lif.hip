// Batch normalisation fused with the multi-step neuron that follows it, for activations laid out [T, B, C, L]
// (time, batch, channels, positions; L contiguous): the block  conv -> BatchNorm1d / BatchNorm2d -> LIFNode  of the
// reference's spiking self-attention and Spikformer stem (layer/attention.py:310-329, 370-384;
// model/spikformer.py:16-99, 107-212), where torch runs batch norm and the neuron as separate passes over the tensor.
//
// Training forward:  bn_stats_kernel reads the convolution output y once (one wavefront per (sample, channel) row,
//   fp32 partial sums of y and y^2), bn_finalize_kernel combines them in fp64 into the per-channel affine map
//   z = y a_c + b_c  (a_c = gamma_c / sqrt(var_c + eps), b_c = beta_c - mean_c a_c) and updates the running statistics,
//   bn_lif_forward_kernel reads y a second time, applies the map and runs the neuron over the T steps in registers,
//   writing spikes dense or bit-packed.  The normalised tensor never exists in memory.  In evaluation mode the map
//   comes from the running statistics and the first pass is skipped.
// Backward:  bn_lif_backward_kernel replays the neuron from y (the forward's own arithmetic, so the replayed h has its
//   bits), walks the BPTT recurrence and writes g = dL/dz; a wavefront owns one (batch, channel) row for all T steps and
//   leaves sum g and sum g y of its row.  bn_backward_finalize_kernel turns those into dgamma, dbeta and the three
//   per-channel coefficients of  dy = p_c g + q_c y + r_c,  which bn_grad_input_kernel applies (in place over g).
// Arithmetic of the neuron is neuron_step / surrogate_grad of the plain neuron kernels.
#include "neuron_bwd.h"
#include "neuron_fwd.h"

namespace sjhip {

namespace {

struct BnLifFwdArgs {
  FwdArgs f;           // x = y [T][N], N = B * C * L
  const float *scale;  // [C]
  const float *shift;  // [C]
  int C, L;
};

struct BnLifBwdArgs {
  FwdArgs f;
  BwdArgs b;           // grad_spike, grad_v_last, grad_x (= g out), grad_v_init
  const float *scale;
  const float *shift;
  float *partial;      // [B * C][2]: sum g, sum g y of the row
  float *k_partial;    // PLIF: [4 x blocks] shares of dL/dk, one per wavefront
  int C, L;
  int64_t rows;        // B * C
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  return v;
}
// the same for a double, in a fixed order; every lane ends up with the total
__device__ __forceinline__ double wave_sum_all(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Sums of two per-work-item values over the rows of a block in which work-item tid holds a piece of row r_local
// (consecutive work-items, consecutive rows): per wavefront one masked reduction per row it touches, the results left
// in LDS, then one work-item per row adds the wavefronts' shares in their order and writes (sum0, sum1) of row
// first_row + r to out[2 (first_row + r)].  Every work-item of the block must call it.
constexpr int kBnRowsMax = 16;  // rows per block: rows of at least 16 quads
__device__ __forceinline__ void block_row_sums(float (&part)[4][kBnRowsMax][2], int r_local, bool valid, int rows_per_block,
                                               float v0, float v1, float *out, int64_t first_row, int64_t rows) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (lane < rows_per_block) { part[wave][lane][0] = 0.0f; part[wave][lane][1] = 0.0f; }
  const int r_first = __builtin_amdgcn_readfirstlane(r_local);
  const int r_last = __builtin_amdgcn_readlane(r_local, 63);
  for (int r = r_first; r <= r_last; ++r) {
    const bool mine = valid && r_local == r;
    const float s0 = wave_sum(mine ? v0 : 0.0f), s1 = wave_sum(mine ? v1 : 0.0f);
    if (lane == 0) { part[wave][r][0] = s0; part[wave][r][1] = s1; }
  }
  __syncthreads();
  if (tid < rows_per_block && first_row + tid < rows) {
    float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) { s0 += part[w][tid][0]; s1 += part[w][tid][1]; }
    out[2 * (first_row + tid)] = s0;
    out[2 * (first_row + tid) + 1] = s1;
  }
}

// one wavefront per row of L contiguous elements: sum and sum of squares.  A wavefront takes kBnStatRows rows in a
// row of at most 256 elements and has their loads all in flight before the first sum (37 -> 31 us on
// [256, 1152, 196]); several whole rows per block with the row sums through LDS, as in bn_lif_backward_rows_kernel,
// measured slower (52 us)
constexpr int kBnStatRows = 4;
__global__ void __launch_bounds__(256) bn_stats_kernel(const float *y, int64_t rows, int L, float *partial) {
  const int lane = threadIdx.x & 63;
  const int64_t row0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * kBnStatRows;
  if (row0 >= rows) return;
  const int quads = L / 4;
  if (quads <= 64) {
    f32x4 v[kBnStatRows];
#pragma unroll
    for (int r = 0; r < kBnStatRows; ++r) {
      const bool ok = row0 + r < rows && lane < quads;
      v[r] = ok ? reinterpret_cast<const f32x4 *>(y + (row0 + r) * L)[lane] : (f32x4)(0.0f);
    }
#pragma unroll
    for (int r = 0; r < kBnStatRows; ++r) {
      float s = (v[r].x + v[r].y) + (v[r].z + v[r].w);
      float q = v[r].x * v[r].x;
      q = fmaf(v[r].y, v[r].y, q); q = fmaf(v[r].z, v[r].z, q); q = fmaf(v[r].w, v[r].w, q);
      s = wave_sum(s);
      q = wave_sum(q);
      if (lane == 0 && row0 + r < rows) { partial[2 * (row0 + r)] = s; partial[2 * (row0 + r) + 1] = q; }
    }
    return;
  }
  for (int r = 0; r < kBnStatRows && row0 + r < rows; ++r) {
    const f32x4 *p = reinterpret_cast<const f32x4 *>(y + (row0 + r) * L);
    float s = 0.0f, q = 0.0f;
    for (int i = lane; i < quads; i += 64) {
      const f32x4 v = p[i];
      s += (v.x + v.y) + (v.z + v.w);
      q = fmaf(v.x, v.x, q); q = fmaf(v.y, v.y, q); q = fmaf(v.z, v.z, q); q = fmaf(v.w, v.w, q);
    }
    s = wave_sum(s);
    q = wave_sum(q);
    if (lane == 0) { partial[2 * (row0 + r)] = s; partial[2 * (row0 + r) + 1] = q; }
  }
}

// partial == nullptr: evaluation mode, the map comes from the running statistics (which stay as they are)
__global__ void __launch_bounds__(256) bn_finalize_kernel(const float *partial, int64_t S, int C, int64_t count,
                                                           const float *gamma, const float *beta, float eps,
                                                           float momentum, float *running_mean, float *running_var,
                                                           float *scale, float *shift, float *mean_out, float *invstd_out,
                                                           int64_t *batches_tracked) {
  // one wavefront per channel: lanes stride over the samples, then a butterfly sum
  if (batches_tracked && blockIdx.x == 0 && threadIdx.x == 0) *batches_tracked += 1;
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= C) return;
  double mean, var;
  if (partial) {
    double s = 0.0, q = 0.0;
    for (int64_t i = lane; i < S; i += 64) { s += (double)partial[2 * (i * C + c)]; q += (double)partial[2 * (i * C + c) + 1]; }
    s = wave_sum_all(s);
    q = wave_sum_all(q);
    if (lane != 0) return;
    mean = s / (double)count;
    var = q / (double)count - mean * mean;
    if (var < 0.0) var = 0.0;
    if (running_mean) running_mean[c] = (float)((1.0 - (double)momentum) * (double)running_mean[c] + (double)momentum * mean);
    if (running_var) {
      const double unbiased = count > 1 ? var * (double)count / (double)(count - 1) : var;
      running_var[c] = (float)((1.0 - (double)momentum) * (double)running_var[c] + (double)momentum * unbiased);
    }
  } else {
    if (lane != 0) return;
    mean = (double)running_mean[c];
    var = (double)running_var[c];
  }
  const double invstd = 1.0 / sqrt(var + (double)eps);
  const double g = gamma ? (double)gamma[c] : 1.0, b = beta ? (double)beta[c] : 0.0;
  const double a = g * invstd;
  scale[c] = (float)a;
  shift[c] = (float)(b - mean * a);
  mean_out[c] = (float)mean;
  invstd_out[c] = (float)invstd;
}

template <int CH, int RS, bool PACKED>
__device__ __forceinline__ void bn_lif_forward_body(const BnLifFwdArgs &a) {
  typedef Acc<float, true, false> A;
  const FwdArgs &f = a.f;
  const int64_t N = f.N, T = f.T;
  const int64_t col = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (col >= N) return;
  // (32-bit quotients where the tensor allows it: a 64-bit integer division is some hundred instructions, as many as
  // the four steps of a short sequence)
  const int c = N <= 0x7fffffffLL ? (int)(((uint32_t)col / (uint32_t)a.L) % (uint32_t)a.C) : (int)((col / a.L) % a.C);
  const float sc = a.scale[c], sh = a.shift[c];
  const float tau = f.k_device ? *f.k_device : f.tau;  // PLIF: k = sigmoid(w), read where torch left it
  const float *yp = (const float *)f.x + col;
  float *sp = (float *)f.spike + col;
  float v[4];
  load_state<float, true, false>(f.v_init, col, f.v_init_broadcast != 0, v);
  constexpr int PF = 4;
  for (int64_t t0 = 0; t0 < T; t0 += PF) {
    f32x4 rows[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) rows[i] = (t0 + i < T) ? A::load(yp + (t0 + i) * N) : A::zero();
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 + i;
      if (t < T) {
        float y[4], h[4], s[4];
        A::unpack(rows[i], y);
#pragma unroll
        for (int j = 0; j < 4; ++j) neuron_step<float, CH, RS>(fmaf(y[j], sc, sh), v[j], h[j], s[j], tau, f);
        if (PACKED) store_spike_bits<4>((uint8_t *)f.spike + t * (N >> 3), col, N, s);
        else A::store(sp + t * N, s);
      }
    }
  }
  if (f.v_last) A::store((float *)f.v_last + col, v);
}

template <int CH, bool PACKED> __device__ __forceinline__ void bn_lif_forward_reset(const BnLifFwdArgs &a) {
  if (a.f.soft_reset) bn_lif_forward_body<CH, RESET_SOFT, PACKED>(a);
  else bn_lif_forward_body<CH, RESET_HARD, PACKED>(a);
}

template <bool PACKED> __global__ void __launch_bounds__(256) bn_lif_forward_kernel(const BnLifFwdArgs a) {
  switch (a.f.charge) {
    case CH_IF: bn_lif_forward_reset<CH_IF, PACKED>(a); break;
    case CH_DECAY_INPUT_DIV: bn_lif_forward_reset<CH_DECAY_INPUT_DIV, PACKED>(a); break;
    case CH_DECAY_INPUT_MUL: bn_lif_forward_reset<CH_DECAY_INPUT_MUL, PACKED>(a); break;
    case CH_PLAIN_INPUT_DIV: bn_lif_forward_reset<CH_PLAIN_INPUT_DIV, PACKED>(a); break;
    default: bn_lif_forward_reset<CH_PLAIN_INPUT_MUL, PACKED>(a); break;
  }
}

// h of every step of this work-item's four neurons, replayed from y
template <int CH, int RS, int TMAX>
__device__ __forceinline__ void replay_h(const FwdArgs &f, int len, const f32x4 (&yv)[TMAX], float sc, float sh, float (&v)[4],
                                         float (&h)[TMAX][4]) {
  const float tau = f.k_device ? *f.k_device : f.tau;
#pragma unroll
  for (int t = 0; t < TMAX; ++t) {
    if (t < len) {
      const float y[4] = {yv[t].x, yv[t].y, yv[t].z, yv[t].w};
      float s;
#pragma unroll
      for (int j = 0; j < 4; ++j) neuron_step<float, CH, RS>(fmaf(y[j], sc, sh), v[j], h[t][j], s, tau, f);
    }
  }
}

template <int CH, int TMAX>
__device__ __forceinline__ void replay_h_reset(const FwdArgs &f, int len, const f32x4 (&yv)[TMAX], float sc, float sh,
                                               float (&v)[4], float (&h)[TMAX][4]) {
  if (f.soft_reset) replay_h<CH, RESET_SOFT, TMAX>(f, len, yv, sc, sh, v, h);
  else replay_h<CH, RESET_HARD, TMAX>(f, len, yv, sc, sh, v, h);
}

// the steps t0 .. t0 + len - 1 (len <= TMAX) of this work-item's four neurons from the state v in front of step t0
template <int TMAX>
__device__ __forceinline__ void replay_h_charge(const FwdArgs &f, int len, const f32x4 (&yv)[TMAX], float sc, float sh,
                                                float (&v)[4], float (&h)[TMAX][4]) {
  switch (f.charge) {
    case CH_IF: replay_h_reset<CH_IF, TMAX>(f, len, yv, sc, sh, v, h); break;
    case CH_DECAY_INPUT_DIV: replay_h_reset<CH_DECAY_INPUT_DIV, TMAX>(f, len, yv, sc, sh, v, h); break;
    case CH_DECAY_INPUT_MUL: replay_h_reset<CH_DECAY_INPUT_MUL, TMAX>(f, len, yv, sc, sh, v, h); break;
    case CH_PLAIN_INPUT_DIV: replay_h_reset<CH_PLAIN_INPUT_DIV, TMAX>(f, len, yv, sc, sh, v, h); break;
    default: replay_h_reset<CH_PLAIN_INPUT_MUL, TMAX>(f, len, yv, sc, sh, v, h); break;
  }
}

// BPTT over the replayed h (recurrence of neuron_bwd.h); writes g = dL/dz and adds this work-item's share of
// sum g and sum g y.  PLIF: also of dL/dk = sum G_t dh_t/dk, dh_t/dk = (h_t - v_{t-1}) / k with input decay (the division
// is left to the final reduction) or v_reset - v_{t-1} without; v_{t-1} is re-derived from h_{t-1} with the forward's
// reset arithmetic, v0 is the state in front of the first of these steps.
template <int SG, int TMAX, bool PLIF>
__device__ __forceinline__ void bptt_rows(const BwdArgs &b, float k, int64_t col, int64_t t0, int len, const f32x4 (&yv)[TMAX],
                                          const float (&h)[TMAX][4], const float (&v0)[4], float (&carry)[4], float &acc_g,
                                          float &acc_gy, float &acc_k) {
#pragma clang fp contract(fast)
  typedef Acc<float, true, true> A;
  const int64_t N = b.N;
  const float *gsp = (const float *)b.grad_spike + col + t0 * N;
  float *gxp = (float *)b.grad_x + col + t0 * N;
  const float kx = b.is_if ? 1.0f : (b.decay_input ? k : 1.0f);
  const float km = b.is_if ? 1.0f : (1.0f - k);
#pragma unroll
  for (int t = TMAX - 1; t >= 0; --t) {
    if (t < len) {
      float gs[4], gz[4];
      A::unpack(A::load(gsp + (int64_t)t * N), gs);
      const float y[4] = {yv[t].x, yv[t].y, yv[t].z, yv[t].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float over = h[t][j] - b.v_th;
        const float s = (over >= 0.0f) ? 1.0f : 0.0f;
        const float sg = surrogate_grad<SG, true>(over, b.alpha);  // hardware exp2 and reciprocal (1 ulp each): this kernel is bound by its arithmetic
        const float dvdh = (1.0f - s * b.cB) + (b.cC - h[t][j] * b.cD) * sg;
        const float G = carry[j] * dvdh + gs[j] * sg;
        gz[j] = G * kx;
        carry[j] = G * km;
        acc_g += gz[j];
        acc_gy = fmaf(gz[j], y[j], acc_gy);
        if constexpr (PLIF) {
          float v_prev = v0[j];
          if (t > 0) {
            const float h_prev = h[t > 0 ? t - 1 : 0][j];
            v_prev = reset_as_forward(h_prev, (h_prev - b.v_th >= 0.0f) ? 1.0f : 0.0f, b);
          }
          acc_k = fmaf(G, b.decay_input ? (h[t][j] - v_prev) : (b.v_reset - v_prev), acc_k);
        }
      }
      Acc<float, true, false>::store(gxp + (int64_t)t * N, gz);  // read again by the next kernel
    }
  }
}

template <int TMAX, bool PLIF>
__device__ __forceinline__ void bptt_rows_surrogate(const BwdArgs &b, float k, int64_t col, int64_t t0, int len,
                                                    const f32x4 (&yv)[TMAX], const float (&h)[TMAX][4], const float (&v0)[4],
                                                    float (&carry)[4], float &acc_g, float &acc_gy, float &acc_k) {
  switch (b.sg) {
    case SJHIP_SG_SIGMOID: bptt_rows<SJHIP_SG_SIGMOID, TMAX, PLIF>(b, k, col, t0, len, yv, h, v0, carry, acc_g, acc_gy, acc_k); break;
    case SJHIP_SG_ATAN: bptt_rows<SJHIP_SG_ATAN, TMAX, PLIF>(b, k, col, t0, len, yv, h, v0, carry, acc_g, acc_gy, acc_k); break;
    case SJHIP_SG_PIECEWISE_QUADRATIC: bptt_rows<SJHIP_SG_PIECEWISE_QUADRATIC, TMAX, PLIF>(b, k, col, t0, len, yv, h, v0, carry, acc_g, acc_gy, acc_k); break;
    case SJHIP_SG_PIECEWISE_EXP: bptt_rows<SJHIP_SG_PIECEWISE_EXP, TMAX, PLIF>(b, k, col, t0, len, yv, h, v0, carry, acc_g, acc_gy, acc_k); break;
    case SJHIP_SG_SOFT_SIGN: bptt_rows<SJHIP_SG_SOFT_SIGN, TMAX, PLIF>(b, k, col, t0, len, yv, h, v0, carry, acc_g, acc_gy, acc_k); break;
    case SJHIP_SG_SUPER_SPIKE: bptt_rows<SJHIP_SG_SUPER_SPIKE, TMAX, PLIF>(b, k, col, t0, len, yv, h, v0, carry, acc_g, acc_gy, acc_k); break;
    default: bptt_rows<SJHIP_SG_ERF, TMAX, PLIF>(b, k, col, t0, len, yv, h, v0, carry, acc_g, acc_gy, acc_k); break;
  }
}

// One work-item's four neurons (quad q of row `row`) for all T steps: replay, BPTT, g written, the sums extended.
template <int TMAX, bool PLIF>
__device__ __forceinline__ void bn_lif_backward_quad(const BnLifBwdArgs &a, int64_t row, int q, float &acc_g, float &acc_gy,
                                                     float &acc_k) {
  typedef Acc<float, true, false> A;
  const FwdArgs &f = a.f;
  const BwdArgs &b = a.b;
  const int c = (int)(row % a.C);
  const float sc = a.scale[c], sh = a.shift[c];
  const float k = (PLIF && b.k_device) ? *b.k_device : b.k;
  const int64_t N = f.N;
  const int64_t col = row * a.L + 4 * q;
  const float *yp = (const float *)f.x + col;
  f32x4 yv[TMAX];
#pragma unroll
  for (int t = 0; t < TMAX; ++t) yv[t] = (t < f.T) ? A::load(yp + (int64_t)t * N) : A::zero();
  float v[4], h[TMAX][4], carry[4];
  load_state<float, true, false>(f.v_init, col, f.v_init_broadcast != 0, v);
  const float v0[4] = {v[0], v[1], v[2], v[3]};
  if (b.grad_v_last) A::unpack(A::load((const float *)b.grad_v_last + col), carry);
  else carry[0] = carry[1] = carry[2] = carry[3] = 0.0f;
  replay_h_charge<TMAX>(f, (int)f.T, yv, sc, sh, v, h);
  bptt_rows_surrogate<TMAX, PLIF>(b, k, col, 0, (int)b.T, yv, h, v0, carry, acc_g, acc_gy, acc_k);
  if (b.grad_v_init) A::store((float *)b.grad_v_init + col, carry);
}

// The same for a sequence of more than kBnPiece steps, walked in pieces of kBnPiece as the plain neuron's replay over
// pieces does: a first pass replays the whole sequence and parks the state in front of every piece in LDS (each
// work-item its own 16 bytes per piece, no barrier), then the pieces are taken from the last to the first, each
// replayed from its parked state into registers and walked backwards; y is read twice.
constexpr int kBnPiece = 16;
constexpr int kBnMaxPieces = 16;  // 256 work-items x 16 bytes x 16 pieces = 64 KiB of LDS
template <bool PLIF>
__device__ __forceinline__ void bn_lif_backward_quad_long(const BnLifBwdArgs &a, int64_t row, int q, float &acc_g, float &acc_gy,
                                                          float &acc_k, f32x4 *parked) {
  typedef Acc<float, true, false> A;
  const FwdArgs &f = a.f;
  const BwdArgs &b = a.b;
  const int c = (int)(row % a.C);
  const float sc = a.scale[c], sh = a.shift[c];
  const int64_t N = f.N;
  const int64_t col = row * a.L + 4 * q;
  const float *yp = (const float *)f.x + col;
  const int T = (int)f.T, pieces = (T + kBnPiece - 1) / kBnPiece;
  f32x4 yv[kBnPiece];
  float v[4], h[kBnPiece][4], carry[4];
  load_state<float, true, false>(f.v_init, col, f.v_init_broadcast != 0, v);
  for (int p = 0; p + 1 < pieces; ++p) {  // (the pieces in front of the last one are whole)
    parked[p * blockDim.x] = f32x4{v[0], v[1], v[2], v[3]};
#pragma unroll
    for (int t = 0; t < kBnPiece; ++t) yv[t] = A::load(yp + (int64_t)(p * kBnPiece + t) * N);
    replay_h_charge<kBnPiece>(f, kBnPiece, yv, sc, sh, v, h);
  }
  parked[(pieces - 1) * blockDim.x] = f32x4{v[0], v[1], v[2], v[3]};
  if (b.grad_v_last) A::unpack(A::load((const float *)b.grad_v_last + col), carry);
  else carry[0] = carry[1] = carry[2] = carry[3] = 0.0f;
  for (int p = pieces - 1; p >= 0; --p) {
    const int t0 = p * kBnPiece, len = min(kBnPiece, T - t0);
#pragma unroll
    for (int t = 0; t < kBnPiece; ++t) yv[t] = (t < len) ? A::load(yp + (int64_t)(t0 + t) * N) : A::zero();
    const f32x4 s = parked[p * blockDim.x];
    v[0] = s.x; v[1] = s.y; v[2] = s.z; v[3] = s.w;
    const float v0[4] = {s.x, s.y, s.z, s.w};
    replay_h_charge<kBnPiece>(f, len, yv, sc, sh, v, h);
    bptt_rows_surrogate<kBnPiece, PLIF>(b, (PLIF && b.k_device) ? *b.k_device : b.k, col, t0, len, yv, h, v0, carry, acc_g,
                                        acc_gy, acc_k);
  }
  if (b.grad_v_init) A::store((float *)b.grad_v_init + col, carry);
}

// A wavefront per row; lanes stride over the row's quads.
// (TMAX = 0: the walk in pieces, with pieces x 256 x 16 bytes of dynamic LDS)
// PLIF: every wavefront also leaves its share of dL/dk in k_partial[4 * block + wavefront] (summed afterwards in a fixed
// order by plif_reduce_kernel, which also divides by k where the charge calls for it).
template <int TMAX, bool PLIF> __global__ void __launch_bounds__(256) bn_lif_backward_kernel(const BnLifBwdArgs a) {
  extern __shared__ f32x4 parked_states[];
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.rows) {
    if (PLIF && lane == 0) a.k_partial[(int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)] = 0.0f;
    return;
  }
  float acc_g = 0.0f, acc_gy = 0.0f, acc_k = 0.0f;
  for (int q = lane; q < a.L / 4; q += 64) {
    if constexpr (TMAX == 0) bn_lif_backward_quad_long<PLIF>(a, row, q, acc_g, acc_gy, acc_k, parked_states + threadIdx.x);
    else bn_lif_backward_quad<TMAX, PLIF>(a, row, q, acc_g, acc_gy, acc_k);
  }
  acc_g = wave_sum(acc_g);
  acc_gy = wave_sum(acc_gy);
  if (PLIF) acc_k = wave_sum(acc_k);
  if (lane == 0) {
    a.partial[2 * row] = acc_g;
    a.partial[2 * row + 1] = acc_gy;
    if (PLIF) a.k_partial[(int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)] = acc_k;
  }
}

// Rows of fewer than 64 quads leave lanes of a wavefront-per-row kernel idle (196 positions: 49 of 64 working), and this
// kernel is bound by its arithmetic.  Here a block of 256 work-items takes as many whole rows as fit (five rows of 49
// quads: 245 working); a row's sums are formed per wavefront (a wavefront holds parts of a few rows: one masked
// reduction per row it touches), left in LDS, and added over the wavefronts in their order by one work-item per row,
// so the result does not depend on timing.
template <int TMAX, bool PLIF>
__global__ void __launch_bounds__(256) bn_lif_backward_rows_kernel(const BnLifBwdArgs a, int quads, int rows_per_block,
                                                                   float inv_quads) {
  __shared__ float part[4][kBnRowsMax][2];
  extern __shared__ f32x4 parked_states[];
  const int tid = threadIdx.x;
  int r_local = (int)(((float)tid + 0.5f) * inv_quads);  // tid / quads (exact: see div_tokens of ssa.hip)
  const int q = tid - r_local * quads;
  const int64_t row = (int64_t)blockIdx.x * rows_per_block + r_local;
  const bool valid = r_local < rows_per_block && row < a.rows;
  if (r_local >= rows_per_block) r_local = rows_per_block - 1;
  float acc_g = 0.0f, acc_gy = 0.0f, acc_k = 0.0f;
  if (valid) {
    if constexpr (TMAX == 0) bn_lif_backward_quad_long<PLIF>(a, row, q, acc_g, acc_gy, acc_k, parked_states + tid);
    else bn_lif_backward_quad<TMAX, PLIF>(a, row, q, acc_g, acc_gy, acc_k);
  }
  if (PLIF) {
    acc_k = wave_sum(acc_k);
    if ((tid & 63) == 0) a.k_partial[(int64_t)blockIdx.x * 4 + (tid >> 6)] = acc_k;
  }
  block_row_sums(part, r_local, valid, rows_per_block, acc_g, acc_gy, a.partial, (int64_t)blockIdx.x * rows_per_block, a.rows);
}

// dgamma, dbeta and the coefficients of dy = p g + q y + r; count = T * B * L elements per channel
__global__ void __launch_bounds__(256) bn_backward_finalize_kernel(const float *partial, int64_t B, int C, int64_t count,
                                                                    int training, const float *gamma, const float *mean,
                                                                    const float *invstd, float *dgamma, float *dbeta,
                                                                    float *coef, float *amax_reset, int64_t amax_floats) {
  if (amax_reset && blockIdx.x == 0)
    for (int64_t i = threadIdx.x; i < amax_floats; i += 256) amax_reset[i] = 0.0f;
  const int lane = threadIdx.x & 63;
  const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (c >= C) return;
  double sg = 0.0, sgy = 0.0;
  for (int64_t i = lane; i < B; i += 64) { sg += (double)partial[2 * (i * C + c)]; sgy += (double)partial[2 * (i * C + c) + 1]; }
  sg = wave_sum_all(sg);
  sgy = wave_sum_all(sgy);
  if (lane != 0) return;
  const double m = (double)mean[c], is = (double)invstd[c], g = gamma ? (double)gamma[c] : 1.0;
  const double dg = is * (sgy - m * sg);  // sum g (y - mean) invstd
  if (dgamma) dgamma[c] = (float)dg;
  if (dbeta) dbeta[c] = (float)sg;
  const double a = g * is;
  coef[c] = (float)a;
  if (training) {
    coef[C + c] = (float)(-a * dg * is / (double)count);
    coef[2 * C + c] = (float)(a * (dg * is * m - sg) / (double)count);
  } else {
    coef[C + c] = 0.0f;
    coef[2 * C + c] = 0.0f;
  }
}

// |x| of a number, 0 for an infinity or a NaN (they take no part in choosing the scale of the tensor)
__device__ __forceinline__ float finite_abs(float x) {
  const float a = fabsf(x);
  return a <= 3.4028234663852886e38f ? a : 0.0f;
}

// dy = p_c g + q_c y + r_c over the flattened [S * C * L] tensor; dy may be g itself.  With AMAX every block also folds
// the largest |dy| it wrote into word (block % SJHIP_PW_AMAX_FLOATS) of amax_bits, bit patterns of non-negative floats
// (they order like unsigned integers, and a maximum does not depend on the order it is taken in), with an atomic whose
// result is not used, so that the block does not wait for it; and every wavefront the largest |dy| of its sample into
// that sample's word, which follow the tensor's (one atomic when its lanes share a sample, else one per lane).
template <bool AMAX>
__global__ void __launch_bounds__(256) bn_grad_input_kernel(const float *g, const float *y, const float *coef, int64_t S, int C,
                                                             int L, int64_t n, float *dy, unsigned *amax_bits) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  float amax = 0.0f;
  int sample = -1;
  if (i < n) {
    int c;  // i = ((sample * C) + channel) * L + position
    if (n <= 0x7fffffffLL) {
      const uint32_t row = (uint32_t)i / (uint32_t)L, smp = row / (uint32_t)C;
      c = (int)(row - smp * (uint32_t)C);
      sample = (int)smp;
    } else {
      const int64_t row = i / L, smp = row / C;
      c = (int)(row - smp * C);
      sample = (int)smp;
    }
    const float p = coef[c], q = coef[C + c], r = coef[2 * C + c];
    const f32x4 gv = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(g + i));
    const f32x4 yv = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(y + i));
    f32x4 o;
    o.x = fmaf(p, gv.x, fmaf(q, yv.x, r));
    o.y = fmaf(p, gv.y, fmaf(q, yv.y, r));
    o.z = fmaf(p, gv.z, fmaf(q, yv.z, r));
    o.w = fmaf(p, gv.w, fmaf(q, yv.w, r));
    *reinterpret_cast<f32x4 *>(dy + i) = o;
    if (AMAX) amax = fmaxf(fmaxf(finite_abs(o.x), finite_abs(o.y)), fmaxf(finite_abs(o.z), finite_abs(o.w)));
  }
  if (AMAX) {
    // One atomic per block for the tensor's words and, when the block lies in one sample (nearly always: a sample is
    // many blocks long), one for that sample's word.
    __shared__ float part[4];
    __shared__ int part_sample[4];
    // (blocks that run at the same time belong to one sample: they fold into different words of it)
    unsigned *sample_bits = amax_bits + SJHIP_PW_AMAX_FLOATS + blockIdx.x % SJHIP_PW_AMAX_SAMPLE_WORDS;
    constexpr int64_t kW = SJHIP_PW_AMAX_SAMPLE_WORDS;
    const int first = __builtin_amdgcn_readfirstlane(sample);
    const bool one_sample = __all(sample == first || sample < 0);
    if (!one_sample && sample >= 0) atomicMax(sample_bits + kW * sample, __builtin_bit_cast(unsigned, amax));
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
    if ((threadIdx.x & 63) == 0) {
      part[threadIdx.x >> 6] = amax;
      part_sample[threadIdx.x >> 6] = one_sample ? first : -1;  // (-1: nothing left to fold for this wavefront)
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      float all = 0.0f, run = 0.0f;
      int run_sample = -1;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        all = fmaxf(all, part[w]);
        if (part_sample[w] < 0) continue;
        if (part_sample[w] != run_sample) {
          if (run_sample >= 0) atomicMax(sample_bits + kW * run_sample, __builtin_bit_cast(unsigned, run));
          run_sample = part_sample[w];
          run = 0.0f;
        }
        run = fmaxf(run, part[w]);
      }
      if (run_sample >= 0) atomicMax(sample_bits + kW * run_sample, __builtin_bit_cast(unsigned, run));
      atomicMax(amax_bits + blockIdx.x % SJHIP_PW_AMAX_FLOATS, __builtin_bit_cast(unsigned, all));
    }
  }
}

int check_layout(const char *what, int64_t T, int64_t B, int64_t C, int64_t L) {
  if (T < 1 || B < 1 || C < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "%s: T=%lld B=%lld C=%lld L=%lld must be >= 1", what, (long long)T, (long long)B, (long long)C, (long long)L);
  if (L % 4 != 0) return fail(SJHIP_ERR_UNSUPPORTED, "%s: L=%lld must be a multiple of 4", what, (long long)L);
  if (C > (1 << 24) || L > (1 << 24) || B * C > (int64_t(1) << 40) || T > (int64_t(1) << 40) / (B * C * L))
    return fail(SJHIP_ERR_TOO_LARGE, "%s: T=%lld B=%lld C=%lld L=%lld", what, (long long)T, (long long)B, (long long)C, (long long)L);
  return SJHIP_OK;
}

bool lif_like(int neuron) { return neuron == SJHIP_NEURON_IF || neuron == SJHIP_NEURON_LIF || neuron == SJHIP_NEURON_PLIF; }

}  // namespace

int launch_bn_stats(const float *y, int64_t S, int64_t C, int64_t L, float *partial, hipStream_t stream) {
  int rc = check_layout("bn_stats", 1, S, C, L);
  if (rc != SJHIP_OK) return rc;
  if (!aligned16(y)) return fail(SJHIP_ERR_UNSUPPORTED, "bn_stats: y must be 16-byte aligned");
  const int64_t rows = S * C, blocks = (rows + 4 * kBnStatRows - 1) / (4 * kBnStatRows);
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bn_stats: %lld rows", (long long)rows);
  ProfileScope prof(KC_BN_STATS, stream);
  hipLaunchKernelGGL(bn_stats_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, y, rows, (int)L, partial);
  return check_launch("bn_stats");
}

// partial [rows][C][2]: sums over `count` elements per channel in all
int launch_bn_finalize(const float *partial, int64_t rows, int64_t count, int64_t C, const float *gamma, const float *beta, float eps,
                       float momentum, float *running_mean, float *running_var, float *scale, float *shift, float *mean,
                       float *invstd, int64_t *batches_tracked, hipStream_t stream) {
  if (C < 1 || C > (1 << 24)) return fail(SJHIP_ERR_INVALID, "bn_finalize: C=%lld", (long long)C);
  if (!partial && (!running_mean || !running_var)) return fail(SJHIP_ERR_INVALID, "bn_finalize: evaluation mode needs the running statistics");
  hipLaunchKernelGGL(bn_finalize_kernel, dim3((unsigned)((C + 3) / 4)), dim3(256), 0, stream, partial, rows, (int)C, count, gamma,
                     beta, eps, momentum, running_mean, running_var, scale, shift, mean, invstd, batches_tracked);
  return check_launch("bn_finalize");
}

int launch_bn_lif_forward(int neuron, const sjhip_neuron_params &p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                          const float *scale, const float *shift, const float *v_init, const float *k_device, float *spike_seq,
                          uint8_t *spike_bits, float *v_last, hipStream_t stream) {
  int rc = check_layout("bn_lif_forward", T, B, C, L);
  if (rc != SJHIP_OK) return rc;
  if (!lif_like(neuron)) return fail(SJHIP_ERR_UNSUPPORTED, "bn_lif_forward: neuron %d (IF, LIF and PLIF only)", neuron);
  if ((neuron == SJHIP_NEURON_PLIF) != (k_device != nullptr))
    return fail(SJHIP_ERR_INVALID, "bn_lif_forward: k in device memory goes with PLIF and only with it");
  const int64_t N = B * C * L;
  const bool broadcast = (p.flags & SJHIP_FLAG_V_INIT_BROADCAST) != 0;
  if (!aligned16(y) || (!broadcast && !aligned16(v_init)) || (spike_seq && !aligned16(spike_seq)) || (v_last && !aligned16(v_last)))
    return fail(SJHIP_ERR_UNSUPPORTED, "bn_lif_forward: tensors must be 16-byte aligned");
  if (spike_bits && N % 8 != 0) return fail(SJHIP_ERR_UNSUPPORTED, "bn_lif_forward: B*C*L=%lld must be a multiple of 8 for bit-packed spikes", (long long)N);
  BnLifFwdArgs a;
  bool round_each = false;
  rc = build_fwd_args(a.f, round_each, neuron, SJHIP_F32, p, T, N, y, v_init, k_device,
                      spike_bits ? (void *)spike_bits : (void *)spike_seq, nullptr, v_last, nullptr);
  if (rc != SJHIP_OK) return rc;
  a.scale = scale; a.shift = shift; a.C = (int)C; a.L = (int)L;
  const int64_t blocks = (N / 4 + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bn_lif_forward: N=%lld", (long long)N);
  ProfileScope prof(KC_BN_LIF_FORWARD, stream);
  if (spike_bits) hipLaunchKernelGGL((bn_lif_forward_kernel<true>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL((bn_lif_forward_kernel<false>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return check_launch("bn_lif_forward");
}

// wavefront shares of dL/dk: four per block of either backward kernel (the one with fewer rows per block bounds it)
int64_t bn_lif_backward_k_workspace_floats(int64_t B, int64_t C, int64_t L) {
  (void)L;
  return 4 * ((B * C + 3) / 4) + 4;
}

int launch_bn_lif_backward(int neuron, const sjhip_neuron_params &p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                           const float *scale, const float *shift, const float *v_init, const float *k_device,
                           const float *grad_spike_seq, const float *grad_v_last, float *grad_z, float *grad_v_init, float *partial,
                           float *grad_k, float *k_workspace, hipStream_t stream) {
  int rc = check_layout("bn_lif_backward", T, B, C, L);
  if (rc != SJHIP_OK) return rc;
  if (!lif_like(neuron)) return fail(SJHIP_ERR_UNSUPPORTED, "bn_lif_backward: neuron %d (IF, LIF and PLIF only)", neuron);
  const bool plif = neuron == SJHIP_NEURON_PLIF;
  if (plif != (k_device != nullptr) || (plif && (!grad_k || !k_workspace)))
    return fail(SJHIP_ERR_INVALID, "bn_lif_backward: k in device memory, grad_k and the workspace go with PLIF and only with it");
  if (T > kBnPiece * kBnMaxPieces)
    return fail(SJHIP_ERR_UNSUPPORTED, "bn_lif_backward: T=%lld (at most %d steps)", (long long)T, kBnPiece * kBnMaxPieces);
  if (p.sg_id < SJHIP_SG_SIGMOID || p.sg_id > SJHIP_SG_ERF) return fail(SJHIP_ERR_UNSUPPORTED, "bn_lif_backward: surrogate id %d", p.sg_id);
  const int64_t N = B * C * L;
  const bool broadcast = (p.flags & SJHIP_FLAG_V_INIT_BROADCAST) != 0;
  if (!aligned16(y) || (!broadcast && !aligned16(v_init)) || !aligned16(grad_spike_seq) || !aligned16(grad_z) ||
      (grad_v_last && !aligned16(grad_v_last)) || (grad_v_init && !aligned16(grad_v_init)))
    return fail(SJHIP_ERR_UNSUPPORTED, "bn_lif_backward: tensors must be 16-byte aligned");
  BnLifBwdArgs a;
  bool round_each = false;
  rc = build_fwd_args(a.f, round_each, neuron, SJHIP_F32, p, T, N, y, v_init, k_device, nullptr, nullptr, nullptr, nullptr);
  if (rc != SJHIP_OK) return rc;
  rc = build_bwd_args(a.b, neuron, SJHIP_F32, p, T, N, grad_spike_seq, nullptr, grad_v_last, nullptr, v_init, k_device, grad_z,
                      grad_v_init, grad_k, k_workspace);
  if (rc != SJHIP_OK) return rc;
  a.scale = scale; a.shift = shift; a.partial = partial; a.k_partial = k_workspace; a.C = (int)C; a.L = (int)L; a.rows = B * C;
  const int64_t blocks = (a.rows + 3) / 4;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bn_lif_backward: %lld rows", (long long)a.rows);
  ProfileScope prof(KC_BN_LIF_BACKWARD, stream);
  // (the walk in pieces parks one state per piece and work-item in LDS: at most 64 KiB, no opt-in needed)
  const unsigned parked = T > kBnPiece ? (unsigned)((T + kBnPiece - 1) / kBnPiece) * 256u * 16u : 0u;
  const int quads = (int)(L / 4);
  const int per = quads > 0 ? 256 / quads : 0;
  // TMAX by sequence length (0: the walk in pieces), with or without the dL/dk term
  auto launch = [&](auto rows_kernel, auto plif_flag) {
    constexpr bool ROWS = decltype(rows_kernel)::value, P = decltype(plif_flag)::value;
    const int64_t nb = ROWS ? (a.rows + per - 1) / per : blocks;
    const float inv = quads > 0 ? 1.0f / (float)quads : 0.0f;
    const dim3 grid((unsigned)nb), threads(256);
    if constexpr (ROWS) {
      if (T <= 4) hipLaunchKernelGGL((bn_lif_backward_rows_kernel<4, P>), grid, threads, 0, stream, a, quads, per, inv);
      else if (T <= 8) hipLaunchKernelGGL((bn_lif_backward_rows_kernel<8, P>), grid, threads, 0, stream, a, quads, per, inv);
      else if (T <= 16) hipLaunchKernelGGL((bn_lif_backward_rows_kernel<16, P>), grid, threads, 0, stream, a, quads, per, inv);
      else hipLaunchKernelGGL((bn_lif_backward_rows_kernel<0, P>), grid, threads, parked, stream, a, quads, per, inv);
    } else {
      if (T <= 4) hipLaunchKernelGGL((bn_lif_backward_kernel<4, P>), grid, threads, 0, stream, a);
      else if (T <= 8) hipLaunchKernelGGL((bn_lif_backward_kernel<8, P>), grid, threads, 0, stream, a);
      else if (T <= 16) hipLaunchKernelGGL((bn_lif_backward_kernel<16, P>), grid, threads, 0, stream, a);
      else hipLaunchKernelGGL((bn_lif_backward_kernel<0, P>), grid, threads, parked, stream, a);
    }
    return nb;
  };
  // more than the four rows a block of the wavefront-per-row kernel takes: more lanes working
  const bool by_rows = quads >= 16 && per > 4;
  if (by_rows && (a.rows + per - 1) / per > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bn_lif_backward: %lld rows", (long long)a.rows);
  int64_t nb;
  if (by_rows) nb = plif ? launch(std::true_type(), std::true_type()) : launch(std::true_type(), std::false_type());
  else nb = plif ? launch(std::false_type(), std::true_type()) : launch(std::false_type(), std::false_type());
  rc = check_launch("bn_lif_backward");
  if (rc != SJHIP_OK || !plif) return rc;
  return launch_plif_reduce(a.b, 4 * nb, grad_k, stream);
}

int launch_bn_backward_finalize(const float *partial, int64_t T, int64_t B, int64_t C, int64_t L, int training, const float *gamma,
                                const float *mean, const float *invstd, float *dgamma, float *dbeta, float *coef,
                                float *amax_reset, hipStream_t stream) {
  if (C < 1 || C > (1 << 24)) return fail(SJHIP_ERR_INVALID, "bn_backward_finalize: C=%lld", (long long)C);
  // (the amax buffer of the dy that sjhip_bn_grad_input_amax writes next: the tensor's words and one per sample)
  hipLaunchKernelGGL(bn_backward_finalize_kernel, dim3((unsigned)((C + 3) / 4)), dim3(256), 0, stream, partial, B, (int)C,
                     T * B * L, training, gamma, mean, invstd, dgamma, dbeta, coef, amax_reset, SJHIP_PW_AMAX_FLOATS + SJHIP_PW_AMAX_SAMPLE_WORDS * T * B);
  return check_launch("bn_backward_finalize");
}

int launch_bn_grad_input(const float *g, const float *y, const float *coef, int64_t S, int64_t C, int64_t L, float *dy, float *amax,
                         hipStream_t stream) {
  int rc = check_layout("bn_grad_input", 1, S, C, L);
  if (rc != SJHIP_OK) return rc;
  if (!aligned16(g) || !aligned16(y) || !aligned16(dy)) return fail(SJHIP_ERR_UNSUPPORTED, "bn_grad_input: tensors must be 16-byte aligned");
  const int64_t n = S * C * L, blocks = (n / 4 + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bn_grad_input: %lld elements", (long long)n);
  ProfileScope prof(KC_BN_GRAD_INPUT, stream);
  if (amax)
    hipLaunchKernelGGL(bn_grad_input_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, g, y, coef, S, (int)C, (int)L, n, dy,
                       reinterpret_cast<unsigned *>(amax));
  else
    hipLaunchKernelGGL(bn_grad_input_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, g, y, coef, S, (int)C, (int)L, n, dy,
                       (unsigned *)nullptr);
  return check_launch("bn_grad_input");
}

}  // namespace sjhip
