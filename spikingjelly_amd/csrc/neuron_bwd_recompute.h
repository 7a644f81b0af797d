// Backward that recomputes h instead of reading a saved h_seq.
//
// Phase 1 replays the forward recurrence from x_seq and v_init with the forward's own arithmetic
// (neuron_step of neuron_fwd.h, so h_t is bit-identical to what the forward computed) and parks h_t
// for every step in LDS as fp32.  Phase 2 is the ordinary BPTT walk of neuron_bwd.h reading h_t
// from LDS.  Each work-item touches only its own LDS words, so no barrier is needed.
//
// With 16-bit storage and every op rounded, h_t is exactly a storage-dtype value and is parked as 16-bit patterns
// (half the LDS, twice the resident wavefronts); with fp32 state it stays fp32.
//
// Why: the forward then never writes h_seq (4 B per neuron-step less to write in the slowest,
// write-dominated kernel) and the backward reads x_seq instead of h_seq (same bytes).  LDS holds
// T * blockDim * V * 4 bytes per block, which also bounds T (see recompute_block()).
#pragma once

#include "neuron_bwd.h"
#include "neuron_fwd.h"

// Rows of x in flight per work-item while h is replayed (4, 8 and 16 measured within 1 % of each other).
#ifndef SJHIP_REPLAY_PF
#define SJHIP_REPLAY_PF 8
#endif
#ifndef SJHIP_REPLAY_PF16
#define SJHIP_REPLAY_PF16 4
#endif

namespace sjhip {

// storage-dtype bit pattern of an h that is already a storage-dtype value
template <typename S> __device__ __forceinline__ uint32_t h_bits(float h) { return Cvt<S>::from_float(h); }
template <typename S> __device__ __forceinline__ uint32_t h_bits(_Float16 h) { return __builtin_bit_cast(uint16_t, h); }

template <typename S, bool ROUND_EACH, int CH, int RS, bool SHORT>
__device__ __forceinline__ void recompute_body(const FwdArgs &a, f32x4 *lds_h, int64_t col) {
  typedef Acc<S, true, SJHIP_REPLAY_X_NT != 0> A;
  typedef typename A::elem_t E;
  typedef typename std::conditional<ROUND_EACH, S, float>::type R;
  constexpr int V = A::V;
  constexpr int PF = SHORT ? kShortRows : ((sizeof(S) == 2 && V == 8) ? SJHIP_REPLAY_PF16 : SJHIP_REPLAY_PF);

  const int64_t N = a.N, T = a.T;
  const E *xp = (const E *)a.x + col;
  const float tau = a.k_device ? *a.k_device : a.tau;

  typename A::raw_t ahead[PF];
#pragma unroll
  for (int i = 0; i < PF; ++i) ahead[i] = (i < T) ? A::load(xp + (int64_t)i * N) : A::zero();
  typedef typename StepNum<S, ROUND_EACH>::type NUM;
  NUM v[V];
  load_state_from<S, true, SJHIP_BWD_NT != 0>(a.v_init, col, a.v_init_broadcast, v);

  for (int64_t t0 = 0; t0 < T; t0 += PF) {
    typename A::raw_t cur[PF];
#pragma unroll
    for (int i = 0; i < PF; ++i) cur[i] = ahead[i];
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t tn = t0 + PF + i;
      if (tn < T) ahead[i] = A::load(xp + tn * N);
    }
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      const int64_t t = t0 + i;
      if (t < T) {
        NUM x[V], h[V], s[V];
        A::unpack(cur[i], x);
#pragma unroll
        for (int j = 0; j < V; ++j) neuron_step<R, CH, RS>(x[j], v[j], h[j], s[j], tau, a);
        if constexpr (ROUND_EACH && sizeof(S) == 2) {
          u32x4 w;
          w.x = h_bits<S>(h[0]) | (h_bits<S>(h[1]) << 16); w.y = h_bits<S>(h[2]) | (h_bits<S>(h[3]) << 16);
          w.z = h_bits<S>(h[4]) | (h_bits<S>(h[5]) << 16); w.w = h_bits<S>(h[6]) | (h_bits<S>(h[7]) << 16);
          reinterpret_cast<u32x4 *>(lds_h)[(int)t * (int)blockDim.x + (int)threadIdx.x] = w;
        } else {
#pragma unroll
          for (int q = 0; q < V / 4; ++q) {
            f32x4 w; w.x = (float)h[4 * q]; w.y = (float)h[4 * q + 1]; w.z = (float)h[4 * q + 2]; w.w = (float)h[4 * q + 3];
            lds_h[((int)t * (V / 4) + q) * (int)blockDim.x + (int)threadIdx.x] = w;
          }
        }
      }
    }
  }
}

template <typename S, bool ROUND_EACH, int CH, bool SHORT>
__device__ __forceinline__ void recompute_reset_dispatch(const FwdArgs &a, f32x4 *lds_h, int64_t col) {
  if constexpr (CH == CH_PLAIN_INPUT_DIV || CH == CH_PLAIN_INPUT_MUL) {
    if (a.soft_reset == RESET_COUNT) {
      recompute_body<S, ROUND_EACH, CH, RESET_COUNT, SHORT>(a, lds_h, col);
      return;
    }
  }
  if (a.soft_reset) recompute_body<S, ROUND_EACH, CH, RESET_SOFT, SHORT>(a, lds_h, col);
  else recompute_body<S, ROUND_EACH, CH, RESET_HARD, SHORT>(a, lds_h, col);
}

// Phase 1 for one work-item: dispatch on the charge equation.
template <typename S, bool ROUND_EACH, bool SHORT>
__device__ __forceinline__ void recompute_charge_dispatch(const FwdArgs &f, f32x4 *lds_h, int64_t col) {
  switch (f.charge) {
    case CH_IF: recompute_reset_dispatch<S, ROUND_EACH, CH_IF, SHORT>(f, lds_h, col); break;
    case CH_DECAY_INPUT_DIV: recompute_reset_dispatch<S, ROUND_EACH, CH_DECAY_INPUT_DIV, SHORT>(f, lds_h, col); break;
    case CH_DECAY_INPUT_MUL: recompute_reset_dispatch<S, ROUND_EACH, CH_DECAY_INPUT_MUL, SHORT>(f, lds_h, col); break;
    case CH_PLAIN_INPUT_DIV: recompute_reset_dispatch<S, ROUND_EACH, CH_PLAIN_INPUT_DIV, SHORT>(f, lds_h, col); break;
    case CH_QIF_DIV: recompute_reset_dispatch<S, ROUND_EACH, CH_QIF_DIV, SHORT>(f, lds_h, col); break;
    case CH_QIF_MUL: recompute_reset_dispatch<S, ROUND_EACH, CH_QIF_MUL, SHORT>(f, lds_h, col); break;
    case CH_EIF_DIV: recompute_reset_dispatch<S, ROUND_EACH, CH_EIF_DIV, SHORT>(f, lds_h, col); break;
    case CH_EIF_MUL: recompute_reset_dispatch<S, ROUND_EACH, CH_EIF_MUL, SHORT>(f, lds_h, col); break;
    default: recompute_reset_dispatch<S, ROUND_EACH, CH_PLAIN_INPUT_MUL, SHORT>(f, lds_h, col); break;
  }
}

// Makes wavefront-uniform scalars opaque to the optimiser at this point, so that values derived from them (copies of
// scalars into vector registers, folded constants of every surrogate's branch) are formed inside the enclosing loop
// iteration and die there, instead of being hoisted in front of the loop and held in registers across all of its
// branches (measured on the kernel below: 256 registers plus 100 to 190 bytes of spills without, 222 and none with).
template <typename T> __device__ __forceinline__ void keep_scalar_local(T &x) { asm volatile("" : "+s"(x)); }
template <typename... Ts> __device__ __forceinline__ void keep_uniform_local(Ts &...x) { (keep_scalar_local(x), ...); }

__device__ __forceinline__ void keep_uniform_local(FwdArgs &a) {
  keep_uniform_local(a.x, a.v_init, a.T, a.N);
}

__device__ __forceinline__ void keep_uniform_local(BwdArgs &a) {
  keep_uniform_local(a.grad_spike, a.grad_v_seq, a.grad_v_last, a.v_init, a.grad_x, a.grad_v_init, a.T, a.N, a.sg, a.soft_reset,
                     a.decay_input, a.is_if, a.exponential, a.detach_reset, a.round_each, a.v_init_broadcast);
}

// A sequence too long for one LDS buffer, walked piece by piece from the last to the first inside one launch: each
// piece is replayed from its checkpoint (left by forward_pieces_kernel) into the same LDS buffer of `chunk` steps and
// walked back; the gradient of the piece's initial state stays in registers (fp32) for the piece before it.  The two
// phases are the ones of backward_recompute_kernel, called with the pointers and the length of the piece.
template <typename S, bool ROUND_EACH, int MODE>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) backward_recompute_pieces_kernel(const FwdArgs f0, const BwdArgs b0,
                                                                                    const PieceArgs p) {
  extern __shared__ f32x4 lds_h[];
  typedef typename Acc<S, true, true>::elem_t E;
  constexpr int V = Acc<S, true, true>::V;
  static_assert(!BwdModeOf<MODE>::SHORT, "pieces are long enough for the deep prefetch");
  const int64_t col = ((int64_t)column_block(b0.spread) * blockDim.x + threadIdx.x) * V;
  const bool active = col < b0.N;
  const float k = b0.k_device ? *b0.k_device : b0.k;
  constexpr int HLDS = (ROUND_EACH && sizeof(S) == 2) ? 2 : 1;
  const int64_t N = b0.N;
  float part = 0.0f;
  float state_gradient[V];
#pragma unroll
  for (int i = 0; i < V; ++i) state_gradient[i] = 0.0f;
  for (int64_t j = p.pieces - 1; j >= 0; --j) {
    const int64_t t0 = j * p.chunk;
    const int64_t len = (b0.T - t0 < p.chunk) ? b0.T - t0 : p.chunk;
    FwdArgs f = f0;
    BwdArgs b = b0;
    f.T = len; b.T = len;
    f.x = (const E *)f0.x + t0 * N;
    if (j > 0) {
      if (p.checkpoints_f32) {
        f.v_init = (const float *)p.checkpoints + (j - 1) * N;
        f.v_init_broadcast = kStateF32;
      } else {
        f.v_init = (const E *)p.checkpoints + (j - 1) * N;
        f.v_init_broadcast = 0;
      }
    }
    b.v_init = f.v_init;
    b.v_init_broadcast = f.v_init_broadcast;
    if (b0.grad_spike) b.grad_spike = (const E *)b0.grad_spike + t0 * N;
    if (b0.grad_v_seq) b.grad_v_seq = (const E *)b0.grad_v_seq + t0 * N;
    b.grad_x = (E *)b0.grad_x + t0 * N;
    StateGradient sgr;
    sgr.regs = state_gradient;
    sgr.from_regs = j + 1 < p.pieces;
    sgr.to_regs = j > 0;
    keep_uniform_local(f);
    keep_uniform_local(b);
    float kj = k;
    keep_scalar_local(kj);
    // request the last rows of the piece's upstream gradients now, so they arrive while h is being replayed
    BwdPrologue<S, true, false> pre;
    if (active) {
      pre.load(b, col);
      recompute_charge_dispatch<S, ROUND_EACH, false>(f, lds_h, col);
    }
    part += backward_sg_dispatch<S, true, MODE, HLDS>(b, active, col, kj, lds_h, &pre, sgr);
  }
  if (BwdModeOf<MODE>::BASE == BWD_PLIF) plif_block_reduce(b0, part, k);
}

template <typename S, bool ROUND_EACH, int MODE>
__global__ void __launch_bounds__(SJHIP_MAX_BLOCK) backward_recompute_kernel(const FwdArgs f, const BwdArgs b) {
  extern __shared__ f32x4 lds_h[];
  constexpr int V = Acc<S, true, true>::V;
  const int64_t col = ((int64_t)column_block(b.spread) * blockDim.x + threadIdx.x) * V;
  const bool active = col < b.N;
  // request the last rows of the upstream gradients now, so they arrive while h is being replayed
  constexpr bool SHORT = BwdModeOf<MODE>::SHORT;
  BwdPrologue<S, true, SHORT> pre;
  if (active) {
    pre.load(b, col);
    switch (f.charge) {
      case CH_IF: recompute_reset_dispatch<S, ROUND_EACH, CH_IF, SHORT>(f, lds_h, col); break;
      case CH_DECAY_INPUT_DIV: recompute_reset_dispatch<S, ROUND_EACH, CH_DECAY_INPUT_DIV, SHORT>(f, lds_h, col); break;
      case CH_DECAY_INPUT_MUL: recompute_reset_dispatch<S, ROUND_EACH, CH_DECAY_INPUT_MUL, SHORT>(f, lds_h, col); break;
      case CH_PLAIN_INPUT_DIV: recompute_reset_dispatch<S, ROUND_EACH, CH_PLAIN_INPUT_DIV, SHORT>(f, lds_h, col); break;
      case CH_QIF_DIV: recompute_reset_dispatch<S, ROUND_EACH, CH_QIF_DIV, SHORT>(f, lds_h, col); break;
      case CH_QIF_MUL: recompute_reset_dispatch<S, ROUND_EACH, CH_QIF_MUL, SHORT>(f, lds_h, col); break;
      case CH_EIF_DIV: recompute_reset_dispatch<S, ROUND_EACH, CH_EIF_DIV, SHORT>(f, lds_h, col); break;
      case CH_EIF_MUL: recompute_reset_dispatch<S, ROUND_EACH, CH_EIF_MUL, SHORT>(f, lds_h, col); break;
      default: recompute_reset_dispatch<S, ROUND_EACH, CH_PLAIN_INPUT_MUL, SHORT>(f, lds_h, col); break;
    }
  }
  const float k = b.k_device ? *b.k_device : b.k;
  constexpr int HLDS = (ROUND_EACH && sizeof(S) == 2) ? 2 : 1;
  const float part = backward_sg_dispatch<S, true, MODE, HLDS>(b, active, col, k, lds_h, &pre);
  if (BwdModeOf<MODE>::BASE == BWD_PLIF) plif_block_reduce(b, part, k);
}

// Launches the recompute kernel of storage dtype S; defined in neuron_bwd_recompute_launch.h and
// instantiated once per dtype (neuron_bwd_recompute_{f32,f16,bf16}.hip).
template <typename S>
int launch_recompute_dtype(const FwdArgs &f, const BwdArgs &b, bool round_each, int mode, int block, unsigned lds,
                           int64_t blocks, hipStream_t stream, const PieceArgs *pieces = nullptr);

}  // namespace sjhip
