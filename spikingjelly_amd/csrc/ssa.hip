// Spiking self-attention contraction  out = scale * (V K^T) Q  and its backward, on MFMA.
//
// Layout and order follow the reference (layer/attention.py:346-353, `_ssa_kernel_torch`): qkv is
// [TB, 3, H, Cph, L] (q, k, v of one sample stacked on dim 1; each head a row-major [Cph, L] tile of
// binary spikes), S = V K^T is [Cph, Cph] (contraction over the L tokens), out = scale * S Q is
// [TB, H, Cph, L].  The work is HBM-bound (about 8 flop per byte), so the kernels are built as streaming
// kernels whose arithmetic happens to run on the matrix cores:
//
//   * one block of four wavefronts owns one (sample, head) problem; each [Cph, L] tile is one contiguous
//     run in memory and is fetched with 16-byte accesses, all loads of a pass issued before any is used;
//   * spikes are parked in LDS as one byte each (0 / 1), so the three tiles of a head take 21 KB for
//     Cph = 32, L = 196 and several blocks are resident per compute unit to overlap load, MFMA and store;
//   * S = V K^T runs on v_mfma_i32_32x32x32_i8: exact integers <= L;
//   * S never goes through LDS: it is produced transposed (K V^T), and in the accumulator layout lane
//     (c1, half) already holds S[c1, c2] for the sixteen c2 = 8 (r / 4) + 4 half + r % 4, which is a valid
//     A operand of the second product as long as the B operand (Q) is gathered with the same k order;
//   * out = S Q on v_mfma_f32_32x32x16_bf16 (S <= 256 and spikes are exact in bf16, fp32 accumulation of
//     integers < 2^24), `scale` (a power of two in the reference, 0.125) is applied once.
// Hence the forward equals an int64 matmul of the spikes times scale, bit for bit, in fp32 output,
// and after one rounding in 16-bit output (what torch's bf16 matmuls also produce).
//
// The backward has one real-valued operand per product (grad_out or dS) and one exact one (spikes, or S <= 256):
//   dS = scale * dO Q^T  (v_mfma_f32_16x16x4_f32, one 16x16 block per wavefront, through LDS; the contraction over the
//        tokens is long and the output small, so splitting dO would cost more VALU work than the fp32 MFMA takes),
//   dQ = scale * S^T dO,  dK = dS^T V,  dV = dS K  on v_mfma_f32_32x32x16_bf16: the real operand is split into three
//        bf16 terms that sum to it exactly (Bf16Terms), so the products are the ones an fp32 MFMA would form; column
//        tiles are dealt to wavefronts, S is recomputed on the int8 MFMA and kept in registers.
//
// MFMA layouts used (lane = 0..63):  32x32: A element of lane is row lane % 32, k group lane / 32; B likewise
// with column lane % 32; accumulator register r sits at row 8 (r / 4) + 4 (lane / 32) + r % 4, column
// lane % 32.  16x16x4: A row lane % 16, k = lane / 16; accumulator register r at row 4 (lane / 16) + r,
// column lane % 16.  Which k a lane's operand element stands for is free as long as A and B agree.
#include "neuron_bwd.h"
#include "neuron_fwd.h"
#include "sjhip_common.h"

#include <algorithm>
#include <mutex>

// Resident blocks per compute unit the backward kernel's register allocation is sized for (heads of up to 32
// channels).  Sized for 2 the kernel takes 124 registers and keeps the split dS operands across the column tiles
// without spilling, so three blocks are resident anyway (what LDS allows); sized for 3 the allocator spills 40
// registers around the same code (80 us against 83 us at 256 samples x 12 heads x 32 x 196).
// Measured on the same shape with bit-packed spikes (us per launch; fetching with one trip to memory per loop iteration
// of the stagings and no integer division: 91): requesting all of a head's grad_out and spike bytes before using any
// (40 registers held): 103; a grid of resident blocks, each fetching its next head into registers while it computes the
// current one: 108 with two resident blocks (the loop around the products takes the allocator to 256 registers) and
// 149 with three (60 registers spilled).  The kernel therefore keeps one block per head and the plain stagings.
#ifndef SJHIP_SSA_BWD_RESIDENT
#define SJHIP_SSA_BWD_RESIDENT 2
#endif
// The same for the backward fused with the neuron, which also holds the gradient of the potential (32 registers):
// sized for 3 it spills 77 registers and takes 155 us on 4 x 64 samples x 12 heads x 32 x 196, sized for 2 it takes all
// 256 registers, spills nothing and takes 131 us.
#ifndef SJHIP_SSA_LIF_BWD_RESIDENT
#define SJHIP_SSA_LIF_BWD_RESIDENT 2
#endif

namespace sjhip {

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr unsigned kSsaMaxLds = 159u * 1024u;
// Work-items per block: four wavefronts for heads of up to 32 channels, eight for larger ones (measured at 64 channels,
// 196 tokens: backward 355 -> 290 us; at 32 channels eight wavefronts change nothing backward and cost 20 % forward).
// Device code asks blockDim.x.
constexpr int ssa_threads(int mc) { return mc == 1 ? 256 : 512; }

struct SsaArgs {
  const uint8_t *qkv_bits;  // when set, the spikes come bit-packed (LSB first over the flattened tensor) and qkv is unused
  const void *qkv;
  const void *grad_out;
  void *out;
  void *grad_qkv;
  int64_t problems;  // TB * heads
  int heads;
  int cph;    // channels per head (<= 64); tiles are zero-padded to 32 or 64 rows in LDS
  int L;      // tokens
  int Lb;     // LDS row stride (bytes) of the spike tiles = L rounded up to 32
  int Lq;     // LDS row stride (floats) of the grad_out tile
  int vec;    // tiles may be fetched four elements at a time (L % 4 == 0 and aligned bases)
  float scale;
};

// Four consecutive elements of a tile, as fetched; and single elements for ragged shapes.
template <typename S> struct Io;
template <> struct Io<float> {
  typedef float elem_t;
  typedef f32x4 quad_t;
  static __device__ __forceinline__ float get(const elem_t *p, int64_t i) { return p[i]; }
  static __device__ __forceinline__ void put(elem_t *p, int64_t i, float v) { p[i] = v; }
  static __device__ __forceinline__ void unpack(quad_t q, float (&f)[4]) { f[0] = q.x; f[1] = q.y; f[2] = q.z; f[3] = q.w; }
};
template <typename H> struct Io16 {
  typedef uint16_t elem_t;
  typedef u32x2 quad_t;
  static __device__ __forceinline__ float get(const elem_t *p, int64_t i) { return Cvt<H>::to_float(p[i]); }
  static __device__ __forceinline__ void put(elem_t *p, int64_t i, float v) { p[i] = Cvt<H>::from_float(v); }
  static __device__ __forceinline__ void unpack(quad_t q, float (&f)[4]) {
    f[0] = Cvt<H>::to_float((uint16_t)(q.x & 0xffffu)); f[1] = Cvt<H>::to_float((uint16_t)(q.x >> 16));
    f[2] = Cvt<H>::to_float((uint16_t)(q.y & 0xffffu)); f[3] = Cvt<H>::to_float((uint16_t)(q.y >> 16));
  }
};
template <> struct Io<f16_t> : Io16<f16_t> {};
template <> struct Io<bf16_t> : Io16<bf16_t> {};

__device__ __forceinline__ uint32_t spike_bytes(const float (&f)[4]) {
  return (f[0] != 0.0f ? 1u : 0u) | (f[1] != 0.0f ? 0x100u : 0u) | (f[2] != 0.0f ? 0x10000u : 0u) |
         (f[3] != 0.0f ? 0x1000000u : 0u);
}

// e / L for 0 <= e < 2^16 and 1 <= L <= 256 without the integer-division sequence: (e + 0.5) / L lies at least
// 0.5 / L away from every integer, far more than the rounding error of the fp32 product.
__device__ __forceinline__ int div_tokens(int e, float inv_L) { return (int)(((float)e + 0.5f) * inv_L); }

// Zero-fills columns [L, stride) of rows [0, cph) and all of rows [cph, rows_pad) of NS byte tiles or one fp32 tile;
// eight work-items per row, so no work-item divides.
template <int NS>
__device__ __forceinline__ void zero_fill_bytes(uint8_t *const (&dst)[NS], int cph, int rows_pad, int L, int Lb) {
  const int tid = threadIdx.x;
  for (int r = tid >> 3; r < cph; r += ((int)blockDim.x / 8))
    for (int c = L + (tid & 7); c < Lb; c += 8) {
#pragma unroll
      for (int s = 0; s < NS; ++s) dst[s][r * Lb + c] = 0;
    }
  for (int i = tid; i < (rows_pad - cph) * (Lb / 4); i += (int)blockDim.x) {
#pragma unroll
    for (int s = 0; s < NS; ++s) reinterpret_cast<uint32_t *>(dst[s] + cph * Lb)[i] = 0u;
  }
}
__device__ __forceinline__ void zero_fill_f32(float *dst, int cph, int rows_pad, int L, int Lq) {
  const int tid = threadIdx.x;
  for (int r = tid >> 3; r < cph; r += ((int)blockDim.x / 8))
    for (int c = L + (tid & 7); c < Lq; c += 8) dst[r * Lq + c] = 0.0f;
  for (int i = tid; i < (rows_pad - cph) * Lq; i += (int)blockDim.x) dst[cph * Lq + i] = 0.0f;
}

// Global tiles -> LDS.  NS spike tiles ([cph, L] each) become
// byte tiles [rows_pad][Lb]; when DO is set the grad_out tile becomes an fp32 tile [rows_pad][Lq].  Rows
// cph..rows_pad-1 and the columns from L to the row stride are zero-filled, by writes that never overlap the
// data writes, so one barrier after this function is enough.
template <typename S, int NS, bool DO, int UN>
__device__ __forceinline__ void stage_tiles(const typename Io<S>::elem_t *const (&src)[NS], uint8_t *const (&dst)[NS],
                                            const typename Io<S>::elem_t *do_src, float *do_dst, int cph, int rows_pad,
                                            int L, int Lb, int Lq, bool vec) {
  typedef typename Io<S>::quad_t Q;
  const int tid = threadIdx.x;
  if (vec) {
    const int G = cph * L / 4;
    const float inv_L = 1.0f / (float)L;
    for (int g0 = tid; g0 < G; g0 += (int)blockDim.x * UN) {
      Q buf[UN][NS + (DO ? 1 : 0)];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int g = g0 + u * (int)blockDim.x;
        if (g < G) {
#pragma unroll
          for (int s = 0; s < NS; ++s) buf[u][s] = reinterpret_cast<const Q *>(src[s])[g];
          if (DO) buf[u][NS] = reinterpret_cast<const Q *>(do_src)[g];
        }
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int g = g0 + u * (int)blockDim.x;
        if (g < G) {
          const int r = div_tokens(4 * g, inv_L), c = 4 * g - r * L;
          float f[4];
#pragma unroll
          for (int s = 0; s < NS; ++s) {
            Io<S>::unpack(buf[u][s], f);
            *reinterpret_cast<uint32_t *>(dst[s] + r * Lb + c) = spike_bytes(f);
          }
          if (DO) {
            Io<S>::unpack(buf[u][NS], f);
            f32x4 w; w.x = f[0]; w.y = f[1]; w.z = f[2]; w.w = f[3];
            *reinterpret_cast<f32x4 *>(do_dst + r * Lq + c) = w;
          }
        }
      }
    }
  } else {
    const int n = cph * L;
    for (int i = tid; i < n; i += (int)blockDim.x) {
      const int r = i / L, c = i - r * L;
#pragma unroll
      for (int s = 0; s < NS; ++s) dst[s][r * Lb + c] = Io<S>::get(src[s], i) != 0.0f ? 1 : 0;
      if (DO) do_dst[r * Lq + c] = Io<S>::get(do_src, i);
    }
  }
  zero_fill_bytes<NS>(dst, cph, rows_pad, L, Lb);
  if (DO) zero_fill_f32(do_dst, cph, rows_pad, L, Lq);
}

// Byte b of the bit-packed tiles (its eight elements 8 b ... 8 b + 7) -> LDS byte tiles.
template <int NS>
__device__ __forceinline__ void expand_byte(const uint32_t (&w)[NS], int b, uint8_t *const (&dst)[NS], int L, int Lb,
                                            float inv_L) {
  if ((L & 3) == 0) {
    // four elements never straddle a row and land on a 4-byte boundary: one 32-bit store per nibble.  The product
    // copies bit i of the nibble to bit 8 i (and to other positions the mask drops; no two copies collide).
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int e = 8 * b + 4 * half;
      const int r = div_tokens(e, inv_L), c = e - r * L;
#pragma unroll
      for (int s = 0; s < NS; ++s)
        *reinterpret_cast<uint32_t *>(dst[s] + r * Lb + c) = (((w[s] >> (4 * half)) & 15u) * 0x00204081u) & 0x01010101u;
    }
  } else {
    int r = div_tokens(8 * b, inv_L), c = 8 * b - r * L;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int s = 0; s < NS; ++s) dst[s][r * Lb + c] = (uint8_t)((w[s] >> i) & 1u);
      if (++c == L) { c = 0; ++r; }
    }
  }
}

// Bit-packed spike tiles -> LDS byte tiles.  The flattened qkv tensor is packed LSB first (byte j bit i = element
// 8 j + i, what bit_pack and the packed neuron forward write); a [cph, L] tile whose element count is a multiple of 8
// starts on a byte and is cph L / 8 bytes long, 32 times less to fetch than fp32 spikes.  A byte's eight elements may
// straddle a row boundary of the tile (L need not be a multiple of 8).  All of a work-item's bytes (four cover 32
// channels of up to 256 tokens) are requested before the first is used: one trip to memory, not one per byte.
template <int NS>
__device__ __forceinline__ void stage_bits(const uint8_t *const (&src)[NS], uint8_t *const (&dst)[NS], int cph,
                                           int rows_pad, int L, int Lb) {
  constexpr int UB = 4;
  const int tid = threadIdx.x;
  const int nbytes = cph * L / 8;
  const float inv_L = 1.0f / (float)L;
  for (int b0 = tid; b0 < nbytes; b0 += (int)blockDim.x * UB) {
    uint32_t w[UB][NS];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const int b = b0 + u * (int)blockDim.x;
      if (b < nbytes) {
#pragma unroll
        for (int s = 0; s < NS; ++s) w[u][s] = src[s][b];
      }
    }
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const int b = b0 + u * (int)blockDim.x;
      if (b < nbytes) expand_byte<NS>(w[u], b, dst, L, Lb, inv_L);
    }
  }
  zero_fill_bytes<NS>(dst, cph, rows_pad, L, Lb);
}

// stage_bits in two halves for tiles of at most 4 * blockDim.x bytes (32 channels of 256 tokens with 256 work-items,
// 64 with 512): the requests, whose results a caller may leave in flight over other work, and the expansion into LDS.
template <int NS>
__device__ __forceinline__ void request_bits(const uint8_t *const (&src)[NS], int nbytes, uint32_t (&w)[4][NS]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int b = (int)threadIdx.x + u * (int)blockDim.x;
#pragma unroll
    for (int s = 0; s < NS; ++s) w[u][s] = src[s][b < nbytes ? b : nbytes - 1];
  }
}
template <int NS>
__device__ __forceinline__ void expand_bits(const uint32_t (&w)[4][NS], uint8_t *const (&dst)[NS], int cph, int rows_pad,
                                            int L, int Lb) {
  const int nbytes = cph * L / 8;
  const float inv_L = 1.0f / (float)L;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int b = (int)threadIdx.x + u * (int)blockDim.x;
    if (b < nbytes) expand_byte<NS>(w[u], b, dst, L, Lb, inv_L);
  }
  zero_fill_bytes<NS>(dst, cph, rows_pad, L, Lb);
}

// Four consecutive grad_out elements -> the fp32 LDS tile [rows_pad][Lq].
template <typename S>
__device__ __forceinline__ void put_grad_out_quad(typename Io<S>::quad_t q, int g, float *do_dst, int L, int Lq, float inv_L) {
  const int r = div_tokens(4 * g, inv_L), c = 4 * g - r * L;
  float f[4];
  Io<S>::unpack(q, f);
  f32x4 w; w.x = f[0]; w.y = f[1]; w.z = f[2]; w.w = f[3];
  *reinterpret_cast<f32x4 *>(do_dst + r * Lq + c) = w;
}

// The grad_out tile alone -> fp32 LDS tile [rows_pad][Lq], zero-padded (the packed backward stages its spikes apart).
template <typename S>
__device__ __forceinline__ void stage_grad_out(const typename Io<S>::elem_t *do_src, float *do_dst, int cph, int rows_pad,
                                               int L, int Lq, bool vec) {
  typedef typename Io<S>::quad_t Q;
  const int tid = threadIdx.x;
  if (vec) {
    const int G = cph * L / 4;
    const float inv_L = 1.0f / (float)L;
    constexpr int UN = 4;
    for (int g0 = tid; g0 < G; g0 += (int)blockDim.x * UN) {
      Q buf[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int g = g0 + u * (int)blockDim.x;
        if (g < G) buf[u] = reinterpret_cast<const Q *>(do_src)[g];
      }
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int g = g0 + u * (int)blockDim.x;
        if (g < G) put_grad_out_quad<S>(buf[u], g, do_dst, L, Lq, inv_L);
      }
    }
  } else {
    const int n = cph * L;
    for (int i = tid; i < n; i += (int)blockDim.x) {
      const int r = i / L, c = i - r * L;
      do_dst[r * Lq + c] = Io<S>::get(do_src, i);
    }
  }
  zero_fill_f32(do_dst, cph, rows_pad, L, Lq);
}

// 32x32 block of  A_rows B_rows^T  over the token axis: rows ra.. of tile `a` against rows rb.. of tile `b`
__device__ __forceinline__ i32x16 spike_gram(const uint8_t *a, int ra, const uint8_t *b, int rb, int Lb, int lane) {
  const uint8_t *ap = a + (ra + (lane & 31)) * Lb + 16 * (lane >> 5);
  const uint8_t *bp = b + (rb + (lane & 31)) * Lb + 16 * (lane >> 5);
  i32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < Lb; k0 += 32)
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(*reinterpret_cast<const i32x4 *>(ap + k0),
                                                *reinterpret_cast<const i32x4 *>(bp + k0), acc, 0, 0, 0);
  return acc;
}

// Eight fp32 values as three bf16 operands whose sum is the values exactly: every term keeps the next eight significant
// bits by truncation (24 in all, an fp32 significand), and the differences taken in between are exact.  A product of a
// term with a spike or with a count <= 256 is exact in fp32, so a bf16 MFMA over the three terms accumulates the same
// products as an fp32 MFMA would, at sixteen times its rate.
struct Bf16Terms {
  uint32_t w[3][4];
  __device__ __forceinline__ void set(int j, float x0, float x1) {
    constexpr uint32_t kTop = 0xffff0000u;
    const uint32_t a0 = __builtin_bit_cast(uint32_t, x0), a1 = __builtin_bit_cast(uint32_t, x1);
    const float r0 = x0 - __builtin_bit_cast(float, a0 & kTop), r1 = x1 - __builtin_bit_cast(float, a1 & kTop);
    const uint32_t b0 = __builtin_bit_cast(uint32_t, r0), b1 = __builtin_bit_cast(uint32_t, r1);
    const float q0 = r0 - __builtin_bit_cast(float, b0 & kTop), q1 = r1 - __builtin_bit_cast(float, b1 & kTop);
    w[0][j] = (a0 >> 16) | (a1 & kTop);
    w[1][j] = (b0 >> 16) | (b1 & kTop);
    w[2][j] = (__builtin_bit_cast(uint32_t, q0) >> 16) | (__builtin_bit_cast(uint32_t, q1) & kTop);
  }
  __device__ __forceinline__ bf16x8 term(int t) const {
    uint32_t v[4] = {w[t][0], w[t][1], w[t][2], w[t][3]};
    return __builtin_bit_cast(bf16x8, v);
  }
};

// accumulator register r of this lane sits at (row, col) of its 32x32 block
__device__ __forceinline__ int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

template <typename S, int MC>
__global__ void __launch_bounds__(ssa_threads(MC)) ssa_forward_kernel(const SsaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ssa_lds[];
  typedef typename Io<S>::elem_t E;
  constexpr int CPH = 32 * MC;
  const int L = a.L, Lb = a.Lb, cph = a.cph;
  uint8_t *q_lds = ssa_lds;
  uint8_t *k_lds = q_lds + CPH * Lb;
  uint8_t *v_lds = k_lds + CPH * Lb;

  const int64_t p = blockIdx.x;
  const int64_t sample = p / a.heads, head = p - sample * a.heads;
  const int64_t tile = (int64_t)cph * L;
  const E *qkv = static_cast<const E *>(a.qkv);
  {
    uint8_t *const dst[3] = {q_lds, k_lds, v_lds};
    if (a.qkv_bits) {
      const int64_t tb = tile / 8;
      const uint8_t *const src[3] = {a.qkv_bits + ((sample * 3 + 0) * a.heads + head) * tb,
                                     a.qkv_bits + ((sample * 3 + 1) * a.heads + head) * tb,
                                     a.qkv_bits + ((sample * 3 + 2) * a.heads + head) * tb};
      stage_bits<3>(src, dst, cph, CPH, L, Lb);
    } else {
      const E *const src[3] = {qkv + ((sample * 3 + 0) * a.heads + head) * tile,
                               qkv + ((sample * 3 + 1) * a.heads + head) * tile,
                               qkv + ((sample * 3 + 2) * a.heads + head) * tile};
      stage_tiles<S, 3, false, 4>(src, dst, nullptr, nullptr, cph, CPH, L, Lb, 0, a.vec != 0);
    }
  }
  __syncthreads();

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, half = lane >> 5;
  const int ntiles = (L + 31) / 32;
  const int units = ntiles * MC;  // unit u: output rows 32 (u % MC).., columns 32 (u / MC)..
  if (wave >= units) return;
  const int ni = wave % MC;  // the same for every unit of this wavefront because MC divides the wavefront count

  // S^T blocks (K V^T): lane (c1, half) register r holds S[32 ni + c1, 32 mi + 8 (r/4) + 4 half + r%4]
  bf16x8 s_op[MC][2];
#pragma unroll
  for (int mi = 0; mi < MC; ++mi) {
    const i32x16 acc = spike_gram(k_lds, mi * 32, v_lds, ni * 32, Lb, lane);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint16_t w[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) w[e] = (uint16_t)(__builtin_bit_cast(uint32_t, (float)acc[8 * h + e]) >> 16);  // exact: <= 256
      s_op[mi][h] = __builtin_bit_cast(bf16x8, w);
    }
  }

  E *og = static_cast<E *>(a.out) + p * tile;
  for (int u = wave; u < units; u += ((int)blockDim.x >> 6)) {
    const int nt = u / MC;
    const int col = nt * 32 + (lane & 31);
    const int colc = col < L ? col : L - 1;
    f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int mi = 0; mi < MC; ++mi) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint16_t w[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int c2 = mi * 32 + 16 * h + 8 * (e >> 2) + 4 * half + (e & 3);
          w[e] = (uint16_t)(q_lds[c2 * Lb + colc] * 0x3f80u);  // 1 -> bf16 1.0
        }
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s_op[mi][h], __builtin_bit_cast(bf16x8, w), acc, 0, 0, 0);
      }
    }
    if (col < L) {
      // 32-bit offsets from the uniform tile base; accumulator row r is a constant number of tile rows from the first
      const uint32_t first = (uint32_t)(ni * 32 + 4 * half) * (uint32_t)L + (uint32_t)col;
      if (cph == CPH) {
#pragma unroll
        for (int r = 0; r < 16; ++r) Io<S>::put(og, first + (uint32_t)(8 * (r >> 2) + (r & 3)) * (uint32_t)L, acc[r] * a.scale);
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (ni * 32 + acc_row(r, lane) < cph)
            Io<S>::put(og, first + (uint32_t)(8 * (r >> 2) + (r & 3)) * (uint32_t)L, acc[r] * a.scale);
      }
    }
  }
}

// The products of the backward for the head whose tiles are in LDS (grad_out as fp32 in do_lds, spikes as bytes):
// dS through ds_lds, then dQ, dK, dV stored at gq + qoff / koff / voff.  Every wavefront of the block calls it.
template <typename S, int MC>
__device__ __forceinline__ void ssa_backward_products(const SsaArgs &a, float *do_lds, float *ds_lds, const uint8_t *q_lds,
                                                      const uint8_t *k_lds, const uint8_t *v_lds, int64_t qoff, int64_t koff,
                                                      int64_t voff) {
  typedef typename Io<S>::elem_t E;
  constexpr int CPH = 32 * MC;
  constexpr int LS = CPH + 1;
  const int L = a.L, Lb = a.Lb, Lq = a.Lq, cph = a.cph;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, half = lane >> 5;
  const float scale = a.scale;

  // dS = scale * dO Q^T, one 16x16 block per wavefront and pass, into LDS
  {
    constexpr int NB = CPH / 16;
    const int Lk = (L + 15) & ~15;
    const int i16 = lane & 15, kq = lane >> 4;
    for (int sb = wave; sb < NB * NB; sb += ((int)blockDim.x >> 6)) {
      const int bi = sb / NB, bj = sb - bi * NB;
      const float *ap = do_lds + (16 * bi + i16) * Lq + 4 * kq;
      const uint8_t *bp = q_lds + (16 * bj + i16) * Lb + 4 * kq;
      f32x4 acc = {0, 0, 0, 0};
      for (int k0 = 0; k0 < Lk; k0 += 16) {
        const f32x4 av = *reinterpret_cast<const f32x4 *>(ap + k0);
        const uint32_t bw = *reinterpret_cast<const uint32_t *>(bp + k0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.x, (float)(bw & 0xffu), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.y, (float)((bw >> 8) & 0xffu), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.z, (float)((bw >> 16) & 0xffu), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(av.w, (float)(bw >> 24), acc, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) ds_lds[(16 * bi + 4 * kq + r) * LS + 16 * bj + i16] = acc[r] * scale;
    }
  }

  __syncthreads();

  E *gq = static_cast<E *>(a.grad_qkv);
  const int ntiles = (L + 31) / 32;
  const int m32 = lane & 31;
#pragma unroll 1
  for (int b = 0; b < MC; ++b) {
    // s_op: S^T blocks (V K^T, exact, <= 256 so exact in bf16) in the order the accumulator holds them: element e of
    // (ai, h) stands for c1 = 32 ai + 16 h + 8 (e / 4) + 4 half + e % 4.  In the dS operands of dK and dV element e of
    // (ai, h) stands for c = 32 ai + 16 h + 8 half + e.
    bf16x8 s_op[MC][2];
#pragma unroll
    for (int ai = 0; ai < MC; ++ai) {
      const i32x16 acc = spike_gram(v_lds, ai * 32, k_lds, b * 32, Lb, lane);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint16_t w[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = (uint16_t)(__builtin_bit_cast(uint32_t, (float)acc[8 * h + e]) >> 16);
        s_op[ai][h] = __builtin_bit_cast(bf16x8, w);
      }
    }
    // One product at a time: sixteen accumulator registers live instead of forty-eight.
    for (int nt = wave; nt < ntiles; nt += ((int)blockDim.x >> 6)) {
      const int col = nt * 32 + m32;
      const int colc = col < L ? col : L - 1;
      const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      // (the dS operands of dK and dV do not depend on the tile: the compiler forms them once, ahead of this loop)
      // 32-bit offsets from one uniform base per tensor: a row of the accumulator is a constant number of tile rows
      // away from the lane's first one
      const uint32_t first = (uint32_t)(b * 32 + 4 * half) * (uint32_t)L + (uint32_t)col;
      auto store = [&](E *tile_base, const f32x16 &acc, float factor) {
        if (col >= L) return;
        if (cph == CPH) {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            Io<S>::put(tile_base, first + (uint32_t)(8 * (r >> 2) + (r & 3)) * (uint32_t)L, acc[r] * factor);
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (b * 32 + acc_row(r, lane) < cph)
              Io<S>::put(tile_base, first + (uint32_t)(8 * (r >> 2) + (r & 3)) * (uint32_t)L, acc[r] * factor);
        }
      };
      {  // dQ[c2, l] = scale * sum_c1 S[c1, c2] dO[c1, l], c1 in the order of s_op
        f32x16 acc = zero;
#pragma unroll
        for (int ai = 0; ai < MC; ++ai) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            Bf16Terms t;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int c1 = ai * 32 + 16 * h + 8 * (j >> 1) + 4 * half + 2 * (j & 1);
              t.set(j, do_lds[c1 * Lq + colc], do_lds[(c1 + 1) * Lq + colc]);
            }
#pragma unroll
            for (int i = 2; i >= 0; --i)  // smallest terms first
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s_op[ai][h], t.term(i), acc, 0, 0, 0);
          }
        }
        store(gq + qoff, acc, scale);
      }
      {  // dK[c2, l] = sum_c dS[c, c2] V[c, l]
        f32x16 acc = zero;
#pragma unroll
        for (int ai = 0; ai < MC; ++ai) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            Bf16Terms t;
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int c = ai * 32 + 16 * h + 8 * half + 2 * j;
              t.set(j, ds_lds[c * LS + b * 32 + m32], ds_lds[(c + 1) * LS + b * 32 + m32]);
              w[j] = ((uint32_t)v_lds[c * Lb + colc] | ((uint32_t)v_lds[(c + 1) * Lb + colc] << 16)) * 0x3f80u;  // 1 -> bf16 1.0
            }
            const bf16x8 spikes = __builtin_bit_cast(bf16x8, w);
#pragma unroll
            for (int i = 2; i >= 0; --i) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t.term(i), spikes, acc, 0, 0, 0);
          }
        }
        store(gq + koff, acc, 1.0f);
      }
      {  // dV[c1, l] = sum_c dS[c1, c] K[c, l]
        f32x16 acc = zero;
#pragma unroll
        for (int ai = 0; ai < MC; ++ai) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            Bf16Terms t;
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int c = ai * 32 + 16 * h + 8 * half + 2 * j;
              t.set(j, ds_lds[(b * 32 + m32) * LS + c], ds_lds[(b * 32 + m32) * LS + c + 1]);
              w[j] = ((uint32_t)k_lds[c * Lb + colc] | ((uint32_t)k_lds[(c + 1) * Lb + colc] << 16)) * 0x3f80u;
            }
            const bf16x8 spikes = __builtin_bit_cast(bf16x8, w);
#pragma unroll
            for (int i = 2; i >= 0; --i) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(t.term(i), spikes, acc, 0, 0, 0);
          }
        }
        store(gq + voff, acc, 1.0f);
      }
    }
  }
}

template <typename S, int MC>
__global__ void __launch_bounds__(ssa_threads(MC), MC == 1 ? SJHIP_SSA_BWD_RESIDENT : 1) ssa_backward_kernel(const SsaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ssa_lds[];
  typedef typename Io<S>::elem_t E;
  constexpr int CPH = 32 * MC;
  constexpr int LS = CPH + 1;  // row stride of the fp32 dS tile
  const int L = a.L, Lb = a.Lb, Lq = a.Lq, cph = a.cph;
  float *do_lds = reinterpret_cast<float *>(ssa_lds);
  float *ds_lds = do_lds + CPH * Lq;
  uint8_t *q_lds = reinterpret_cast<uint8_t *>(ds_lds + CPH * LS);  // CPH * LS * 4 is a multiple of 16
  uint8_t *k_lds = q_lds + CPH * Lb;
  uint8_t *v_lds = k_lds + CPH * Lb;

  const int64_t p = blockIdx.x;
  const int64_t sample = p / a.heads, head = p - sample * a.heads;
  const int64_t tile = (int64_t)cph * L;
  const E *qkv = static_cast<const E *>(a.qkv);
  const int64_t qoff = ((sample * 3 + 0) * a.heads + head) * tile;
  const int64_t koff = ((sample * 3 + 1) * a.heads + head) * tile;
  const int64_t voff = ((sample * 3 + 2) * a.heads + head) * tile;
  {
    uint8_t *const dst[3] = {q_lds, k_lds, v_lds};
    if (a.qkv_bits) {
      const uint8_t *const src[3] = {a.qkv_bits + qoff / 8, a.qkv_bits + koff / 8, a.qkv_bits + voff / 8};
      stage_grad_out<S>(static_cast<const E *>(a.grad_out) + p * tile, do_lds, cph, CPH, L, Lq, a.vec != 0);
      stage_bits<3>(src, dst, cph, CPH, L, Lb);
    } else {
      const E *const src[3] = {qkv + qoff, qkv + koff, qkv + voff};
      stage_tiles<S, 3, true, 2>(src, dst, static_cast<const E *>(a.grad_out) + p * tile, do_lds, cph, CPH, L, Lb, Lq,
                                 a.vec != 0);
    }
  }
  __syncthreads();

  ssa_backward_products<S, MC>(a, do_lds, ds_lds, q_lds, k_lds, v_lds, qoff, koff, voff);
}

// ---- the contraction fused with the LIF behind it -------------------------------------------------------------------
// The reference's attention block feeds  out = scale (V K^T) Q  into a multi-step LIF (`attn_lif`, layer/attention.py:
// 321-322, 383-384).  A block owns one (batch element, head) and walks the T steps: the product of step t is still in
// the accumulators when the neuron takes it as its input, the membrane potential of the block's [Cph, L] positions
// stays in registers in the accumulator layout, and `out` is never written.  For the backward the forward leaves h
// (the potential before firing) instead; the backward walks the steps from the last to the first with the gradient of
// the potential in registers, in the layout in which a work-item stages grad_out, forms dL/d out of step t from
// grad_spike and h on the way into LDS and runs the products of ssa_backward_kernel on it.
// Measured at T = 4, 64 x 12 heads of [32, 196] (us per launch): forward 49 against 25 (contraction) + 28 (neuron),
// backward 131 against 82 + 44.  The fused kernels move 8.4 and 20.4 bytes per element instead of 12.4 and 28.4, but
// bytes are not what bounds either side: the forward runs 1216 vector instructions per wavefront and step (the
// expansion of the bits, the gather of Q, the neuron, the transposition of h; vector ALU 48 % busy, memory at
// 3.3 TB/s), a block per (batch element, head) gives only 768 blocks, three or two per compute unit, and each walks
// its steps phase after phase between barriers.  Requesting the next step's bits during the current step and
// writing h and the spikes in whole rows changed nothing (49 us either way).  The callers therefore use these
// kernels only on request (configure.hip_fuse_ssa_lif).
// Makes a wavefront-uniform value opaque to the optimiser at this point of a loop body: what is computed from it (LDS
// addresses, per-row store offsets) is then formed inside the iteration and dies there, instead of being hoisted in
// front of the loop over the steps and held in registers across it.
template <typename T> __device__ __forceinline__ void per_step(T &x) { asm volatile("" : "+s"(x)); }

constexpr int kLifUnits = 2;  // accumulator tiles of a wavefront whose potentials are kept: 32 * MC rows x 256 tokens
constexpr int kLifQuads = 8;  // grad_out quads of a work-item whose potential gradients are kept

struct SsaLifArgs {
  SsaArgs s;             // qkv_bits, heads, cph, L, Lb, Lq, scale; problems = B * heads
  FwdArgs f;             // the neuron's constants (forward)
  BwdArgs b;             // the neuron's constants (backward)
  int64_t T, B;
  const float *v_init;   // [B][heads][cph][L], or one element (f.v_init_broadcast)
  float *spikes;         // [T][B][heads][cph][L]
  float *h_seq;          // forward: written unless null; backward: read
  float *v_last;         // [B][heads][cph][L] or null
  const float *grad_spikes;  // [T][B][heads][cph][L] or null (no gradient reaches the spikes)
  const float *grad_v_last;  // or null
  float *grad_v_init;        // or null
};

template <int MC, int CH, int RS>
__device__ __forceinline__ void ssa_lif_forward_body(const SsaLifArgs &a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ssa_lds[];
  constexpr int CPH = 32 * MC;
  const int L = a.s.L, Lb = a.s.Lb, cph = a.s.cph;
  float *h_lds = reinterpret_cast<float *>(ssa_lds);  // [CPH][Lq]: h of the step, on its way out in whole rows
  uint8_t *q_lds = reinterpret_cast<uint8_t *>(h_lds + CPH * a.s.Lq);
  uint8_t *k_lds = q_lds + CPH * Lb;
  uint8_t *v_lds = k_lds + CPH * Lb;
  uint8_t *const dst[3] = {q_lds, k_lds, v_lds};

  const int64_t bh = blockIdx.x;  // (batch element, head)
  const int64_t batch = bh / a.s.heads, head = bh - batch * a.s.heads;
  const int64_t tile = (int64_t)cph * L;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, half = lane >> 5;
  const int nw = (int)blockDim.x >> 6;
  const int ntiles = (L + 31) / 32;
  const int units = ntiles * MC;  // unit u: output rows 32 (u % MC).., columns 32 (u / MC)..
  const int ni = wave % MC;
  const float tau = a.f.tau, scale = a.s.scale;

  // the potentials of this wavefront's units, in the accumulator layout
  float v[kLifUnits][16];
#pragma unroll
  for (int j = 0; j < kLifUnits; ++j) {
    const int u = wave + j * nw;
    const int col = (u / MC) * 32 + (lane & 31);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = ni * 32 + acc_row(r, lane);
      const bool in = u < units && col < L && row < cph;
      v[j][r] = in ? (a.f.v_init_broadcast ? a.v_init[0] : a.v_init[bh * tile + (int64_t)row * L + col]) : 0.0f;
    }
  }

  // the bits of a step are requested while the step before it is computed
  const int64_t tb = tile / 8;
  uint32_t bits_w[4][3];
  auto request = [&](int64_t t) {
    const int64_t sample = t * a.B + batch;
    const uint8_t *const src[3] = {a.s.qkv_bits + ((sample * 3 + 0) * a.s.heads + head) * tb,
                                   a.s.qkv_bits + ((sample * 3 + 1) * a.s.heads + head) * tb,
                                   a.s.qkv_bits + ((sample * 3 + 2) * a.s.heads + head) * tb};
    request_bits<3>(src, (int)tb, bits_w);
  };
  request(0);
  for (int64_t t = 0; t < a.T; ++t) {
    int L = a.s.L, Lb = a.s.Lb, Lq = a.s.Lq, cph = a.s.cph;
    per_step(L); per_step(Lb); per_step(Lq); per_step(cph);
    const int64_t sample = t * a.B + batch;
    expand_bits<3>(bits_w, dst, cph, CPH, L, Lb);
    __syncthreads();
    request(t + 1 < a.T ? t + 1 : t);  // unconditional: the last step asks for its own bits again
    if (wave < units) {
      bf16x8 s_op[MC][2];
#pragma unroll
      for (int mi = 0; mi < MC; ++mi) {
        const i32x16 acc = spike_gram(k_lds, mi * 32, v_lds, ni * 32, Lb, lane);
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          uint16_t w[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) w[e] = (uint16_t)(__builtin_bit_cast(uint32_t, (float)acc[8 * h2 + e]) >> 16);  // exact: <= 256
          s_op[mi][h2] = __builtin_bit_cast(bf16x8, w);
        }
      }
#pragma unroll
      for (int j = 0; j < kLifUnits; ++j) {
        const int u = wave + j * nw;
        if (u < units) {
          const int nt = u / MC;
          const int col = nt * 32 + (lane & 31);
          const int colc = col < L ? col : L - 1;
          f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
          for (int mi = 0; mi < MC; ++mi) {
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
              uint16_t w[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) {
                const int c2 = mi * 32 + 16 * h2 + 8 * (e >> 2) + 4 * half + (e & 3);
                w[e] = (uint16_t)(q_lds[c2 * Lb + colc] * 0x3f80u);  // 1 -> bf16 1.0
              }
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s_op[mi][h2], __builtin_bit_cast(bf16x8, w), acc, 0, 0, 0);
            }
          }
          float h[16], sp[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) neuron_step<float, CH, RS>(acc[r] * scale, v[j][r], h[r], sp[r], tau, a.f);
          // h goes to LDS in the accumulator layout (a row of 32 tokens per store) and leaves it below in whole rows
          if (col < L) {
            float *hp = h_lds + (ni * 32 + 4 * half) * Lq + col;
#pragma unroll
            for (int r = 0; r < 16; ++r) hp[(8 * (r >> 2) + (r & 3)) * Lq] = h[r];
          }
        }
      }
    }
    __syncthreads();  // h of the step is complete, and the spike tiles are read no more
    {
      // 16 bytes per work-item, consecutive work-items consecutive addresses; the spike is recomputed from h with
      // the comparison of neuron_step
      float *sp_tile = a.spikes + (sample * a.s.heads + head) * tile;
      float *h_tile = a.h_seq ? a.h_seq + (sample * a.s.heads + head) * tile : nullptr;
      const int G = cph * L / 4;
      const float inv_L = 1.0f / (float)L;
      for (int g = threadIdx.x; g < G; g += (int)blockDim.x) {
        const int r = div_tokens(4 * g, inv_L), c = 4 * g - r * L;
        const f32x4 hv = *reinterpret_cast<const f32x4 *>(h_lds + r * Lq + c);
        f32x4 sv;
        {
#pragma clang fp contract(off)
          sv.x = (hv.x - a.f.vth_sub >= 0.0f) ? 1.0f : 0.0f;
          sv.y = (hv.y - a.f.vth_sub >= 0.0f) ? 1.0f : 0.0f;
          sv.z = (hv.z - a.f.vth_sub >= 0.0f) ? 1.0f : 0.0f;
          sv.w = (hv.w - a.f.vth_sub >= 0.0f) ? 1.0f : 0.0f;
        }
        reinterpret_cast<f32x4 *>(sp_tile)[g] = sv;
        if (h_tile) reinterpret_cast<f32x4 *>(h_tile)[g] = hv;
      }
    }
  }

  if (a.v_last) {
#pragma unroll
    for (int j = 0; j < kLifUnits; ++j) {
      const int u = wave + j * nw;
      const int col = (u / MC) * 32 + (lane & 31);
      if (u < units && col < L) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = ni * 32 + acc_row(r, lane);
          if (row < cph) a.v_last[bh * tile + (int64_t)row * L + col] = v[j][r];
        }
      }
    }
  }
}

template <int MC, int CH> __device__ __forceinline__ void ssa_lif_forward_reset(const SsaLifArgs &a) {
  if (a.f.soft_reset) ssa_lif_forward_body<MC, CH, RESET_SOFT>(a);
  else ssa_lif_forward_body<MC, CH, RESET_HARD>(a);
}
// the charge and the reset rule are chosen outside the loop over the steps, so that each copy of the loop holds the
// constants of one rule only
template <int MC>
__global__ void __launch_bounds__(ssa_threads(MC)) ssa_lif_forward_kernel(const SsaLifArgs a) {
  switch (a.f.charge) {
    case CH_IF: ssa_lif_forward_reset<MC, CH_IF>(a); break;
    case CH_DECAY_INPUT_DIV: ssa_lif_forward_reset<MC, CH_DECAY_INPUT_DIV>(a); break;
    case CH_DECAY_INPUT_MUL: ssa_lif_forward_reset<MC, CH_DECAY_INPUT_MUL>(a); break;
    case CH_PLAIN_INPUT_DIV: ssa_lif_forward_reset<MC, CH_PLAIN_INPUT_DIV>(a); break;
    default: ssa_lif_forward_reset<MC, CH_PLAIN_INPUT_MUL>(a); break;
  }
}

// dL/d input and the gradient handed to the step before, for four neurons of one step: the recurrence of
// backward_body (neuron_bwd.h) for IF / LIF with a hard or soft, detached or attached reset.
template <int SG>
__device__ __forceinline__ void lif_quad_backward(const float (&gs)[4], const float (&h)[4], float (&gv)[4], float (&gx)[4],
                                                  const BwdArgs &b, float kx, float km) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma clang fp contract(fast)
    const float over = h[j] - b.v_th;
    const float s = (over >= 0.0f) ? 1.0f : 0.0f;
    const float sg = surrogate_grad<SG, false>(over, b.alpha);
    const float dvdh = (1.0f - s * b.cB) + (b.cC - h[j] * b.cD) * sg;
    const float G = gv[j] * dvdh + gs[j] * sg;
    gx[j] = G * kx;
    gv[j] = G * km;
  }
}
template <int MC, int SG>
__device__ __forceinline__ void ssa_lif_backward_body(const SsaLifArgs &a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ssa_lds[];
  constexpr int CPH = 32 * MC;
  constexpr int LS = CPH + 1;
  const int L = a.s.L, Lb = a.s.Lb, Lq = a.s.Lq, cph = a.s.cph;
  float *do_lds = reinterpret_cast<float *>(ssa_lds);
  float *ds_lds = do_lds + CPH * Lq;
  uint8_t *q_lds = reinterpret_cast<uint8_t *>(ds_lds + CPH * LS);
  uint8_t *k_lds = q_lds + CPH * Lb;
  uint8_t *v_lds = k_lds + CPH * Lb;
  uint8_t *const dst[3] = {q_lds, k_lds, v_lds};

  const int64_t bh = blockIdx.x;
  const int64_t batch = bh / a.s.heads, head = bh - batch * a.s.heads;
  const int64_t tile = (int64_t)cph * L;
  const int tid = threadIdx.x, nthreads = (int)blockDim.x;
  const int G = cph * L / 4;  // quads of a tile; L is a multiple of 4
  const float inv_L = 1.0f / (float)L;
  const float kx = a.b.is_if ? 1.0f : (a.b.decay_input ? a.b.k : 1.0f);
  const float km = a.b.is_if ? 1.0f : (1.0f - a.b.k);

  // gradient of the potential after the step being processed, for the quads this work-item stages
  float gv[kLifQuads][4];
#pragma unroll
  for (int j = 0; j < kLifQuads; ++j) {
    const int g = tid + j * nthreads;
    f32x4 w = {0.0f, 0.0f, 0.0f, 0.0f};
    if (a.grad_v_last && g < G) w = reinterpret_cast<const f32x4 *>(a.grad_v_last + bh * tile)[g];
    gv[j][0] = w.x; gv[j][1] = w.y; gv[j][2] = w.z; gv[j][3] = w.w;
  }
  zero_fill_f32(do_lds, cph, CPH, L, Lq);  // the padding of the grad_out tile: written once, never overwritten

  for (int64_t t = a.T - 1; t >= 0; --t) {
    SsaArgs sa = a.s;
    per_step(sa.L); per_step(sa.Lb); per_step(sa.Lq); per_step(sa.cph);
    const int L = sa.L, Lb = sa.Lb, Lq = sa.Lq, cph = sa.cph;
    const int64_t sample = t * a.B + batch;
    const int64_t p = sample * a.s.heads + head;
    const int64_t qoff = ((sample * 3 + 0) * a.s.heads + head) * tile;
    const int64_t koff = ((sample * 3 + 1) * a.s.heads + head) * tile;
    const int64_t voff = ((sample * 3 + 2) * a.s.heads + head) * tile;
    {
      // dL/d out of this step from grad_spike and h, on its way into LDS
      const f32x4 *gsp = a.grad_spikes ? reinterpret_cast<const f32x4 *>(a.grad_spikes + p * tile) : nullptr;
      const f32x4 *hp = reinterpret_cast<const f32x4 *>(a.h_seq + p * tile);
      f32x4 gs_q[kLifQuads], h_q[kLifQuads];
#pragma unroll
      for (int j = 0; j < kLifQuads; ++j) {
        const int g = tid + j * nthreads;
        const int gc = g < G ? g : G - 1;  // requests are unconditional; what lies beyond the tile is not used
        h_q[j] = hp[gc];
        if (gsp) gs_q[j] = gsp[gc];
        else gs_q[j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
      }
#pragma unroll
      for (int j = 0; j < kLifQuads; ++j) {
        const int g = tid + j * nthreads;
        if (g < G) {
          const float gs[4] = {gs_q[j].x, gs_q[j].y, gs_q[j].z, gs_q[j].w};
          const float h[4] = {h_q[j].x, h_q[j].y, h_q[j].z, h_q[j].w};
          float gx[4];
          lif_quad_backward<SG>(gs, h, gv[j], gx, a.b, kx, km);
          const int r = div_tokens(4 * g, inv_L), c = 4 * g - r * L;
          f32x4 w; w.x = gx[0]; w.y = gx[1]; w.z = gx[2]; w.w = gx[3];
          *reinterpret_cast<f32x4 *>(do_lds + r * Lq + c) = w;
        }
      }
      const uint8_t *const src[3] = {a.s.qkv_bits + qoff / 8, a.s.qkv_bits + koff / 8, a.s.qkv_bits + voff / 8};
      stage_bits<3>(src, dst, cph, CPH, L, Lb);
    }
    __syncthreads();
    ssa_backward_products<float, MC>(sa, do_lds, ds_lds, q_lds, k_lds, v_lds, qoff, koff, voff);
    __syncthreads();  // the tiles are read no more: the step before may overwrite them
  }

  if (a.grad_v_init) {
#pragma unroll
    for (int j = 0; j < kLifQuads; ++j) {
      const int g = tid + j * nthreads;
      if (g < G) {
        f32x4 w; w.x = gv[j][0]; w.y = gv[j][1]; w.z = gv[j][2]; w.w = gv[j][3];
        reinterpret_cast<f32x4 *>(a.grad_v_init + bh * tile)[g] = w;
      }
    }
  }
}

template <int MC>
__global__ void __launch_bounds__(ssa_threads(MC), MC == 1 ? SJHIP_SSA_LIF_BWD_RESIDENT : 1) ssa_lif_backward_kernel(const SsaLifArgs a) {
  switch (a.b.sg) {
    case SJHIP_SG_SIGMOID: ssa_lif_backward_body<MC, SJHIP_SG_SIGMOID>(a); break;
    case SJHIP_SG_ATAN: ssa_lif_backward_body<MC, SJHIP_SG_ATAN>(a); break;
    case SJHIP_SG_PIECEWISE_QUADRATIC: ssa_lif_backward_body<MC, SJHIP_SG_PIECEWISE_QUADRATIC>(a); break;
    case SJHIP_SG_PIECEWISE_EXP: ssa_lif_backward_body<MC, SJHIP_SG_PIECEWISE_EXP>(a); break;
    case SJHIP_SG_SOFT_SIGN: ssa_lif_backward_body<MC, SJHIP_SG_SOFT_SIGN>(a); break;
    case SJHIP_SG_SUPER_SPIKE: ssa_lif_backward_body<MC, SJHIP_SG_SUPER_SPIKE>(a); break;
    default: ssa_lif_backward_body<MC, SJHIP_SG_ERF>(a); break;
  }
}

int lds_row_bytes(int L) { return (L + 31) & ~31; }
int lds_row_f32(int L) { return ((L + 15) & ~15) + 4; }

int padded_rows(int cph) { return cph <= 32 ? 32 : 64; }
unsigned forward_lds(int cph, int L) { return (unsigned)(3 * padded_rows(cph) * lds_row_bytes(L)); }
unsigned backward_lds(int cph, int L) {
  const int c = padded_rows(cph);
  return (unsigned)(3 * c * lds_row_bytes(L) + (c * lds_row_f32(L) + c * (c + 1)) * 4);
}

template <typename K>
int launch_with_lds(K kernel, const SsaArgs &a, int threads, unsigned lds, hipStream_t stream, std::once_flag &once,
                    hipError_t &attr_rc, const char *what) {
  std::call_once(once, [&]() {
    attr_rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)kSsaMaxLds);
    (void)hipGetLastError();
  });
  if (lds > 64u * 1024u && attr_rc != hipSuccess)
    return fail(SJHIP_ERR_LAUNCH, "%s: cannot raise the dynamic LDS limit: %s", what, hipGetErrorString(attr_rc));
  hipLaunchKernelGGL(kernel, dim3((unsigned)a.problems), dim3(threads), lds, stream, a);
  return check_launch(what);
}

template <typename S, int MC>
int launch_fwd(const SsaArgs &a, hipStream_t stream) {
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  return launch_with_lds(ssa_forward_kernel<S, MC>, a, ssa_threads(MC), forward_lds(a.cph, a.L), stream, once, attr_rc, "ssa_forward");
}
template <typename S, int MC>
int launch_bwd(const SsaArgs &a, hipStream_t stream) {
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  return launch_with_lds(ssa_backward_kernel<S, MC>, a, ssa_threads(MC), backward_lds(a.cph, a.L), stream, once, attr_rc, "ssa_backward");
}

template <typename S>
int launch_dtype(const SsaArgs &a, bool backward, hipStream_t stream) {
  if (a.cph <= 32) return backward ? launch_bwd<S, 1>(a, stream) : launch_fwd<S, 1>(a, stream);
  return backward ? launch_bwd<S, 2>(a, stream) : launch_fwd<S, 2>(a, stream);
}

}  // namespace

bool ssa_supported(int dtype, int cph, int64_t L) {
  if (dtype != SJHIP_F32 && dtype != SJHIP_F16 && dtype != SJHIP_BF16) return false;
  if (cph < 1 || cph > 64) return false;
  if (L < 1 || L > 256) return false;  // S = V K^T <= L must stay exact in bf16
  return backward_lds(cph, (int)L) <= kSsaMaxLds;
}

int launch_ssa(bool backward, int dtype, int64_t samples, int heads, int cph, int64_t L, float scale, const void *qkv,
               const uint8_t *qkv_bits, const void *grad_out, void *out, void *grad_qkv, hipStream_t stream) {
  if (!ssa_supported(dtype, cph, L))
    return fail(SJHIP_ERR_UNSUPPORTED, "ssa: dtype %d, %d channels per head, %lld tokens is not supported "
                "(needs at most 64 channels per head, at most 256 tokens, and the tiles of one head fitting in LDS)", dtype, cph, (long long)L);
  if (samples < 1 || heads < 1 || samples * heads > 0x7fffffffLL)
    return fail(SJHIP_ERR_INVALID, "ssa: samples=%lld heads=%d", (long long)samples, heads);
  if (qkv_bits && ((int64_t)cph * L) % 8 != 0)
    return fail(SJHIP_ERR_UNSUPPORTED, "ssa(packed): %d channels x %lld tokens is not a multiple of 8, a tile would not start on a byte",
                cph, (long long)L);
  SsaArgs a;
  a.qkv_bits = qkv_bits;
  a.qkv = qkv; a.grad_out = grad_out; a.out = out; a.grad_qkv = grad_qkv;
  a.problems = samples * heads; a.heads = heads; a.cph = cph; a.L = (int)L;
  a.Lb = lds_row_bytes((int)L); a.Lq = lds_row_f32((int)L); a.scale = scale;
  // four elements per access need every tile base on a four-element boundary
  const uintptr_t quad = dtype == SJHIP_F32 ? 15u : 7u;
  a.vec = (L % 4 == 0) && (qkv_bits != nullptr || (reinterpret_cast<uintptr_t>(qkv) & quad) == 0) &&
          (grad_out == nullptr || (reinterpret_cast<uintptr_t>(grad_out) & quad) == 0);
  ProfileScope prof(backward ? KC_SSA_BACKWARD : KC_SSA_FORWARD, stream);
  switch (dtype) {
    case SJHIP_F32: return launch_dtype<float>(a, backward, stream);
    case SJHIP_F16: return launch_dtype<f16_t>(a, backward, stream);
    default: return launch_dtype<bf16_t>(a, backward, stream);
  }
}

int launch_ssa_lif(bool backward, int neuron, const sjhip_neuron_params &p, int64_t T, int64_t B, int heads, int cph, int64_t L,
                   float scale, const uint8_t *qkv_bits, const float *v_init, float *spikes, float *h_seq, float *v_last,
                   const float *grad_spikes, const float *grad_v_last, float *grad_qkv, float *grad_v_init,
                   hipStream_t stream) {
  const char *what = backward ? "ssa_lif_backward" : "ssa_lif_forward";
  if (neuron != SJHIP_NEURON_IF && neuron != SJHIP_NEURON_LIF)
    return fail(SJHIP_ERR_UNSUPPORTED, "%s: neuron %d (IF and LIF only)", what, neuron);
  if (!ssa_supported(SJHIP_F32, cph, L) || L % 4 != 0 || ((int64_t)cph * L) % 8 != 0)
    return fail(SJHIP_ERR_UNSUPPORTED, "%s: %d channels per head x %lld tokens (at most 64 channels, at most 256 tokens, tokens a "
                "multiple of 4, a tile a multiple of 8 elements)", what, cph, (long long)L);
  if (T < 1 || B < 1 || heads < 1 || B * heads > 0x7fffffffLL || T > (int64_t(1) << 40) / (B * heads))
    return fail(SJHIP_ERR_INVALID, "%s: T=%lld B=%lld heads=%d", what, (long long)T, (long long)B, heads);
  const bool broadcast = (p.flags & SJHIP_FLAG_V_INIT_BROADCAST) != 0;
  if (!aligned16(spikes) || !aligned16(h_seq) || !aligned16(grad_spikes) || !aligned16(grad_v_last) || !aligned16(grad_v_init))
    return fail(SJHIP_ERR_UNSUPPORTED, "%s: spike_seq, h_seq and the gradients must be 16-byte aligned", what);
  SsaLifArgs a;
  const int64_t N = B * heads * cph * L;
  bool round_each = false;
  int rc = build_fwd_args(a.f, round_each, neuron, SJHIP_F32, p, T, N, nullptr, v_init, nullptr, nullptr, nullptr, nullptr, nullptr);
  if (rc != SJHIP_OK) return rc;
  if (backward) {
    rc = build_bwd_args(a.b, neuron, SJHIP_F32, p, T, N, grad_spikes, nullptr, grad_v_last, h_seq, v_init, nullptr, nullptr,
                        grad_v_init, nullptr, nullptr);
    if (rc != SJHIP_OK) return rc;
  } else {
    a.b = BwdArgs();
  }
  a.f.v_init_broadcast = broadcast ? 1 : 0;
  a.s.qkv_bits = qkv_bits; a.s.qkv = nullptr; a.s.grad_out = nullptr; a.s.out = nullptr; a.s.grad_qkv = grad_qkv;
  a.s.problems = B * heads; a.s.heads = heads; a.s.cph = cph; a.s.L = (int)L;
  a.s.Lb = lds_row_bytes((int)L); a.s.Lq = lds_row_f32((int)L); a.s.vec = 1; a.s.scale = scale;
  a.T = T; a.B = B;
  a.v_init = v_init; a.spikes = spikes; a.h_seq = h_seq; a.v_last = v_last;
  a.grad_spikes = grad_spikes; a.grad_v_last = grad_v_last; a.grad_v_init = grad_v_init;
  const int mc = cph <= 32 ? 1 : 2;
  const unsigned lds = backward ? backward_lds(cph, (int)L)
                                : forward_lds(cph, (int)L) + (unsigned)(padded_rows(cph) * lds_row_f32((int)L) * 4);
  const void *kernel = backward ? (mc == 1 ? (const void *)ssa_lif_backward_kernel<1> : (const void *)ssa_lif_backward_kernel<2>)
                                : (mc == 1 ? (const void *)ssa_lif_forward_kernel<1> : (const void *)ssa_lif_forward_kernel<2>);
  static std::once_flag once[4];
  static hipError_t attr_rc[4] = {hipSuccess, hipSuccess, hipSuccess, hipSuccess};
  const int slot = (backward ? 2 : 0) + (mc - 1);
  std::call_once(once[slot], [&]() {
    attr_rc[slot] = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSsaMaxLds);
    (void)hipGetLastError();
  });
  if (lds > 64u * 1024u && attr_rc[slot] != hipSuccess)
    return fail(SJHIP_ERR_LAUNCH, "%s: cannot raise the dynamic LDS limit: %s", what, hipGetErrorString(attr_rc[slot]));
  ProfileScope prof(backward ? KC_SSA_BACKWARD : KC_SSA_FORWARD, stream);
  const dim3 grid((unsigned)(B * heads)), threads(ssa_threads(mc));
  if (backward) {
    if (mc == 1) hipLaunchKernelGGL(ssa_lif_backward_kernel<1>, grid, threads, lds, stream, a);
    else hipLaunchKernelGGL(ssa_lif_backward_kernel<2>, grid, threads, lds, stream, a);
  } else {
    if (mc == 1) hipLaunchKernelGGL(ssa_lif_forward_kernel<1>, grid, threads, lds, stream, a);
    else hipLaunchKernelGGL(ssa_lif_forward_kernel<2>, grid, threads, lds, stream, a);
  }
  return check_launch(what);
}

}  // namespace sjhip
