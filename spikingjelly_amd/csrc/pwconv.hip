// Pointwise (kernel size 1) convolution over [S, C, L] activations on the 16-bit matrix cores with fp32 accuracy.
//
// Two ways of putting fp32 operands on those cores, the same kernels for both (template parameter H):
//   * two fp16 terms (H): x is scaled by a power of two, hi = fp16(x), lo = fp16(x - hi); hi + lo holds x to 2^-23 or
//     better, and hi*hi + hi*lo + lo*hi (three v_mfma_f32_32x32x16_f16 products, fp32 accumulation) drops only lo*lo,
//     below 2^-22 of the product.  The scale keeps the terms inside fp16's exponent range: per row of A for the weights
//     (split_weight_f16_kernel, taken out per row of the result); for activations and gradients the power of two that
//     takes a largest magnitude into [2^14, 2^15): that of the sample in pw_gemm_kernel, whose columns are (sample,
//     position) pairs, that of the whole tensor in the weight gradient, which sums over samples (amax_kernel or the
//     producer of the tensor finds both, the kernels read them from a small device buffer).  Measured: 2^-23 of
//     sum |a||b| against float64.
//   * up to three bf16 terms: no scaling (bf16 has fp32's exponent range), six products for fp32 accuracy; described
//     next, and what the measurements below were taken with unless they say otherwise.  The fp16 split runs the qkv
//     shape in 0.19 ms (forward / input gradient) and 0.24 ms (weight gradient) against 0.27 and 0.30 ms.
//
// The reference computes the block Conv1d(k=1) -> BatchNorm1d -> LIF of its spiking self-attention with torch's
// convolution (layer/attention.py:310-329, 370-384; Conv2d(k=1) in model/spikformer.py:16-99).  A kernel-size-1
// convolution is the GEMM  Y[s] = W X[s]  per sample s, with X[s] a row-major [K, L] tile (tokens contiguous), and its
// backward the two GEMMs  dX[s] = W^T dY[s]  and  dW = sum_s dY[s] X[s]^T.  fp32 operands are split on the fly into up to
// three bf16 terms that sum to the value exactly (round to nearest, remainder, again); the products of the leading
// terms run on v_mfma_f32_32x32x16_bf16 with fp32 accumulation.  With three terms per operand and the six products
// whose combined order is at most two, the dropped part is below 2^-24 of each product: the accuracy of an fp32 GEMM
// at a multiple of the fp32 MFMA rate; an operand that is exact in bf16 (spikes, small counts) needs one term and
// halves the products.  Fewer terms trade accuracy for speed (two terms: about 2^-17 relative per product).
//
//   pw_gemm_kernel     C[s][m][l] = sum_k A[m][k] B[s][k][l]     (forward with A = W, input gradient with A = W^T)
//       A comes pre-split as bf16 planes [3][M_pad / 128][K_pad / 32][128][32] (split_weight_kernel, zero padded), B is
//       fp32 in memory.
//       The S * L columns of all samples form one column index, so tiles of 128 columns carry no padding whatever L
//       is.  A block of four wavefronts owns a 128 x 128 tile (each wavefront 64 x 64 = 2 x 2 MFMA tiles) and walks K
//       in steps of 32.  The matrix cores want, per lane, eight consecutive k of one row (A) or column (B): A tiles are
//       copied to LDS as they are; for B a work-item fetches eight k of two adjacent columns (consecutive lanes fetch
//       consecutive column pairs, so every access of a wavefront is one contiguous run), splits them and stores them
//       k-contiguous, which transposes the tile on the way in and leaves 16-byte fragment reads for both operands.
//       The global loads of the next two tiles are in flight while the current one is multiplied.
//       Measured on the qkv convolution of a Spikformer block (M = 1152, K = 384, 50 176 columns): 0.36 ms with six
//       products, 124 fp32-equivalent TFLOP/s.  Timing the kernel with parts cut out (only the loads 0.12 ms, only the
//       staging 0.05, only fragment reads + MFMA 0.15, empty loop + stores 0.07) gives parts that add up to the whole,
//       and neither wavefronts specialised as producers and consumers over two LDS buffers nor fewer, wider loads
//       changed the total: the phases do not hide behind each other on this chip at this matrix-core load.  Later
//       measurements on the same shape: tile requests made unconditional in the steady state of the K loop (a request
//       under a condition turns every later wait into a wait for all outstanding loads): 0.318 -> 0.301 ms; two LDS
//       buffers of half the depth with one barrier per step, staging of the next tile and multiplication of the current
//       one in the same step: 0.334 ms, and 0.352 ms with scheduler hints that ask for the staging instructions between
//       the matrix-core instructions; not kept.  Two groups of four wavefronts per block, each with its own tile and
//       one barrier apart so that one group multiplies while the other stages: 0.339 against 0.345 ms on random data,
//       not kept either.  The timestamp counter (clock64) around the phases of a K step (one wavefront, steady state):
//       with one block per compute unit staging 1150, multiplication 2160 (48 matrix-core instructions of 32 cycles
//       would be 1536), barriers 320 ticks, 45 k ticks per tile of 30.8 us; with two blocks 1280 / 3060 / 360 and 59 k
//       ticks per tile of 49.3 us: the second block adds a third to the throughput, not a factor of two.  How fast
//       the chip runs depends on what the matrix cores are fed: the same launch on an all-zero input takes 0.265
//       instead of 0.330 ms, and GRBM_GUI_ACTIVE over the kernel's duration gives 1.93 GHz here against 2.5 GHz in a
//       kernel that hardly uses them, so what a better overlap of the phases gains in cycles is partly lost in clock.
//       Raising the wavefront priority for the multiplication (s_setprio 2 around it): 0.348 and 0.331 ms
//       (Y = W X and dX) against 0.338 and 0.300; not kept.
//       By number of products (M = 1152, K = 384, random data): 1 product 0.15-0.16 ms, 2: 0.17-0.18, 3: 0.22,
//       6: 0.33-0.35.  The weight planes are stored tile by tile ([row tile][k step][row][k], 8 KiB per staged tile in
//       a row) so that every 128-byte line a block fetches is used whole: 0.345 -> 0.338 ms, one-term activations
//       0.229 -> 0.215 ms.
//   pw_dw_kernel       dW[m][n] = sum_{s,l} dY[s][m][l] X[s][n][l]
//       both operands are contiguous along the contraction index l; a block owns a 128 x 128 tile of dW for a chunk
//       of samples and writes its partial tile, dw_reduce_kernel adds the chunks in a fixed order.
// Blocks that share operand tiles are numbered so that they run on the same XCD (one L2 each, blocks are dealt
// round-robin over the eight XCDs).
#include "sjhip_common.h"

namespace sjhip {

namespace {


typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kPwThreads = 256;
constexpr int kTile = 128;            // rows and columns of a block's output tile
constexpr int kTileK = 32;            // contraction elements per LDS stage (two MFMA k steps of 16)
constexpr int kRowBytes = 80;         // K-contiguous operand row in LDS: 32 bf16 + 16 bytes, so that the 16-byte fragment
                                      // reads of eight consecutive rows fall on all 32 banks
constexpr int kRowPlane = kTile * kRowBytes;
constexpr int kPlanePitch = 320;      // a k row of a B tile kept as it lies in memory (128 columns of fp16, n contiguous): 256
                                      // bytes + 64, so that the four k rows a transposing read of 32 lanes touches (64 bytes
                                      // of each) fall on distinct banks
static_assert(kTileK * kPlanePitch == kRowPlane, "a B tile takes the same LDS in either layout");
constexpr int kXcds = 8;
// where the B operand of pw_gemm_kernel comes from
constexpr int kBFloat = 0;   // fp32 [S][K][L], split into terms while it is staged
constexpr int kBBits = 1;    // bit-packed spikes over [S][K][L]
constexpr int kBPlanes = 2;  // fp16 term planes [TB][K][ld] with the columns of all samples in a row (split_planes_kernel)
typedef short s16x4 __attribute__((ext_vector_type(4)));
#ifndef SJHIP_PW_F16_WAVES
#define SJHIP_PW_F16_WAVES 3
#endif
// Wavefronts per SIMD of pw_gemm_kernel: with the fp16 split (two operand planes instead of three) 168 registers hold a
// wavefront's state (3 spilled), and a third resident block per compute unit is worth 9 % (191 -> 174 us on the qkv
// shape).  Not so for pw_dw_kernel, which splits both operands on the fly: 22 registers spilled, 237 -> 344 us; with
// one tile in flight instead of two it fits without spilling and takes the same 244 us, and the attention block's
// step 1.50 instead of 1.46 ms.
constexpr int pw_waves(bool h) { return h ? SJHIP_PW_F16_WAVES : 2; }
#ifndef SJHIP_PW_ROWS
#define SJHIP_PW_ROWS 1
#endif

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  bf16x2 p;
  p.x = (__bf16)lo;
  p.y = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, p);
}
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// Word t holds term t of (x0, x1): term 0 is the value rounded to bf16, term 1 the rounded remainder, term 2 what is
// left (exact for fp32 inputs: 3 x 8 significant bits).  The remainders are exact differences.
// With H the terms are fp16 (round to nearest, subnormals kept): two of them hold 22 to 24 significant bits of a value
// whose magnitude lies between 2^-2 and 2^16, which the callers arrange by scaling with a power of two.
template <int TERMS, bool H = false> __device__ __forceinline__ void split_pair(float x0, float x1, uint32_t (&w)[TERMS]) {
#pragma unroll
  for (int t = 0; t < TERMS; ++t) {
    if (H) {
      f16x2 p;
      p.x = (_Float16)x0;
      p.y = (_Float16)x1;
      w[t] = __builtin_bit_cast(uint32_t, p);
      if (t + 1 < TERMS) {
        x0 -= (float)p.x;
        x1 -= (float)p.y;
      }
    } else {
      w[t] = pack_bf16(x0, x1);
      if (t + 1 < TERMS) {
        x0 -= bf16_lo(w[t]);
        x1 -= bf16_hi(w[t]);
      }
    }
  }
}

// The terms of (s x0, s x1) for a power of two s, for the kernels' inner loops.  With two fp16 terms the remainder is one
// fused multiply-add per value, lo = fp16(fma(x, s, -hi)): s x and s x - hi are both exact in fp32, so this is the value
// that the separate product, conversion back and difference of split_pair give, and it compiles to the mixed-precision
// instruction that reads hi as fp16 and writes lo as fp16 (five vector instructions per pair of values instead of ten).
// Otherwise s is not applied (operands of one term, and bf16 terms, are not scaled).
template <int TERMS, bool H> __device__ __forceinline__ void split_scaled_pair(float x0, float x1, float s, uint32_t (&w)[TERMS]) {
  if constexpr (H && TERMS == 2) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    f32x2 y;
    y.x = x0 * s;
    y.y = x1 * s;
    const f16x2 hi = __builtin_convertvector(y, f16x2);
    f16x2 lo;
    lo.x = (_Float16)__builtin_fmaf(x0, s, -(float)hi.x);
    lo.y = (_Float16)__builtin_fmaf(x1, s, -(float)hi.y);
    w[0] = __builtin_bit_cast(uint32_t, hi);
    w[1] = __builtin_bit_cast(uint32_t, lo);
  } else {
    split_pair<TERMS, H>(x0, x1, w);
  }
}

// |x| of a number, 0 for an infinity or a NaN: non-finite elements take no part in choosing a scale (they still
// propagate through the products as they would in fp32).
__device__ __forceinline__ float finite_abs(float x) {
  const float a = fabsf(x);
  return a <= 3.4028234663852886e38f ? a : 0.0f;
}

// The power of two that brings a largest magnitude `amax` into [2^14, 2^15), and its inverse; 1 for a zero, subnormal
// or non-finite amax.  Multiplying by either is exact.
__device__ __forceinline__ void scale_for(float amax, float &scale, float &inverse) {
  const int field = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xffu);
  scale = inverse = 1.0f;
  if (field == 0 || field == 255) return;
  int sf = 268 - field;  // biased exponent of 2^(14 - (field - 127))
  sf = sf < 1 ? 1 : (sf > 253 ? 253 : sf);
  scale = __builtin_bit_cast(float, (uint32_t)sf << 23);
  inverse = __builtin_bit_cast(float, (uint32_t)(254 - sf) << 23);
}

// Block number -> position in the order in which blocks that share tiles should be resident together: hardware block b
// runs on XCD b % 8, so XCD x gets the contiguous range of logical blocks it would get if the grid were cut in eight.
__device__ __forceinline__ int64_t xcd_order(int64_t b, int64_t n) {
  const int64_t q = n / kXcds, r = n % kXcds, x = b % kXcds, i = b / kXcds;
  return x * q + (x < r ? x : r) + i;
}

// planes[t][r][c] = term t of src[r * ld_r + c * ld_c] for r < rows, c < cols, zero in the padding
__global__ void __launch_bounds__(256) split_weight_kernel(const float *src, int64_t rows, int64_t cols, int64_t ld_r,
                                                            int64_t ld_c, int64_t rows_pad, int64_t cols_pad,
                                                            uint16_t *planes) {
  const int64_t pairs = rows_pad * (cols_pad / 2);
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= pairs) return;
  const int64_t r = i / (cols_pad / 2), c = 2 * (i % (cols_pad / 2));
  float x0 = 0.0f, x1 = 0.0f;
  if (r < rows) {
    if (c < cols) x0 = src[r * ld_r + c * ld_c];
    if (c + 1 < cols) x1 = src[r * ld_r + (c + 1) * ld_c];
  }
  uint32_t w[3];
  split_pair<3>(x0, x1, w);
  // tile order: the 128 rows x 32 k that a block stages in one step are 8 KiB in a row, [row tile][k step][row][k]
  const int64_t at = (((r / kTile) * (cols_pad / kTileK) + c / kTileK) * kTile + r % kTile) * kTileK + c % kTileK;
#pragma unroll
  for (int t = 0; t < 3; ++t)
    reinterpret_cast<uint32_t *>(planes + (int64_t)t * rows_pad * cols_pad)[at / 2] = w[t];
}

// fp16 planes[t][tile order] = term t of scale_r * src[r][c], with a power-of-two scale per row r (a row of A is a row
// of the product, so the GEMM's epilogue takes the scale out again); the inverse scales follow the two planes as
// rows_pad floats.  One wavefront per row.
__global__ void __launch_bounds__(256) split_weight_f16_kernel(const float *src, int64_t rows, int64_t cols, int64_t ld_r,
                                                                int64_t ld_c, int64_t rows_pad, int64_t cols_pad,
                                                                uint16_t *planes, float *amax_reset, int64_t amax_floats) {
  if (amax_reset && blockIdx.x == 0)
    for (int64_t i = threadIdx.x; i < amax_floats; i += 256) amax_reset[i] = 0.0f;
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows_pad) return;
  float amax = 0.0f;
  if (r < rows) {
#pragma unroll 8
    for (int64_t c = lane; c < cols; c += 64) amax = fmaxf(amax, finite_abs(src[r * ld_r + c * ld_c]));
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
  float scale, inverse;
  scale_for(amax, scale, inverse);
#pragma unroll 4
  for (int64_t c = 2 * lane; c < cols_pad; c += 128) {
    float x0 = 0.0f, x1 = 0.0f;
    if (r < rows) {
      if (c < cols) x0 = src[r * ld_r + c * ld_c] * scale;
      if (c + 1 < cols) x1 = src[r * ld_r + (c + 1) * ld_c] * scale;
    }
    uint32_t w[2];
    split_pair<2, true>(x0, x1, w);
    const int64_t at = (((r / kTile) * (cols_pad / kTileK) + c / kTileK) * kTile + r % kTile) * kTileK + c % kTileK;
#pragma unroll
    for (int t = 0; t < 2; ++t)
      reinterpret_cast<uint32_t *>(planes + (int64_t)t * rows_pad * cols_pad)[at / 2] = w[t];
  }
  if (lane == 0) reinterpret_cast<float *>(planes + 2 * rows_pad * cols_pad)[r] = inverse;
}

// The largest magnitude of a tensor is kept as SJHIP_PW_AMAX_FLOATS non-negative floats whose maximum it is: blocks fold
// their share into word (block % SJHIP_PW_AMAX_FLOATS) with an integer atomic maximum (the bit patterns of non-negative
// floats order like unsigned integers, and a maximum does not depend on the order it is taken in).  Several words,
// and an atomic whose result is not used, so that a block neither meets tens of thousands of others on one address nor
// waits for memory before it ends: the kernel that writes the gradients of the qkv convolution takes 73 us with it
// (68 without), against 109 us with one word that a block reads first to skip atomics that would not raise it, and
// 93 us with that read spread over 256 words.
__device__ __forceinline__ void fold_amax(unsigned *amax_bits, float block_max) {
  atomicMax(amax_bits + blockIdx.x % SJHIP_PW_AMAX_FLOATS, __builtin_bit_cast(unsigned, block_max));
}
// The maximum of those words, in every lane of a wavefront.
__device__ __forceinline__ float tensor_amax(const float *amax) {
  static_assert(SJHIP_PW_AMAX_FLOATS == 256, "one 16-byte load per lane");
  const f32x4 v = reinterpret_cast<const f32x4 *>(amax)[threadIdx.x & 63];
  float m = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) m = fmaxf(m, __shfl_xor(m, d));
  return m;
}
// The words of every sample's own largest magnitude follow the SJHIP_PW_AMAX_FLOATS words of the tensor's
// (SJHIP_PW_AMAX_SAMPLE_WORDS adjacent words per sample, whose maximum is the sample's amax: blocks that run at the
// same time belong to one sample, and atomics on one address are served one after the other): the GEMMs whose
// columns are (sample, position) pairs scale every sample by its own power of two (a sample whose values are all small
// beside another's keeps its significant bits), the weight gradient, which sums over the samples, by the tensor's.
__device__ __forceinline__ float sample_amax(const float *sample_words, int64_t s) {
  static_assert(SJHIP_PW_AMAX_SAMPLE_WORDS == 16, "four 16-byte loads per sample");
  const f32x4 *p = reinterpret_cast<const f32x4 *>(sample_words) + 4 * s;
  const f32x4 a = p[0], b = p[1], c = p[2], d = p[3];
  const f32x4 m = {fmaxf(fmaxf(a.x, b.x), fmaxf(c.x, d.x)), fmaxf(fmaxf(a.y, b.y), fmaxf(c.y, d.y)),
                   fmaxf(fmaxf(a.z, b.z), fmaxf(c.z, d.z)), fmaxf(fmaxf(a.w, b.w), fmaxf(c.w, d.w))};
  return fmaxf(fmaxf(m.x, m.y), fmaxf(m.z, m.w));
}
// x holds samples of per_sample elements each (a multiple of 4 when x is 16-byte aligned, so that a 16-byte access lies
// in one sample); a block takes 4096 consecutive elements.  One atomic per block for the tensor's words and one for
// a word of each of the (nearly always one, at most two) samples it lies in; what lies in further samples (samples
// shorter than a block) the work-items fold themselves.
constexpr int kAmaxChunk = 4096;
__global__ void __launch_bounds__(256) amax_kernel(const float *x, int64_t S, int64_t per_sample, unsigned *amax_bits) {
  const int64_t n = S * per_sample;
  __shared__ float part[4], part_first[4], part_second[4];
  unsigned *sample_bits = amax_bits + SJHIP_PW_AMAX_FLOATS + blockIdx.x % SJHIP_PW_AMAX_SAMPLE_WORDS;
  constexpr int64_t kW = SJHIP_PW_AMAX_SAMPLE_WORDS;
  const int64_t e0 = (int64_t)blockIdx.x * kAmaxChunk;
  const int64_t s0 = e0 / per_sample;                // the block's first sample (the same for every work-item)
  const int64_t next = (s0 + 1) * per_sample;        // first element of the following sample
  float amax = 0.0f;                                 // over everything the work-item reads
  float first = 0.0f, second = 0.0f;                 // over its elements of samples s0 and s0 + 1
  auto take = [&](int64_t e, float m) {
    amax = fmaxf(amax, m);
    if (e < next) first = fmaxf(first, m);
    else if (e < next + per_sample) second = fmaxf(second, m);
    else atomicMax(sample_bits + kW * (e / per_sample), __builtin_bit_cast(unsigned, m));  // (samples shorter than a block)
  };
  if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0 && per_sample % 4 == 0) {
    f32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t e = e0 + (int64_t)(k * 256 + threadIdx.x) * 4;
      v[k] = e + 4 <= n ? __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x + e)) : (f32x4)(0.0f);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int64_t e = e0 + (int64_t)(k * 256 + threadIdx.x) * 4;
      if (e + 4 <= n) take(e, fmaxf(fmaxf(finite_abs(v[k].x), finite_abs(v[k].y)), fmaxf(finite_abs(v[k].z), finite_abs(v[k].w))));
    }
  } else {  // any alignment, any sample length: element by element
    for (int k = 0; k < 16; ++k) {
      const int64_t e = e0 + (int64_t)k * 256 + threadIdx.x;
      if (e < n) take(e, finite_abs(x[e]));
    }
  }
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) {
    amax = fmaxf(amax, __shfl_xor(amax, d));
    first = fmaxf(first, __shfl_xor(first, d));
    second = fmaxf(second, __shfl_xor(second, d));
  }
  if ((threadIdx.x & 63) == 0) {
    part[threadIdx.x >> 6] = amax;
    part_first[threadIdx.x >> 6] = first;
    part_second[threadIdx.x >> 6] = second;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    fold_amax(amax_bits, fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3])));
    if (e0 < n) atomicMax(sample_bits + kW * s0, __builtin_bit_cast(unsigned, fmaxf(fmaxf(part_first[0], part_first[1]), fmaxf(part_first[2], part_first[3]))));
    if (next < n && next < e0 + kAmaxChunk)
      atomicMax(sample_bits + kW * (s0 + 1), __builtin_bit_cast(unsigned, fmaxf(fmaxf(part_second[0], part_second[1]), fmaxf(part_second[2], part_second[3]))));
  }
}

struct PwGemmArgs {
  const uint16_t *a_planes;  // [3][M_pad / 128][K_pad / 32][128][32] bf16
  const float *b;            // [S][K][L]
  float *c;                  // [S][M][L]
  int64_t plane_stride;      // M_pad * K_pad
  int64_t ncols;             // S * L
  int M, K, K_pad, L;
  int m_blocks;
  float *stats;              // nullptr, or [2 x column blocks][M][2]: per row of c the sum and the sum of squares over
                             // each half (64 columns) of every column block
  const float *a_inverse;    // fp16 terms: the inverse scale of every (padded) row of A
  const float *b_amax;       // fp16 terms: nullptr (b needs no scale), or the words whose maximum is max |b|
  const float *b_amax_samples;  // kBFloat with two fp16 terms: the per-sample words of b's amax buffer (they follow b_amax's words)
  int64_t amax_s0, amax_S;      // the first sample of this launch, the samples of the tensor
  const uint16_t *b_planes;  // kBPlanes: fp16 terms of b, [TB][K][ld], column s * L + l of row k holds b[s][k][l]
  int64_t b_plane_stride;    // K * ld
  int ld;                    // columns per row of a plane: a multiple of 8, at least ncols
  int wide_out;              // L is a multiple of 4 and c is 16-byte aligned: the tile leaves through LDS as 16-byte row pieces
};
#ifndef SJHIP_PW_WIDE_OUT
#define SJHIP_PW_WIDE_OUT 1
#endif
constexpr int kOutPitch = 68;                              // floats per row of the output staging buffer (64 columns + 4)
constexpr unsigned kOutLds = 4 * 32 * kOutPitch * 4;       // 32 rows x 64 columns per wavefront
constexpr int kStatPitch = 33;                             // floats per row of the transposing buffer: no bank conflicts
constexpr unsigned kStatLds = 4 * 64 * kStatPitch * 4;     // one buffer of 64 rows x 32 column pairs per wavefront

// Term pairs whose product is kept: combined order at most max(TA, TB) - 1.
template <int TA, int TB> struct Pairs {
  static constexpr int kMax = (TA > TB ? TA : TB) - 1;
  static __device__ __forceinline__ constexpr bool keep(int ta, int tb) { return ta + tb <= kMax; }
};

// One k step of 16 for a wavefront's 2 x 2 tiles: operands in registers, smallest terms first.
template <int TA, int TB, bool H>
__device__ __forceinline__ void mfma_step(const u32x4 (&af)[2][TA], const u32x4 (&bf)[2][TB], f32x16 (&acc)[2][2]) {
#pragma unroll
  for (int order = Pairs<TA, TB>::kMax; order >= 0; --order) {
#pragma unroll
    for (int ta = 0; ta < TA; ++ta) {
      const int tb = order - ta;
      if (tb < 0 || tb >= TB) continue;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
          acc[mt][nt] = H ? __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, af[mt][ta]),
                                                                    __builtin_bit_cast(f16x8, bf[nt][tb]), acc[mt][nt], 0, 0, 0)
                          : __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[mt][ta]),
                                                                     __builtin_bit_cast(bf16x8, bf[nt][tb]), acc[mt][nt], 0, 0, 0);
    }
  }
}

// Fragment of a K-contiguous operand: row `row` of the tile, k group (lane / 32) of k step ks.
__device__ __forceinline__ u32x4 row_fragment(const uint8_t *plane, int row, int ks, int lane) {
  return *reinterpret_cast<const u32x4 *>(plane + row * kRowBytes + ks * 32 + (lane >> 5) * 16);
}

// BSRC == kBBits: b is a spike tensor that arrives bit-packed (the layout of sjhip_bit_pack over [S][K][L]: bit e % 8 of
// byte e / 8 is element e), 1/32 of the bytes of fp32 spikes; a work-item fetches the byte that holds its two columns of
// a row.
// BSRC == kBPlanes: b arrives as fp16 term planes that its producer wrote already scaled and split, rows of K with the
// columns of all samples in a row.  A tile of 32 k x 128 columns is copied to LDS as it lies in memory (16 bytes per
// work-item and row, no arithmetic), and the wavefronts fetch their fragments with the transposing LDS read
// (ds_read_b64_tr_b16: the 16 lanes of a group each point at four consecutive columns of a k row, four rows of 16
// columns in all, and lane j of the group receives column j of the four rows), which delivers the eight consecutive k of
// a column that the matrix cores want from a tile whose rows run along the columns.
template <int TA, int TB, bool H, int BSRC = kBFloat>
__global__ void __launch_bounds__(kPwThreads) __attribute__((amdgpu_waves_per_eu(pw_waves(H), pw_waves(H)))) pw_gemm_kernel(const PwGemmArgs a) {
  constexpr bool BITS = BSRC == kBBits;
  constexpr bool PLANES = BSRC == kBPlanes;
  static_assert(!BITS || TB == 1, "a bit-packed operand has one term");
  static_assert(!PLANES || H, "term planes are fp16");
  extern __shared__ __align__(16) uint8_t lds[];
  uint8_t *As = lds;                   // [TA][128][kRowBytes]
  uint8_t *Bs = lds + TA * kRowPlane;  // [TB][128][kRowBytes], column-major: a row holds 32 k of one column
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t logical = xcd_order(blockIdx.x, gridDim.x);
  const int mb = (int)(logical % a.m_blocks);
  const int64_t nb = logical / a.m_blocks;
  const int m0 = mb * kTile;
  const int64_t j0 = nb * kTile;
  const int M = a.M, K = a.K, L = a.L;
  const int K_pad = a.K_pad;

  // Addresses are a wavefront-uniform 64-bit base (scalar registers) plus a 32-bit per-lane byte offset, and every load
  // is unconditional (a branch per load would serialise them): offsets are clamped into the tensors and what lies
  // outside the matrices is zeroed, under one uniform branch, when the tile is staged.
  // A: two 16-byte chunks per term and thread; chunk q = tid + 256 i -> row q / 4, k chunk q % 4
  uint32_t a_off[2];
  int a_dst[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = tid + kPwThreads * i, row = q >> 2, kc = q & 3;
    a_off[i] = (uint32_t)((mb * (K_pad / kTileK) * (kTile * kTileK) + 8 * q) * 2);
    a_dst[i] = row * kRowBytes + kc * 16;
  }
  // B: eight k (one fragment) of two adjacent columns, fetched as 8-byte accesses: columns 2 (tid % 64) and the next,
  // k group = the wavefront's number.  Consecutive lanes fetch consecutive column pairs, so every access of a wavefront
  // is one contiguous run, and a lane ends up with the eight k of a column that the matrix cores want from it.
  const int bc = 2 * (tid & 63);
  const int bk = __builtin_amdgcn_readfirstlane(wave * 8);
  const int64_t jc = j0 + bc;
  const bool col_ok = jc < a.ncols;  // L is even, so the two columns are in one sample and both valid or both not
  uint32_t b_off = 0;  // byte offset of the column pair in row 0 of its sample; with BITS the bit index
  if (col_ok) {
    const int64_t s = jc / L;
    b_off = (uint32_t)(((s * K) * (int64_t)L + (jc - s * L)) * (BITS ? 1 : 4));
  }
  const bool edge_cols = __builtin_amdgcn_readfirstlane(j0 + kTile > a.ncols ? 1 : 0) != 0;
  const char *a_base = reinterpret_cast<const char *>(a.a_planes);
  const char *b_base = reinterpret_cast<const char *>(a.b);
  // The scale of b: a sample's own power of two when b is split here (a work-item stages columns of one sample), the
  // tensor's when b arrives as planes (split with it).
  constexpr bool SAMPLE_SCALE = H && TB > 1 && BSRC == kBFloat;
  float b_scale = 1.0f, b_inverse = 1.0f;
  if (H && TB > 1 && !SAMPLE_SCALE && a.b_amax != nullptr) scale_for(tensor_amax(a.b_amax), b_scale, b_inverse);
  // A tile of 128 columns lies in at most two samples when a sample has that many positions: their two maxima are
  // fetched once per block from addresses that do not depend on the lane; shorter samples are looked up per column.
  const bool two_samples = L >= kTile;
  const int64_t tile_sample = j0 / L, next_sample_col = (tile_sample + 1) * L;
  float tile_amax[2] = {0.0f, 0.0f};
  if (SAMPLE_SCALE && a.b_amax_samples != nullptr && two_samples) {
    const int64_t s_a = a.amax_s0 + tile_sample, s_b = s_a + 1 < a.amax_S ? s_a + 1 : s_a;
    tile_amax[0] = sample_amax(a.b_amax_samples, s_a);
    tile_amax[1] = sample_amax(a.b_amax_samples, s_b);
  }
  auto column_amax = [&](int64_t j) {
    return two_samples ? (j < next_sample_col ? tile_amax[0] : tile_amax[1]) : sample_amax(a.b_amax_samples, a.amax_s0 + j / L);
  };
  if (SAMPLE_SCALE && a.b_amax_samples != nullptr && col_ok) scale_for(column_amax(jc), b_scale, b_inverse);
  // planes: 16-byte chunk pc (eight columns) of the k rows pr and pr + 16 of every plane
  const int pc = tid & 15, pr = tid >> 4;
  const uint32_t ld2 = PLANES ? (uint32_t)a.ld * 2u : 0u;
  const uint32_t p_col = (PLANES && j0 + 8 * pc < a.ld) ? 16u * pc : 0u;  // (ld is a multiple of 8: a chunk is inside a row or not)
  const char *bp_base = reinterpret_cast<const char *>(a.b_planes) + j0 * 2;

  // Two B tiles are in flight in registers (sets 0 and 1): a tile is requested two multiplications before it is staged,
  // which covers a miss to HBM.  The A tiles (weight planes, a few MB that every block reads) come from L2, one ahead.
  u32x4 ra[TA][2];
  u32x2 rb[2][8];       // [set][k]: the fp32 bit patterns of the two columns
  u32x4 rbp[2][TB][2];  // planes: [set][term][row pr + 16 i]  (of rb and rbp only the one that the mode uses exists)
  auto fetch_a = [&](int k0) {
#pragma unroll
    for (int t = 0; t < TA; ++t) {
      const char *plane = a_base + ((int64_t)t * a.plane_stride + (int64_t)(k0 / kTileK) * (kTile * kTileK)) * 2;
#pragma unroll
      for (int i = 0; i < 2; ++i) ra[t][i] = *reinterpret_cast<const u32x4 *>(plane + a_off[i]);
    }
  };
  auto fetch_b = [&](int k0, int set) {
    if constexpr (PLANES) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int k = k0 + pr + 16 * i;
        const uint32_t off = (uint32_t)(k < K ? k : K - 1) * ld2 + p_col;
#pragma unroll
        for (int t = 0; t < TB; ++t)
          rbp[set][t][i] = *reinterpret_cast<const u32x4 *>(bp_base + (int64_t)t * a.b_plane_stride * 2 + off);
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + bk + i;
      if (BITS) {  // K * L is a multiple of 8 and L is even: the two bits share a byte
        const uint32_t e = b_off + (uint32_t)(k < K ? k : K - 1) * (uint32_t)L;
        rb[set][i].x = *reinterpret_cast<const uint8_t *>(b_base + (e >> 3));
        rb[set][i].y = e & 7u;
        continue;
      }
      const char *row = b_base + (int64_t)(k < K ? k : K - 1) * L * 4;
      rb[set][i] = *reinterpret_cast<const u32x2 *>(row + b_off);
    }
  };
  auto stage = [&](int k0, int set) {
#pragma unroll
    for (int t = 0; t < TA; ++t)
#pragma unroll
      for (int i = 0; i < 2; ++i) *reinterpret_cast<u32x4 *>(As + t * kRowPlane + a_dst[i]) = ra[t][i];
    if constexpr (PLANES) {
      if (edge_cols || k0 + kTileK > K) {  // rows beyond K and columns beyond the matrix hold zeros
        const int64_t left = a.ncols - (j0 + 8 * pc);
        const int nvalid = left < 0 ? 0 : (left > 8 ? 8 : (int)left);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int n = (k0 + pr + 16 * i < K) ? nvalid : 0;
#pragma unroll
          for (int t = 0; t < TB; ++t) {
            u32x4 &v = rbp[set][t][i];
            v.x &= n >= 2 ? 0xffffffffu : (n == 1 ? 0xffffu : 0u);
            v.y &= n >= 4 ? 0xffffffffu : (n == 3 ? 0xffffu : 0u);
            v.z &= n >= 6 ? 0xffffffffu : (n == 5 ? 0xffffu : 0u);
            v.w &= n >= 8 ? 0xffffffffu : (n == 7 ? 0xffffu : 0u);
          }
        }
      }
#pragma unroll
      for (int t = 0; t < TB; ++t)
#pragma unroll
        for (int i = 0; i < 2; ++i)
          *reinterpret_cast<u32x4 *>(Bs + t * kRowPlane + (pr + 16 * i) * kPlanePitch + pc * 16) = rbp[set][t][i];
      return;
    }
    if (edge_cols || k0 + kTileK > K) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (!(col_ok && k0 + bk + i < K)) rb[set][i] = (u32x2)(0u);
    }
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      uint32_t w[4][TB];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u32x2 lo = rb[set][2 * i], hi = rb[set][2 * i + 1];
        float x0 = __builtin_bit_cast(float, c ? lo.y : lo.x), x1 = __builtin_bit_cast(float, c ? hi.y : hi.x);
        if (BITS) {
          x0 = (float)((lo.x >> (lo.y + c)) & 1u);
          x1 = (float)((hi.x >> (hi.y + c)) & 1u);
        }
        split_scaled_pair<TB, H>(x0, x1, b_scale, w[i]);
      }
#pragma unroll
      for (int t = 0; t < TB; ++t) {
        u32x4 v;
        v.x = w[0][t]; v.y = w[1][t]; v.z = w[2][t]; v.w = w[3][t];
        *reinterpret_cast<u32x4 *>(Bs + t * kRowPlane + (bc + c) * kRowBytes + bk * 2) = v;
      }
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;

  auto multiply = [&]() {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4 af[2][TA], bf[2][TB];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int t = 0; t < TA; ++t) af[mt][t] = row_fragment(As + t * kRowPlane, wm * 64 + mt * 32 + (lane & 31), ks, lane);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int t = 0; t < TB; ++t) {
          if constexpr (PLANES) {
            // group g = lane / 16 of a transposing read: columns 16 (g % 2) + 0..15 of the 32, k rows 8 (g / 2) + 0..3 (and + 4
            // in the second read) of the 16; lane i of the group points at columns 4 (i % 4) + 0..3 of row i / 4
            const int g = lane >> 4, i = lane & 15;
            const uint8_t *src = Bs + t * kRowPlane + (ks * 16 + 8 * (g >> 1) + (i >> 2)) * kPlanePitch +
                                 (wn * 64 + nt * 32 + 16 * (g & 1) + 4 * (i & 3)) * 2;
            typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
            const u32x2 k03 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(src)));
            const u32x2 k47 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(src + 4 * kPlanePitch)));
            bf[nt][t].x = k03.x; bf[nt][t].y = k03.y; bf[nt][t].z = k47.x; bf[nt][t].w = k47.y;
          } else {
            bf[nt][t] = row_fragment(Bs + t * kRowPlane, wn * 64 + nt * 32 + (lane & 31), ks, lane);
          }
        }
      mfma_step<TA, TB, H>(af, bf, acc);
    }
  };
  // One K step: stage the tile whose loads were requested earlier, request later tiles, multiply.  In the steady state
  // both requests are unconditional, so the compiler knows how many younger loads are outstanding when it waits for the
  // tile being staged and leaves them in flight; a request under a condition makes it wait for everything (vmcnt(0)),
  // which is tolerable only in the last steps.
  auto step = [&](int k0, int set, bool more_a, bool more_b) {
    __syncthreads();  // the previous tile has been read by every wavefront
    stage(k0, set);
    __syncthreads();
    if (more_a) fetch_a(k0 + kTileK);
    if (more_b) fetch_b(k0 + 2 * kTileK, set);
    multiply();
  };
  fetch_b(0, 0);
  fetch_a(0);
  fetch_b(kTileK, 1);  // rows beyond K are clamped, the tile is never staged then
  int k0 = 0;
  for (; k0 + 3 * kTileK < K_pad; k0 += 2 * kTileK) {
    step(k0, 0, true, true);
    step(k0 + kTileK, 1, true, true);
  }
  if (k0 < K_pad) step(k0, 0, k0 + kTileK < K_pad, k0 + 2 * kTileK < K_pad);
  if (k0 + kTileK < K_pad) step(k0 + kTileK, 1, k0 + 2 * kTileK < K_pad, false);
  if (k0 + 2 * kTileK < K_pad) step(k0 + 2 * kTileK, 0, false, false);

  // accumulator register r of a 32 x 32 tile: row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32
  float b_inv_col[2] = {b_inverse, b_inverse};  // of the two columns whose results this lane holds
  if (SAMPLE_SCALE && a.b_amax_samples != nullptr) {
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int64_t j = j0 + wn * 64 + nt * 32 + (lane & 31);
      float unused;
      b_inv_col[nt] = 1.0f;
      if (j < a.ncols) scale_for(column_amax(j), unused, b_inv_col[nt]);
    }
  }
  if (H) {  // take the power-of-two scales of the row of A and of b out again: exact
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float inv = a.a_inverse[m0 + wm * 64 + mt * 32 + 4 * (lane >> 5) + 8 * (r >> 2) + (r & 3)];
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) acc[mt][nt][r] = acc[mt][nt][r] * inv * b_inv_col[nt];
      }
  }
  if (a.wide_out) {
    // The accumulators hold four rows of one column per group of registers, so a direct store writes 4-byte pieces of
    // 128-byte row segments, 64 instructions per wavefront.  Through LDS a wavefront's 64 x 64 tile leaves in two halves
    // of 32 rows as 16-byte pieces: a store instruction writes four rows of 256 contiguous bytes, 16 per wavefront.  A
    // piece of four columns lies in one sample (L is a multiple of 4).
    float *buf = reinterpret_cast<float *>(lds) + wave * (32 * kOutPitch);
    const int c4 = 4 * (lane & 15), rsub = lane >> 4;
    const int64_t j4 = j0 + wn * 64 + c4;
    const bool ok4 = j4 < a.ncols;
    const int64_t s4 = ok4 ? j4 / L : 0;
    float *cp4 = a.c + (s4 * M) * (int64_t)L + (ok4 ? (int)(j4 - s4 * L) : 0);
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      __syncthreads();  // the operand tiles (first half) or the rows of the first half (second) are no longer read
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          buf[(8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)) * kOutPitch + nt * 32 + (lane & 31)] = acc[mt][nt][r];
      __syncthreads();
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int row_local = 4 * i + rsub;
        const int row = m0 + wm * 64 + mt * 32 + row_local;
        const f32x4 v = *reinterpret_cast<const f32x4 *>(buf + row_local * kOutPitch + c4);
        if (ok4 && row < M) *reinterpret_cast<f32x4 *>(cp4 + (int64_t)row * L) = v;
      }
      // the batch-norm sums of these 32 rows over the wavefront's 64 columns (columns beyond the matrix hold exact
      // zeros): lane i adds row i from the staged half, in a fixed order
      if (a.stats && lane < 32) {
        const float *rowp = buf + lane * kOutPitch;
        float sum = 0.0f, squares = 0.0f;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const f32x4 v = *reinterpret_cast<const f32x4 *>(rowp + 4 * j);
          sum += (v.x + v.y) + (v.z + v.w);
          squares = fmaf(v.x, v.x, squares); squares = fmaf(v.y, v.y, squares);
          squares = fmaf(v.z, v.z, squares); squares = fmaf(v.w, v.w, squares);
        }
        const int row = m0 + wm * 64 + mt * 32 + lane;
        if (row < M) {
          float *out = a.stats + ((2 * nb + wn) * (int64_t)M + row) * 2;
          out[0] = sum;
          out[1] = squares;
        }
      }
    }
    return;
  } else {
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int64_t j = j0 + wn * 64 + nt * 32 + (lane & 31);
      if (j >= a.ncols) continue;
      const int64_t s = j / L;
      const int l = (int)(j - s * L);
      float *cp = a.c + (s * M) * (int64_t)L + l;
  #pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const int rbase = m0 + wm * 64 + mt * 32 + 4 * (lane >> 5);
  #pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = rbase + 8 * (r >> 2) + (r & 3);
          if (row < M) cp[(int64_t)row * L] = acc[mt][nt][r];
        }
      }
    }
  
}

  // Batch-norm statistics of the tile, so that no kernel has to read c again for them: per row the sum and the sum of
  // squares over the wavefront's 64 columns (columns beyond the matrix hold exact zeros).  A lane holds 32 rows of one
  // column pair; the values go through LDS, transposed, and lane i adds the 32 pairs of row i in a fixed order.
  if (a.stats) {
    __syncthreads();  // the operand tiles are no longer read
    float *buf = reinterpret_cast<float *>(lds) + wave * (64 * kStatPitch);
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float v0 = acc[mt][0][r], v1 = acc[mt][1][r];
          const int row_local = mt * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          buf[row_local * kStatPitch + (lane & 31)] = pass == 0 ? v0 + v1 : v0 * v0 + v1 * v1;
        }
      __syncthreads();
      float sum = 0.0f;
#pragma unroll
      for (int j = 0; j < 32; ++j) sum += buf[lane * kStatPitch + j];
      const int row = m0 + wm * 64 + lane;
      if (row < M) a.stats[((2 * nb + wn) * (int64_t)M + row) * 2 + pass] = sum;
      __syncthreads();
    }
  }
}

// LDS of pw_gemm_rows_kernel: two B tiles (or the output staging of the epilogue, whichever is larger), then 128 floats
constexpr unsigned rows_inverse_offset(int tb) { return 2u * tb * kRowPlane > kOutLds ? 2u * tb * kRowPlane : kOutLds; }

// pw_gemm_rows_kernel: the same product, term order and batch-norm sums as pw_gemm_kernel<2, TB, true, kBFloat> (bit for
// bit), laid out for what a compute unit can move.  Measured per compute unit: LDS reads of 16 bytes per lane run at
// 256 bytes per cycle but writes at 64-78, and the vector memory path issues one wavefront load of 8 or 16 bytes per lane
// every 16 cycles (58 bytes per cycle from L1), so in pw_gemm_kernel a K step of a block costs about as many cycles of LDS
// (16 KB of A and 16 KB of B written, 64 KB read) and of the load path (32 eight-byte loads of B, 16 of A) as of the matrix
// cores (768 per SIMD).  Here
//   * a wavefront owns 32 rows of the tile and all 128 columns, and fetches its A fragments straight from the weight
//     planes (the 16 bytes a lane needs are contiguous in the tile-ordered planes): A never passes through LDS and no two
//     wavefronts fetch the same fragment;
//   * B is fetched as 16-byte pieces of a k row (four positions of one sample; L is a multiple of 4), half the load
//     instructions, split, and stored as it lies in memory (k rows of 128 columns); the wavefronts fetch their
//     fragments with the transposing LDS read, as pw_gemm_kernel does for term planes;
//   * two B tiles alternate in LDS, so a K step has one barrier.
// Per K step of a block: 16 KB written to and 64 KB read from LDS, 16 + 16 load instructions; 146 registers, three
// wavefronts per SIMD.
template <int TB>
__global__ void __launch_bounds__(kPwThreads) __attribute__((amdgpu_waves_per_eu(3, 3))) pw_gemm_rows_kernel(const PwGemmArgs a) {
  constexpr int TA = 2;
  constexpr int kBuf = TB * kRowPlane;  // one B tile: [TB][32 k][kPlanePitch]
  extern __shared__ __align__(16) uint8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t logical = xcd_order(blockIdx.x, gridDim.x);
  const int mb = (int)(logical % a.m_blocks);
  const int64_t nb = logical / a.m_blocks;
  const int64_t j0 = nb * kTile;
  const int M = a.M, K = a.K, L = a.L;
  const int steps = a.K_pad / kTileK;

  // the inverse row scales of the tile wait in LDS (beyond the operand tiles) for the epilogue
  float *inverse_lds = reinterpret_cast<float *>(lds + rows_inverse_offset(TB));
  const float inverse_mine = tid < kTile ? a.a_inverse[mb * kTile + tid] : 0.0f;

  // A: lane (r, g) wants k chunk 2 ks + g (eight k, 16 bytes) of row r of the wavefront's 32 rows
  const char *a_base = reinterpret_cast<const char *>(a.a_planes) + (int64_t)mb * steps * (kTile * kTileK * 2);
  const uint32_t a_lane = (uint32_t)(((wave * 32 + (lane & 31)) * kTileK + (lane >> 5) * 8) * 2);
  // B: the 16 bytes of columns 4 (tid % 32) .. + 3 in the k rows tid / 32 + 8 i
  const int q4 = tid & 31, kr = tid >> 5;
  const int64_t jc = j0 + 4 * q4;
  const bool col_ok = jc < a.ncols;
  uint32_t b_off = 0;
  if (col_ok) {
    const int64_t s = jc / L;
    b_off = (uint32_t)(((s * K) * (int64_t)L + (jc - s * L)) * 4);
  }
  const uint32_t row_bytes = (uint32_t)L * 4u;
  const bool edge_cols = __builtin_amdgcn_readfirstlane(j0 + kTile > a.ncols ? 1 : 0) != 0;
  const char *b_base = reinterpret_cast<const char *>(a.b);
  float b_scale = 1.0f, b_inverse = 1.0f;
  const bool per_sample = TB > 1 && a.b_amax_samples != nullptr;
  if (TB > 1 && !per_sample && a.b_amax != nullptr) scale_for(tensor_amax(a.b_amax), b_scale, b_inverse);
  const bool two_samples = L >= kTile;
  const int64_t tile_sample = j0 / L, next_sample_col = (tile_sample + 1) * L;
  float tile_amax[2] = {0.0f, 0.0f};
  if (per_sample && two_samples) {
    const int64_t s_a = a.amax_s0 + tile_sample, s_b = s_a + 1 < a.amax_S ? s_a + 1 : s_a;
    tile_amax[0] = sample_amax(a.b_amax_samples, s_a);
    tile_amax[1] = sample_amax(a.b_amax_samples, s_b);
  }
  auto column_amax = [&](int64_t j) {
    return two_samples ? (j < next_sample_col ? tile_amax[0] : tile_amax[1]) : sample_amax(a.b_amax_samples, a.amax_s0 + j / L);
  };
  if (per_sample && col_ok) scale_for(column_amax(jc), b_scale, b_inverse);

  u32x4 af[2][TA];  // [ks][term]: the fragments of the step being multiplied, refilled as they are used up
  u32x4 rb[2][4];   // [set][i]: k row kr + 8 i of a tile, fp32 bit patterns of four columns
  auto fetch_a = [&](int tile, int ks) {  // every request is unconditional: k steps beyond the last repeat it
    const int t_ = tile < steps ? tile : steps - 1;
    const char *src = a_base + (int64_t)t_ * (kTile * kTileK * 2) + ks * 32;
#pragma unroll
    for (int ta = 0; ta < TA; ++ta) af[ks][ta] = *reinterpret_cast<const u32x4 *>(src + (int64_t)ta * a.plane_stride * 2 + a_lane);
  };
  auto fetch_b = [&](int tile, int set) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = tile * kTileK + kr + 8 * i;
      rb[set][i] = *reinterpret_cast<const u32x4 *>(b_base + (b_off + (uint32_t)(k < K ? k : K - 1) * row_bytes));
    }
  };
  auto stage = [&](int tile, int set) {
    uint8_t *Bs = lds + (tile & 1) * kBuf;
    if (edge_cols || (tile + 1) * kTileK > K) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (!(col_ok && tile * kTileK + kr + 8 * i < K)) rb[set][i] = (u32x4)(0u);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // (the components go through scalars first: a bit cast applied to a vector component directly reads component 0)
      const uint32_t u0 = rb[set][i].x, u1 = rb[set][i].y, u2 = rb[set][i].z, u3 = rb[set][i].w;
      float x0 = __builtin_bit_cast(float, u0), x1 = __builtin_bit_cast(float, u1);
      float x2 = __builtin_bit_cast(float, u2), x3 = __builtin_bit_cast(float, u3);
      uint32_t w01[TB], w23[TB];
      split_scaled_pair<TB, true>(x0, x1, b_scale, w01);
      split_scaled_pair<TB, true>(x2, x3, b_scale, w23);
#pragma unroll
      for (int tb = 0; tb < TB; ++tb) {
        u32x2 v;
        v.x = w01[tb]; v.y = w23[tb];
        *reinterpret_cast<u32x2 *>(Bs + tb * kRowPlane + (kr + 8 * i) * kPlanePitch + q4 * 8) = v;
      }
    }
  };

  f32x16 acc[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int q = 0; q < 16; ++q) acc[nt][q] = 0.0f;
  // the transposing read: group g = lane / 16 fetches columns 16 (g % 2) + 0..15 of the 32, k rows 8 (g / 2) + 0..3 (and
  // + 4 in the second read) of the 16; lane i of the group points at columns 4 (i % 4) + 0..3 of row i / 4
  const int tr_g = lane >> 4, tr_i = lane & 15;
  const uint32_t tr_off = (uint32_t)((8 * (tr_g >> 1) + (tr_i >> 2)) * kPlanePitch + (16 * (tr_g & 1) + 4 * (tr_i & 3)) * 2);
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  auto multiply = [&](int tile, int next_a) {
    const uint8_t *Bs = lds + (tile & 1) * kBuf + tr_off;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4 bf[4][TB];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
          const uint8_t *src = Bs + tb * kRowPlane + ks * 16 * kPlanePitch + nt * 64;
          const u32x2 k03 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(src)));
          const u32x2 k47 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(src + 4 * kPlanePitch)));
          bf[nt][tb].x = k03.x; bf[nt][tb].y = k03.y; bf[nt][tb].z = k47.x; bf[nt][tb].w = k47.y;
        }
      // smallest terms first, as mfma_step
#pragma unroll
      for (int order = Pairs<TA, TB>::kMax; order >= 0; --order) {
#pragma unroll
        for (int ta = 0; ta < TA; ++ta) {
          const int tb = order - ta;
          if (tb < 0 || tb >= TB) continue;
#pragma unroll
          for (int nt = 0; nt < 4; ++nt)
            acc[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, af[ks][ta]),
                                                              __builtin_bit_cast(f16x8, bf[nt][tb]), acc[nt], 0, 0, 0);
        }
      }
      fetch_a(next_a, ks);
      __builtin_amdgcn_sched_barrier(0);  // (the requests stay here: left alone, the compiler moves them to the end of the step)
    }
  };

  fetch_b(0, 0);
  fetch_a(0, 0);
  fetch_a(0, 1);
  fetch_b(1, 1);
  stage(0, 0);
  if (tid < kTile) inverse_lds[tid] = inverse_mine;
  fetch_b(2, 0);
  __syncthreads();
  // step i: tile i + 1 (requested two steps ago) goes into the other LDS buffer, tile i + 3 is requested into the registers
  // that frees, tile i is multiplied while the A fragments of tile i + 1 replace the ones used up
  int i = 0;
  for (; i + 1 < steps; i += 2) {
    stage(i + 1, 1);
    fetch_b(i + 3, 1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(i, i + 1);
    __syncthreads();
    if (i + 2 < steps) stage(i + 2, 0);
    fetch_b(i + 4, 0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(i + 1, i + 2);
    __syncthreads();
  }
  if (i < steps) {
    multiply(i, i);
    __syncthreads();
  }

  // accumulator register q of a 32 x 32 tile: row 8 (q / 4) + 4 (lane / 32) + q % 4, column lane % 32
  float b_inv_col[4] = {b_inverse, b_inverse, b_inverse, b_inverse};
  if (per_sample) {
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      const int64_t j = j0 + nt * 32 + (lane & 31);
      float unused;
      b_inv_col[nt] = 1.0f;
      if (j < a.ncols) scale_for(column_amax(j), unused, b_inv_col[nt]);
    }
  }
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 inv4 = *reinterpret_cast<const f32x4 *>(inverse_lds + wave * 32 + 8 * g + 4 * (lane >> 5));
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float inv = e == 0 ? inv4.x : (e == 1 ? inv4.y : (e == 2 ? inv4.z : inv4.w));
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) acc[nt][4 * g + e] = acc[nt][4 * g + e] * inv * b_inv_col[nt];
    }
  }
  // The tile leaves through LDS (the operand tiles are no longer read: the barrier above) in pieces of 32 rows x 64
  // columns per wavefront, as in pw_gemm_kernel: a store instruction writes four rows of 256 contiguous bytes, and lane i
  // adds row i of the staged piece for the batch-norm sums, in the same order.
  float *buf = reinterpret_cast<float *>(lds) + wave * (32 * kOutPitch);
  const int c4 = 4 * (lane & 15), rsub = lane >> 4;
  const int wave_row0 = mb * kTile + wave * 32;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int64_t j4 = j0 + half * 64 + c4;
    const bool ok4 = j4 < a.ncols;
    const int64_t s4 = ok4 ? j4 / L : 0;
    float *cp4 = a.c + (s4 * M) * (int64_t)L + (ok4 ? (int)(j4 - s4 * L) : 0);
    __builtin_amdgcn_wave_barrier();  // the piece staged before has been read (LDS serves a wavefront's accesses in order)
#pragma unroll
    for (int ntl = 0; ntl < 2; ++ntl)
#pragma unroll
      for (int q = 0; q < 16; ++q)
        buf[(8 * (q >> 2) + 4 * (lane >> 5) + (q & 3)) * kOutPitch + ntl * 32 + (lane & 31)] = acc[2 * half + ntl][q];
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int row_local = 4 * q + rsub;
      const int row = wave_row0 + row_local;
      const f32x4 v = *reinterpret_cast<const f32x4 *>(buf + row_local * kOutPitch + c4);
      if (ok4 && row < M) *reinterpret_cast<f32x4 *>(cp4 + (int64_t)row * L) = v;
    }
    if (a.stats && lane < 32) {
      const float *rowp = buf + lane * kOutPitch;
      float sum = 0.0f, squares = 0.0f;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(rowp + 4 * j);
        sum += (v.x + v.y) + (v.z + v.w);
        squares = fmaf(v.x, v.x, squares); squares = fmaf(v.y, v.y, squares);
        squares = fmaf(v.z, v.z, squares); squares = fmaf(v.w, v.w, squares);
      }
      const int row = wave_row0 + lane;
      if (row < M) {
        float *out = a.stats + ((2 * nb + half) * (int64_t)M + row) * 2;
        out[0] = sum;
        out[1] = squares;
      }
    }
  }
}

struct PwDwArgs {
  const float *dy;   // [S][M][L]
  const float *x;    // [S][N][L]
  float *partials;   // [chunks][M][N]
  int64_t S;
  int M, N, L;
  int s_per_chunk;
  int flat;  // the K steps run over the positions of all samples of a chunk in a row (see pw_dw_kernel)
  int m_blocks, n_blocks;
  const float *dy_amax, *x_amax;  // fp16 terms: nullptr (no scale), or the words whose maximum is the tensor's max |.|
};

// BITS: x is a spike tensor that arrives bit-packed (as in pw_gemm_kernel); a work-item fetches the byte whose low or
// high half holds its four consecutive positions of a row (L and N * L are multiples of 4 and 8).
template <int TA, int TB, bool H, bool BITS = false>
__global__ void __launch_bounds__(kPwThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) pw_dw_kernel(const PwDwArgs a) {
  static_assert(!BITS || TB == 1, "a bit-packed operand has one term");
  extern __shared__ __align__(16) uint8_t lds[];
  uint8_t *As = lds;                   // [TA][128][kRowBytes]
  uint8_t *Bs = lds + TA * kRowPlane;  // [TB][128][kRowBytes]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t logical = xcd_order(blockIdx.x, gridDim.x);
  const int tiles = a.m_blocks * a.n_blocks;
  const int chunk = (int)(logical / tiles);
  const int tile = (int)(logical % tiles);
  const int mb = tile % a.m_blocks, nb = tile / a.m_blocks;
  const int m0 = mb * kTile, n0 = nb * kTile;
  const int M = a.M, N = a.N, L = a.L;
  const int64_t s_begin = (int64_t)chunk * a.s_per_chunk;
  const int64_t s_end = s_begin + a.s_per_chunk < a.S ? s_begin + a.s_per_chunk : a.S;
  const int l_steps = (L + kTileK - 1) / kTileK;
  // flat: the contraction index runs over the quads (four positions) of all samples of the chunk in a row, so a K step of
  // eight quads may take the last quads of one sample and the first of the next, and only the last step of a chunk is
  // partly empty (a row of 196 positions is 6.125 steps instead of 7).  Needs at least eight quads per sample (a step
  // then touches two samples at most) and samples of less than 2^31 bytes (a lane's offset reaches into the second).
  const bool flat = a.flat != 0;
  const int Q = L >> 2;
  const int n_samples = (int)(s_end - s_begin);
  const int64_t total_quads = (int64_t)n_samples * Q;
  const int64_t iters = flat ? (total_quads + 7) / 8 : (int64_t)n_samples * l_steps;
  const uint32_t a_sample = (uint32_t)(M * L * 4), b_sample = (uint32_t)(N * L * (BITS ? 1 : 4));  // bytes; with BITS bits
  int f_s = 0, f_q = 0;  // flat: sample and quad at which the next step to be fetched begins
  int g_s = 0, g_q = 0;  // flat: the same for the next step to be staged

  // a thread fetches quad q4 (four consecutive l) of rows rr, rr + 32, rr + 64, rr + 96 of both operand tiles; addresses
  // are a uniform base (the sample) plus 32-bit per-lane offsets (row; position), loads are unconditional from clamped
  // offsets and the outside of the matrices is zeroed when the tile is staged
  const int q4 = tid & 7, rr = tid >> 3;
  uint32_t a_off[4], b_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = rr + 32 * i;
    a_off[i] = (uint32_t)((m0 + row < M ? m0 + row : M - 1) * L * 4);
    b_off[i] = (uint32_t)((n0 + row < N ? n0 + row : N - 1) * L * (BITS ? 1 : 4));  // bytes; with BITS bits
  }
  const bool edge_rows = __builtin_amdgcn_readfirstlane((m0 + kTile > M || n0 + kTile > N) ? 1 : 0) != 0;
  const char *dy_base = reinterpret_cast<const char *>(a.dy);
  const char *x_base = reinterpret_cast<const char *>(a.x);
  float a_scale = 1.0f, a_inverse = 1.0f, b_scale = 1.0f, b_inverse = 1.0f;
  if (H && TA > 1 && a.dy_amax != nullptr) scale_for(tensor_amax(a.dy_amax), a_scale, a_inverse);
  if (H && TB > 1 && a.x_amax != nullptr) scale_for(tensor_amax(a.x_amax), b_scale, b_inverse);
  f32x4 ra[2][4], rb[2][4];  // two tiles in flight, as in pw_gemm_kernel
  auto fetch = [&](int64_t it, int set) {  // (called for it = 0, 1, 2, ... in this order)
    int64_t s;
    uint32_t l_off, sa = 0, sb = 0;
    if (flat) {
      int q = f_q + q4;
      const bool second = q >= Q;
      if (second) q -= Q;
      const bool ok = f_s + (second ? 1 : 0) < n_samples;
      s = s_begin + f_s;
      l_off = ok ? (uint32_t)q * 16u : 0u;
      if (ok && second) {
        sa = a_sample;
        sb = b_sample;
      }
      f_q += 8;
      if (f_q >= Q) {
        f_q -= Q;
        ++f_s;
      }
    } else {
      s = s_begin + it / l_steps;
      const int l = (int)(it % l_steps) * kTileK + 4 * q4;
      l_off = (uint32_t)((l < L ? l : L - 4) * 4);
    }
    const char *pa = dy_base + (s * M) * (int64_t)L * 4;
    const char *pb = x_base + (BITS ? ((s * N) * (int64_t)L >> 3) : (s * N) * (int64_t)L * 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[set][i] = *reinterpret_cast<const f32x4 *>(pa + (a_off[i] + sa + l_off));
      if (BITS) {
        const uint32_t e = b_off[i] + sb + (l_off >> 2);
        rb[set][i].x = __builtin_bit_cast(float, (uint32_t)*reinterpret_cast<const uint8_t *>(pb + (e >> 3)));
      } else {
        rb[set][i] = *reinterpret_cast<const f32x4 *>(pb + (b_off[i] + sb + l_off));
      }
    }
  };
  auto stage = [&](int64_t it, int set) {  // (called for it = 0, 1, 2, ... in this order)
    bool l_ok, tail;
    int lq;  // the position of the work-item's quad in its row (for the bit offset)
    if (flat) {
      int q = g_q + q4;
      const bool second = q >= Q;
      if (second) q -= Q;
      l_ok = g_s + (second ? 1 : 0) < n_samples;
      lq = l_ok ? 4 * q : 0;
      tail = (int64_t)g_s * Q + g_q + 8 > total_quads;
      g_q += 8;
      if (g_q >= Q) {
        g_q -= Q;
        ++g_s;
      }
    } else {
      const int l0 = (int)(it % l_steps) * kTileK;
      l_ok = l0 + 4 * q4 < L;
      lq = l_ok ? l0 + 4 * q4 : L - 4;
      tail = l0 + kTileK > L;
    }
    if (edge_rows || tail) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (!(l_ok && m0 + rr + 32 * i < M)) ra[set][i] = (f32x4)(0.0f);
        if (!(l_ok && n0 + rr + 32 * i < N)) rb[set][i] = (f32x4)(0.0f);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int off = (rr + 32 * i) * kRowBytes + q4 * 8;
      {
        uint32_t w01[TA], w23[TA];
        const f32x4 v = ra[set][i];
        split_scaled_pair<TA, H>(v.x, v.y, a_scale, w01);
        split_scaled_pair<TA, H>(v.z, v.w, a_scale, w23);
#pragma unroll
        for (int t = 0; t < TA; ++t) {
          u32x2 w;
          w.x = w01[t];
          w.y = w23[t];
          *reinterpret_cast<u32x2 *>(As + t * kRowPlane + off) = w;
        }
      }
      {
        uint32_t w01[TB], w23[TB];
        f32x4 v = rb[set][i];
        if (BITS) {  // (a whole sample is a multiple of 8 bits: the shift does not depend on the sample)
          const uint32_t e = b_off[i] + (uint32_t)lq;
          const uint32_t four = __builtin_bit_cast(uint32_t, rb[set][i].x) >> (e & 7u);
          v.x = (float)(four & 1u);
          v.y = (float)((four >> 1) & 1u);
          v.z = (float)((four >> 2) & 1u);
          v.w = (float)((four >> 3) & 1u);
        }
        split_scaled_pair<TB, H>(v.x, v.y, b_scale, w01);
        split_scaled_pair<TB, H>(v.z, v.w, b_scale, w23);
#pragma unroll
        for (int t = 0; t < TB; ++t) {
          u32x2 w;
          w.x = w01[t];
          w.y = w23[t];
          *reinterpret_cast<u32x2 *>(Bs + t * kRowPlane + off) = w;
        }
      }
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;

  auto multiply = [&](int64_t it) {
    // the second half of the last stage of a row (flat: of the chunk) may hold nothing
    const int ksteps = flat ? ((it + 1 == iters && total_quads - 8 * it <= 4) ? 1 : 2)
                            : (((int)(it % l_steps) * kTileK + 16 < L) ? 2 : 1);
    for (int ks = 0; ks < ksteps; ++ks) {
      u32x4 af[2][TA], bf[2][TB];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int t = 0; t < TA; ++t) af[mt][t] = row_fragment(As + t * kRowPlane, wm * 64 + mt * 32 + (lane & 31), ks, lane);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int t = 0; t < TB; ++t) bf[nt][t] = row_fragment(Bs + t * kRowPlane, wn * 64 + nt * 32 + (lane & 31), ks, lane);
      mfma_step<TA, TB, H>(af, bf, acc);
    }
  };
  // as in pw_gemm_kernel: unconditional requests in the steady state, conditions only in the last steps
  auto step = [&](int64_t it, int set, bool more) {
    __syncthreads();
    stage(it, set);
    __syncthreads();
    if (more) fetch(it + 2, set);
    multiply(it);
  };
  if (iters > 0) fetch(0, 0);
  if (iters > 1) fetch(1, 1);
  int64_t it = 0;
  for (; it + 3 < iters; it += 2) {
    step(it, 0, true);
    step(it + 1, 1, true);
  }
  if (it < iters) step(it, 0, it + 2 < iters);
  if (it + 1 < iters) step(it + 1, 1, false);
  if (it + 2 < iters) step(it + 2, 0, false);

  float *out = a.partials + (int64_t)chunk * M * N;
  if (H) {
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mt][nt][r] = acc[mt][nt][r] * a_inverse * b_inverse;
  }
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const int col = n0 + wn * 64 + nt * 32 + (lane & 31);
    if (col >= N) continue;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      const int rbase = m0 + wm * 64 + mt * 32 + 4 * (lane >> 5);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = rbase + 8 * (r >> 2) + (r & 3);
        if (row < M) out[(int64_t)row * N + col] = acc[mt][nt][r];
      }
    }
  }
}


struct PwDwPlanesArgs {
  const uint16_t *dy_planes;  // [2][M][ld] fp16 terms of dy, column s * L + l of row m holds dy[s][m][l]
  const uint16_t *x_planes;   // [TB][N][ld], likewise
  float *partials;            // [chunks][M][N]
  int64_t dy_plane_stride, x_plane_stride;  // M * ld, N * ld
  int64_t ncols;              // S * L
  int ld;
  int M, N;
  int64_t steps_per_chunk;    // K steps (32 columns each) per partial tile
  int m_blocks, n_blocks;
  const float *dy_amax, *x_amax;
};

// The weight gradient from term planes: dW[m][n] = sum_j dy[m][j] x[n][j] with both operands contiguous along the
// contraction index j (the columns of all samples in a row), so a tile of either is copied to LDS as it lies in memory,
// 16 bytes per work-item and row, and read back as fragments; no arithmetic on the way, and no sample boundaries.
template <int TB>
__global__ void __launch_bounds__(kPwThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) pw_dw_planes_kernel(const PwDwPlanesArgs a) {
  constexpr int TA = 2;
  extern __shared__ __align__(16) uint8_t lds[];
  uint8_t *As = lds;                   // [TA][128][kRowBytes]
  uint8_t *Bs = lds + TA * kRowPlane;  // [TB][128][kRowBytes]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t logical = xcd_order(blockIdx.x, gridDim.x);
  const int tiles = a.m_blocks * a.n_blocks;
  const int chunk = (int)(logical / tiles);
  const int tile = (int)(logical % tiles);
  const int mb = tile % a.m_blocks, nb = tile / a.m_blocks;
  const int m0 = mb * kTile, n0 = nb * kTile;
  const int M = a.M, N = a.N;
  const int64_t steps_total = (a.ncols + kTileK - 1) / kTileK;
  const int64_t it_begin = (int64_t)chunk * a.steps_per_chunk;
  const int64_t it_end = it_begin + a.steps_per_chunk < steps_total ? it_begin + a.steps_per_chunk : steps_total;
  const int64_t iters = it_end - it_begin;

  // a work-item copies the 16-byte chunks q = tid and tid + 256 of a tile: row q / 4, eight columns 8 (q % 4)
  const uint32_t ld2 = (uint32_t)a.ld * 2u;
  uint32_t a_off[2], b_off[2];
  int dst[2];
  const int kc = tid & 3;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = (tid >> 2) + 64 * i;
    a_off[i] = (uint32_t)(m0 + row < M ? m0 + row : M - 1) * ld2;
    b_off[i] = (uint32_t)(n0 + row < N ? n0 + row : N - 1) * ld2;
    dst[i] = row * kRowBytes + kc * 16;
  }
  const bool edge_rows = __builtin_amdgcn_readfirstlane((m0 + kTile > M || n0 + kTile > N) ? 1 : 0) != 0;
  const char *dy_base = reinterpret_cast<const char *>(a.dy_planes);
  const char *x_base = reinterpret_cast<const char *>(a.x_planes);
  float a_scale, a_inverse = 1.0f, b_scale, b_inverse = 1.0f;
  if (a.dy_amax != nullptr) scale_for(tensor_amax(a.dy_amax), a_scale, a_inverse);
  if (TB > 1 && a.x_amax != nullptr) scale_for(tensor_amax(a.x_amax), b_scale, b_inverse);
  u32x4 ra[2][TA][2], rb[2][TB][2];  // two tiles in flight
  auto fetch = [&](int64_t it, int set) {
    const int64_t j = (it_begin + it) * kTileK;  // first column of the step; a chunk beyond the row is fetched from its start
    const uint32_t col = (j + 8 * kc < a.ld) ? (uint32_t)kc * 16u : 0u;
    const char *pa = dy_base + j * 2, *pb = x_base + j * 2;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int t = 0; t < TA; ++t) ra[set][t][i] = *reinterpret_cast<const u32x4 *>(pa + (int64_t)t * a.dy_plane_stride * 2 + (a_off[i] + col));
#pragma unroll
      for (int t = 0; t < TB; ++t) rb[set][t][i] = *reinterpret_cast<const u32x4 *>(pb + (int64_t)t * a.x_plane_stride * 2 + (b_off[i] + col));
    }
  };
  auto stage = [&](int64_t it, int set) {
    const int64_t j = (it_begin + it) * kTileK;
    const bool tail = j + kTileK > a.ncols;
    if (edge_rows || tail) {  // rows beyond the matrices and columns beyond the last sample hold zeros
      const int64_t left = a.ncols - (j + 8 * kc);
      const int nvalid = left < 0 ? 0 : (left > 8 ? 8 : (int)left);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = (tid >> 2) + 64 * i;
        const int na = m0 + row < M ? nvalid : 0, nb_ = n0 + row < N ? nvalid : 0;
#pragma unroll
        for (int t = 0; t < TA; ++t) {
          u32x4 &v = ra[set][t][i];
          v.x &= na >= 2 ? 0xffffffffu : (na == 1 ? 0xffffu : 0u);
          v.y &= na >= 4 ? 0xffffffffu : (na == 3 ? 0xffffu : 0u);
          v.z &= na >= 6 ? 0xffffffffu : (na == 5 ? 0xffffu : 0u);
          v.w &= na >= 8 ? 0xffffffffu : (na == 7 ? 0xffffu : 0u);
        }
#pragma unroll
        for (int t = 0; t < TB; ++t) {
          u32x4 &v = rb[set][t][i];
          v.x &= nb_ >= 2 ? 0xffffffffu : (nb_ == 1 ? 0xffffu : 0u);
          v.y &= nb_ >= 4 ? 0xffffffffu : (nb_ == 3 ? 0xffffu : 0u);
          v.z &= nb_ >= 6 ? 0xffffffffu : (nb_ == 5 ? 0xffffu : 0u);
          v.w &= nb_ >= 8 ? 0xffffffffu : (nb_ == 7 ? 0xffffu : 0u);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int t = 0; t < TA; ++t) *reinterpret_cast<u32x4 *>(As + t * kRowPlane + dst[i]) = ra[set][t][i];
#pragma unroll
      for (int t = 0; t < TB; ++t) *reinterpret_cast<u32x4 *>(Bs + t * kRowPlane + dst[i]) = rb[set][t][i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.0f;

  auto multiply = [&](int64_t it) {
    // the second half of the last step of the matrix may hold nothing
    const int ksteps = (a.ncols - (it_begin + it) * kTileK <= 16) ? 1 : 2;
    for (int ks = 0; ks < ksteps; ++ks) {
      u32x4 af[2][TA], bf[2][TB];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int t = 0; t < TA; ++t) af[mt][t] = row_fragment(As + t * kRowPlane, wm * 64 + mt * 32 + (lane & 31), ks, lane);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int t = 0; t < TB; ++t) bf[nt][t] = row_fragment(Bs + t * kRowPlane, wn * 64 + nt * 32 + (lane & 31), ks, lane);
      mfma_step<TA, TB, true>(af, bf, acc);
    }
  };
  // as in pw_gemm_kernel: unconditional requests in the steady state, conditions only in the last steps
  auto step = [&](int64_t it, int set, bool more) {
    __syncthreads();
    stage(it, set);
    __syncthreads();
    if (more) fetch(it + 2, set);
    multiply(it);
  };
  if (iters > 0) fetch(0, 0);
  if (iters > 1) fetch(1, 1);
  int64_t it = 0;
  for (; it + 3 < iters; it += 2) {
    step(it, 0, true);
    step(it + 1, 1, true);
  }
  if (it < iters) step(it, 0, it + 2 < iters);
  if (it + 1 < iters) step(it + 1, 1, false);
  if (it + 2 < iters) step(it + 2, 0, false);

  float *out = a.partials + (int64_t)chunk * M * N;
  const float inv = a_inverse * b_inverse;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const int col = n0 + wn * 64 + nt * 32 + (lane & 31);
    if (col >= N) continue;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
      const int rbase = m0 + wm * 64 + mt * 32 + 4 * (lane >> 5);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = rbase + 8 * (r >> 2) + (r & 3);
        if (row < M) out[(int64_t)row * N + col] = acc[mt][nt][r] * inv;
      }
    }
  }
}

// planes[t][c][s * L + l] = term t of scale * x[s][c][l] for x [S][C][L] fp32: two fp16 terms (TERMS == 2: the scale is the
// power of two that the words of amax give, as in the kernels that split on the fly) or one (TERMS == 1: values that
// fp16 holds exactly, no scale).  A work-item takes four consecutive l.
template <int TERMS>
__global__ void __launch_bounds__(256) split_planes_kernel(const float *x, int64_t quads, int C, int L, const float *amax,
                                                            uint16_t *planes, int64_t plane_stride, int ld) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  float scale = 1.0f, inverse = 1.0f;
  if (TERMS > 1 && amax != nullptr) scale_for(tensor_amax(amax), scale, inverse);
  if (i >= quads) return;
  const int qpr = L >> 2;
  const int64_t row = i / qpr;  // s * C + c
  const int l = (int)(i - row * qpr) * 4;
  const int64_t s = row / C;
  const int c = (int)(row - s * C);
  f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(x) + i);
  v *= scale;
  uint32_t w01[TERMS], w23[TERMS];
  split_pair<TERMS, true>(v.x, v.y, w01);
  split_pair<TERMS, true>(v.z, v.w, w23);
  uint16_t *dst = planes + (int64_t)c * ld + s * L + l;
#pragma unroll
  for (int t = 0; t < TERMS; ++t) {
    u32x2 w;
    w.x = w01[t];
    w.y = w23[t];
    *reinterpret_cast<u32x2 *>(dst + (int64_t)t * plane_stride) = w;
  }
}

__global__ void __launch_bounds__(256) dw_reduce_scalar_kernel(const float *partials, int chunks, int64_t count, float *out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float sum = 0.0f;
  for (int c = 0; c < chunks; ++c) sum += partials[(int64_t)c * count + i];
  out[i] = sum;
}

// count a multiple of 4 and 16-byte aligned buffers: four elements per work-item, the chunks in their order, four
// loads in flight
__global__ void __launch_bounds__(256) dw_reduce_kernel(const float *partials, int chunks, int64_t count, float *out) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= count) return;
  f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
  int c = 0;
  for (; c + 4 <= chunks; c += 4) {
    f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(partials + (int64_t)(c + u) * count + i));
#pragma unroll
    for (int u = 0; u < 4; ++u) sum += v[u];
  }
  for (; c < chunks; ++c) sum += __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(partials + (int64_t)c * count + i));
  *reinterpret_cast<f32x4 *>(out + i) = sum;
}

int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

template <int TA, int TB, bool H = false, int BSRC = kBFloat>
int launch_gemm_terms(const PwGemmArgs &a, int64_t blocks, hipStream_t stream) {
  unsigned lds = (TA + TB) * kRowPlane;
  if (a.stats && lds < kStatLds) lds = kStatLds;
  if (a.wide_out && lds < kOutLds) lds = kOutLds;
  hipLaunchKernelGGL((pw_gemm_kernel<TA, TB, H, BSRC>), dim3((unsigned)blocks), dim3(kPwThreads), lds, stream, a);
  return check_launch("pwconv_gemm");
}

template <int TB>
int launch_gemm_rows(const PwGemmArgs &a, int64_t blocks, hipStream_t stream) {
  hipLaunchKernelGGL((pw_gemm_rows_kernel<TB>), dim3((unsigned)blocks), dim3(kPwThreads), rows_inverse_offset(TB) + kTile * 4, stream, a);
  return check_launch("pwconv_gemm");
}

template <int TA, int TB, bool H = false, bool BITS = false>
int launch_dw_terms(const PwDwArgs &a, int64_t blocks, hipStream_t stream) {
  const unsigned lds = (TA + TB) * kRowPlane;
  hipLaunchKernelGGL((pw_dw_kernel<TA, TB, H, BITS>), dim3((unsigned)blocks), dim3(kPwThreads), lds, stream, a);
  return check_launch("pwconv_grad_weight");
}

// Samples per partial tile of dW.  Two blocks are resident per compute unit (512 on the chip); the chunk count is the
// largest that keeps tiles x chunks within one (few tiles) or two full generations of resident blocks, so that no
// generation runs nearly empty.  Measured, kernel + reduction: 27 tiles: 38 chunks (1026 blocks) 312 + 11 us, 37 chunks
// 305 + 11, 19 chunks (513 blocks) 444 + 7, 18 chunks 318 + 7; 9 tiles: 114 chunks 101 + 11, 113 chunks 99 + 11,
// 56 chunks 85 + 7.
int dw_samples_per_chunk(int64_t S, int tiles) {
  const int rounds = tiles >= 16 ? 2 : 1;
  int64_t chunks = (int64_t)rounds * 512 / tiles;
  if (chunks < 1) chunks = 1;
  if (chunks > S) chunks = S;
  return (int)((S + chunks - 1) / chunks);
}

}  // namespace

int64_t pwconv_planes_elems(int64_t rows, int64_t cols) { return 3 * round_up(rows, kTile) * round_up(cols, kTileK); }

int launch_pwconv_split_weight(const float *w, int64_t rows, int64_t cols, int transpose, uint16_t *planes,
                               hipStream_t stream) {
  // planes hold the matrix A of a later GEMM, K-contiguous: A = W ([rows][cols]) or A = W^T ([cols][rows])
  const int64_t ar = transpose ? cols : rows, ac = transpose ? rows : cols;
  const int64_t rows_pad = round_up(ar, kTile), cols_pad = round_up(ac, kTileK);
  const int64_t pairs = rows_pad * (cols_pad / 2);
  const int64_t blocks = (pairs + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_split_weight: %lld x %lld", (long long)rows, (long long)cols);
  hipLaunchKernelGGL(split_weight_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, w, ar, ac,
                     transpose ? (int64_t)1 : cols, transpose ? cols : (int64_t)1, rows_pad, cols_pad, planes);
  return check_launch("pwconv_split_weight");
}

int launch_pwconv_split_weight_f16(const float *w, int64_t rows, int64_t cols, int transpose, uint16_t *planes,
                                   float *amax_reset, int64_t amax_floats, hipStream_t stream) {
  const int64_t ar = transpose ? cols : rows, ac = transpose ? rows : cols;
  const int64_t rows_pad = round_up(ar, kTile), cols_pad = round_up(ac, kTileK);
  const int64_t blocks = rows_pad / 4;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_split_weight_f16: %lld x %lld", (long long)rows, (long long)cols);
  hipLaunchKernelGGL(split_weight_f16_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, w, ar, ac,
                     transpose ? (int64_t)1 : cols, transpose ? cols : (int64_t)1, rows_pad, cols_pad, planes, amax_reset, amax_floats);
  return check_launch("pwconv_split_weight_f16");
}

int launch_pwconv_amax(const float *x, int64_t S, int64_t per_sample, float *amax, hipStream_t stream) {
  const int64_t n = S * per_sample, blocks = (n + kAmaxChunk - 1) / kAmaxChunk;
  if (S > 0x7fffffffLL || blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_amax: %lld samples of %lld elements", (long long)S, (long long)per_sample);
  hipLaunchKernelGGL(amax_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, S, per_sample, reinterpret_cast<unsigned *>(amax));
  return check_launch("pwconv_amax");
}

namespace {
const int64_t kPwOffsetLimit = int64_t(1) << 30;  // per-lane offsets into A and B are 32-bit byte offsets
const int64_t kPwPlaneLimit = int64_t(1) << 30;   // elements of one fp16 plane: 32-bit byte offsets within it
int64_t gemm_samples_per_launch(int64_t K, int64_t L) { return (kPwOffsetLimit - 1) / (K * L); }
}  // namespace

int64_t pwconv_gemm_stats_rows(int64_t K, int64_t S, int64_t L) {
  if (K < 1 || L < 1 || K * L >= kPwOffsetLimit) return 0;
  const int64_t s_step = gemm_samples_per_launch(K, L);
  int64_t rows = 0;
  for (int64_t s0 = 0; s0 < S; s0 += s_step) {
    const int64_t s_count = S - s0 < s_step ? S - s0 : s_step;
    rows += 2 * ((s_count * L + kTile - 1) / kTile);
  }
  return rows;
}

int launch_pwconv_gemm(const uint16_t *a_planes, int a_terms, int64_t M, int64_t K, const float *b, int b_terms,
                       const float *b_amax, int64_t S, int64_t L, float *c, float *stats, hipStream_t stream, bool b_bits) {
  if (L % 2 != 0 || !aligned16(a_planes) || (!b_bits && (reinterpret_cast<uintptr_t>(b) & 7u)))
    return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_gemm: L=%lld must be even, the weight planes 16-byte and the activations 8-byte aligned", (long long)L);
  if (b_bits && ((K * L) % 8 != 0 || a_terms != (SJHIP_PW_F16 | 2) || b_terms != 1))
    return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_gemm: bit-packed activations need K*L=%lld to be a multiple of 8, fp16 weight planes and one activation term", (long long)(K * L));
  const int64_t limit = kPwOffsetLimit;
  if (round_up(M, kTile) * round_up(K, kTileK) >= limit || K * L >= limit)
    return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm: M=%lld K=%lld L=%lld", (long long)M, (long long)K, (long long)L);
  const int64_t s_step = gemm_samples_per_launch(K, L);
  ProfileScope prof(KC_PW_GEMM, stream);
  for (int64_t s0 = 0; s0 < S; s0 += s_step) {
    const int64_t s_count = S - s0 < s_step ? S - s0 : s_step;
    PwGemmArgs a;
    a.a_planes = a_planes; a.c = c + s0 * M * L;
    a.b = b_bits ? reinterpret_cast<const float *>(reinterpret_cast<const uint8_t *>(b) + s0 * K * L / 8) : b + s0 * K * L;
    a.M = (int)M; a.K = (int)K; a.K_pad = (int)round_up(K, kTileK); a.L = (int)L;
    a.plane_stride = round_up(M, kTile) * a.K_pad;
    a.ncols = s_count * L;
    a.m_blocks = (int)(round_up(M, kTile) / kTile);
    a.stats = stats;
    a.a_inverse = reinterpret_cast<const float *>(a_planes + 2 * a.plane_stride);
    a.b_amax = b_amax;
    a.b_amax_samples = b_amax ? b_amax + SJHIP_PW_AMAX_FLOATS : nullptr;
    a.amax_s0 = s0; a.amax_S = S;
    a.b_planes = nullptr; a.b_plane_stride = 0; a.ld = 0;
    a.wide_out = (SJHIP_PW_WIDE_OUT != 0 && L % 4 == 0 && aligned16(c)) ? 1 : 0;
    if (stats) stats += 2 * ((a.ncols + kTile - 1) / kTile) * M * 2;
    const int64_t blocks = a.m_blocks * ((a.ncols + kTile - 1) / kTile);
    if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm: %lld blocks", (long long)blocks);
    int rc;
    // real fp32 activations, positions in fours, everything 16-byte aligned: the kernel that keeps A out of LDS
    const bool rows_kernel = SJHIP_PW_ROWS != 0 && a_terms == (SJHIP_PW_F16 | 2) && !b_bits && L % 4 == 0 && aligned16(b) && aligned16(c);
    if (rows_kernel && (b_terms == 1 || b_terms == 2)) {
      rc = b_terms == 2 ? launch_gemm_rows<2>(a, blocks, stream) : launch_gemm_rows<1>(a, blocks, stream);
      if (rc != SJHIP_OK) return rc;
      continue;
    }
    switch (a_terms * 10 + b_terms) {
      case 33: rc = launch_gemm_terms<3, 3>(a, blocks, stream); break;
      case 31: rc = launch_gemm_terms<3, 1>(a, blocks, stream); break;
      case 22: rc = launch_gemm_terms<2, 2>(a, blocks, stream); break;
      case 21: rc = launch_gemm_terms<2, 1>(a, blocks, stream); break;
      case 11: rc = launch_gemm_terms<1, 1>(a, blocks, stream); break;
      case (SJHIP_PW_F16 | 2) * 10 + 2: rc = launch_gemm_terms<2, 2, true>(a, blocks, stream); break;
      case (SJHIP_PW_F16 | 2) * 10 + 1:
        rc = b_bits ? launch_gemm_terms<2, 1, true, kBBits>(a, blocks, stream) : launch_gemm_terms<2, 1, true>(a, blocks, stream);
        break;
      default: return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_gemm: %d weight terms with %d activation terms (bf16: 3/3, 3/1, 2/2, 2/1, 1/1; fp16: 2/2, 2/1)", a_terms, b_terms);
    }
    if (rc != SJHIP_OK) return rc;
  }
  return SJHIP_OK;
}

int64_t pwconv_dw_workspace_floats(int64_t M, int64_t N, int64_t S) {
  const int tiles = (int)(round_up(M, kTile) / kTile * (round_up(N, kTile) / kTile));
  const int spc = dw_samples_per_chunk(S, tiles);
  return (S + spc - 1) / spc * M * N;
}

int launch_pwconv_grad_weight(const float *dy, int dy_terms, const float *dy_amax, const float *x, int x_terms,
                              const float *x_amax, int64_t S, int64_t M, int64_t N, int64_t L, float *dw, float *workspace,
                              hipStream_t stream, bool x_bits) {
  if (x_bits && ((N * L) % 8 != 0 || dy_terms != (SJHIP_PW_F16 | 2) || x_terms != 1))
    return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_grad_weight: bit-packed activations need N*L=%lld to be a multiple of 8, two fp16 gradient terms and one activation term", (long long)(N * L));
  if (L % 4 != 0 || !aligned16(dy) || (!x_bits && !aligned16(x)))
    return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_grad_weight: L=%lld must be a multiple of 4 and the tensors 16-byte aligned", (long long)L);
  if (M * L >= (int64_t(1) << 30) || N * L >= (int64_t(1) << 30) || M * N >= (int64_t(1) << 40))  // 32-bit per-lane byte offsets
    return fail(SJHIP_ERR_TOO_LARGE, "pwconv_grad_weight: M=%lld N=%lld L=%lld", (long long)M, (long long)N, (long long)L);
  PwDwArgs a;
  a.dy = dy; a.x = x; a.partials = workspace; a.S = S;
  a.dy_amax = dy_amax; a.x_amax = x_amax;
  a.flat = (L >= 32 && M * L < (int64_t(1) << 29) && N * L < (int64_t(1) << 29)) ? 1 : 0;
  a.M = (int)M; a.N = (int)N; a.L = (int)L;
  a.m_blocks = (int)(round_up(M, kTile) / kTile);
  a.n_blocks = (int)(round_up(N, kTile) / kTile);
  const int tiles = a.m_blocks * a.n_blocks;
  a.s_per_chunk = dw_samples_per_chunk(S, tiles);
  const int chunks = (int)((S + a.s_per_chunk - 1) / a.s_per_chunk);
  const int64_t blocks = (int64_t)tiles * chunks;
  int rc;
  {
    ProfileScope prof(KC_PW_GRAD_WEIGHT, stream);
    const int key = dy_terms * 10 + x_terms;
    switch (key) {
      case 33: rc = launch_dw_terms<3, 3>(a, blocks, stream); break;
      case 31: rc = launch_dw_terms<3, 1>(a, blocks, stream); break;
      case 22: rc = launch_dw_terms<2, 2>(a, blocks, stream); break;
      case 21: rc = launch_dw_terms<2, 1>(a, blocks, stream); break;
      case 11: rc = launch_dw_terms<1, 1>(a, blocks, stream); break;
      case (SJHIP_PW_F16 | 2) * 10 + 2: rc = launch_dw_terms<2, 2, true>(a, blocks, stream); break;
      case (SJHIP_PW_F16 | 2) * 10 + 1:
        rc = x_bits ? launch_dw_terms<2, 1, true, true>(a, blocks, stream) : launch_dw_terms<2, 1, true>(a, blocks, stream);
        break;
      default: return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_grad_weight: %d gradient terms with %d activation terms (bf16: 3/3, 3/1, 2/2, 2/1, 1/1; fp16: 2/2, 2/1)", dy_terms, x_terms);
    }
    if (rc != SJHIP_OK) return rc;
    const int64_t count = M * N;
    if (count % 4 == 0 && aligned16(workspace) && aligned16(dw))
      hipLaunchKernelGGL(dw_reduce_kernel, dim3((unsigned)((count / 4 + 255) / 256)), dim3(256), 0, stream, workspace, chunks, count, dw);
    else
      hipLaunchKernelGGL(dw_reduce_scalar_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, workspace, chunks, count, dw);
    rc = check_launch("pwconv_grad_weight(reduce)");
  }
  return rc;
}

// ---- operands that arrive as fp16 term planes -------------------------------------------------------------------------
namespace {
// K steps per partial tile of the weight gradient from planes: as dw_samples_per_chunk, over the steps of 32 columns
int64_t dw_planes_steps_per_chunk(int64_t ncols, int tiles) {
  const int64_t steps = (ncols + kTileK - 1) / kTileK;
  const int rounds = tiles >= 16 ? 2 : 1;
  int64_t chunks = (int64_t)rounds * 512 / tiles;
  if (chunks < 1) chunks = 1;
  if (chunks > steps) chunks = steps > 0 ? steps : 1;
  return (steps + chunks - 1) / chunks;
}
}  // namespace

int64_t pwconv_plane_ld(int64_t S, int64_t L) { return round_up(S * L, 8); }

int launch_pwconv_split_planes(const float *x, int64_t S, int64_t C, int64_t L, int terms, const float *amax, uint16_t *planes,
                               hipStream_t stream) {
  if (S < 1 || C < 1 || L < 1 || L % 4 != 0 || !aligned16(x) || !aligned16(planes) || (terms != 1 && terms != 2))
    return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_split_planes: S=%lld C=%lld L=%lld (a multiple of 4), %d terms (1 or 2), 16-byte aligned buffers", (long long)S, (long long)C, (long long)L, terms);
  if (terms == 2 && (amax == nullptr || !aligned16(amax)))
    return fail(SJHIP_ERR_INVALID, "pwconv_split_planes: two terms need the 16-byte aligned amax buffer of the tensor");
  const int64_t ld = pwconv_plane_ld(S, L);
  if (C > (1 << 24) || L > (1 << 24) || C * ld >= kPwPlaneLimit)
    return fail(SJHIP_ERR_TOO_LARGE, "pwconv_split_planes: S=%lld C=%lld L=%lld", (long long)S, (long long)C, (long long)L);
  const int64_t quads = S * C * (L / 4), blocks = (quads + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_split_planes: %lld elements", (long long)(quads * 4));
  if (terms == 2)
    hipLaunchKernelGGL(split_planes_kernel<2>, dim3((unsigned)blocks), dim3(256), 0, stream, x, quads, (int)C, (int)L, amax, planes, C * ld, (int)ld);
  else
    hipLaunchKernelGGL(split_planes_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, x, quads, (int)C, (int)L, amax, planes, C * ld, (int)ld);
  return check_launch("pwconv_split_planes");
}

int64_t pwconv_gemm_planes_stats_rows(int64_t S, int64_t L) { return 2 * ((S * L + kTile - 1) / kTile); }

int launch_pwconv_gemm_planes(const uint16_t *a_planes, int64_t M, int64_t K, const uint16_t *b_planes, int b_terms,
                              const float *b_amax, int64_t S, int64_t L, float *c, float *stats, hipStream_t stream) {
  if (M < 1 || K < 1 || S < 1 || L < 1 || !aligned16(a_planes) || !aligned16(b_planes) || (b_terms != 1 && b_terms != 2))
    return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_gemm_planes: M=%lld K=%lld S=%lld L=%lld, %d activation terms (1 or 2), 16-byte aligned planes", (long long)M, (long long)K, (long long)S, (long long)L, b_terms);
  if (b_terms == 2 && (b_amax == nullptr || !aligned16(b_amax)))
    return fail(SJHIP_ERR_INVALID, "pwconv_gemm_planes: two activation terms need the 16-byte aligned amax buffer they were scaled by");
  const int64_t ld = pwconv_plane_ld(S, L);
  if (round_up(M, kTile) * round_up(K, kTileK) >= kPwOffsetLimit || K * ld >= kPwPlaneLimit || M * L >= (int64_t(1) << 40))
    return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm_planes: M=%lld K=%lld S=%lld L=%lld", (long long)M, (long long)K, (long long)S, (long long)L);
  PwGemmArgs a;
  a.a_planes = a_planes; a.b = nullptr; a.c = c;
  a.M = (int)M; a.K = (int)K; a.K_pad = (int)round_up(K, kTileK); a.L = (int)L;
  a.plane_stride = round_up(M, kTile) * a.K_pad;
  a.ncols = S * L;
  a.m_blocks = (int)(round_up(M, kTile) / kTile);
  a.stats = stats;
  a.a_inverse = reinterpret_cast<const float *>(a_planes + 2 * a.plane_stride);
  a.b_amax = b_terms == 2 ? b_amax : nullptr;
  a.b_amax_samples = nullptr; a.amax_s0 = 0; a.amax_S = 0;
  a.b_planes = b_planes; a.b_plane_stride = K * ld; a.ld = (int)ld;
  a.wide_out = (SJHIP_PW_WIDE_OUT != 0 && L % 4 == 0 && aligned16(c)) ? 1 : 0;
  const int64_t blocks = a.m_blocks * ((a.ncols + kTile - 1) / kTile);
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm_planes: %lld blocks", (long long)blocks);
  ProfileScope prof(KC_PW_GEMM, stream);
  return b_terms == 2 ? launch_gemm_terms<2, 2, true, kBPlanes>(a, blocks, stream)
                      : launch_gemm_terms<2, 1, true, kBPlanes>(a, blocks, stream);
}

int64_t pwconv_dw_planes_workspace_floats(int64_t M, int64_t N, int64_t S, int64_t L) {
  const int tiles = (int)(round_up(M, kTile) / kTile * (round_up(N, kTile) / kTile));
  const int64_t steps = (S * L + kTileK - 1) / kTileK, spc = dw_planes_steps_per_chunk(S * L, tiles);
  return (steps + spc - 1) / spc * M * N;
}

int launch_pwconv_grad_weight_planes(const uint16_t *dy_planes, const float *dy_amax, const uint16_t *x_planes, int x_terms,
                                     const float *x_amax, int64_t S, int64_t M, int64_t N, int64_t L, float *dw,
                                     float *workspace, hipStream_t stream) {
  if (M < 1 || N < 1 || S < 1 || L < 1 || !aligned16(dy_planes) || !aligned16(x_planes) || (x_terms != 1 && x_terms != 2))
    return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_grad_weight_planes: M=%lld N=%lld S=%lld L=%lld, %d activation terms (1 or 2), 16-byte aligned planes", (long long)M, (long long)N, (long long)S, (long long)L, x_terms);
  if (dy_amax == nullptr || !aligned16(dy_amax) || (x_terms == 2 && (x_amax == nullptr || !aligned16(x_amax))))
    return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight_planes: operands of two terms need the 16-byte aligned amax buffers they were scaled by");
  const int64_t ld = pwconv_plane_ld(S, L);
  if (M * ld >= kPwPlaneLimit || N * ld >= kPwPlaneLimit || M * N >= (int64_t(1) << 40))
    return fail(SJHIP_ERR_TOO_LARGE, "pwconv_grad_weight_planes: M=%lld N=%lld S=%lld L=%lld", (long long)M, (long long)N, (long long)S, (long long)L);
  PwDwPlanesArgs a;
  a.dy_planes = dy_planes; a.x_planes = x_planes; a.partials = workspace;
  a.dy_plane_stride = M * ld; a.x_plane_stride = N * ld; a.ncols = S * L; a.ld = (int)ld;
  a.M = (int)M; a.N = (int)N;
  a.m_blocks = (int)(round_up(M, kTile) / kTile);
  a.n_blocks = (int)(round_up(N, kTile) / kTile);
  a.dy_amax = dy_amax; a.x_amax = x_terms == 2 ? x_amax : nullptr;
  const int tiles = a.m_blocks * a.n_blocks;
  a.steps_per_chunk = dw_planes_steps_per_chunk(a.ncols, tiles);
  const int64_t steps = (a.ncols + kTileK - 1) / kTileK;
  const int chunks = (int)((steps + a.steps_per_chunk - 1) / a.steps_per_chunk);
  const int64_t blocks = (int64_t)tiles * chunks;
  ProfileScope prof(KC_PW_GRAD_WEIGHT, stream);
  const unsigned lds = (2 + x_terms) * kRowPlane;
  if (x_terms == 2) hipLaunchKernelGGL(pw_dw_planes_kernel<2>, dim3((unsigned)blocks), dim3(kPwThreads), lds, stream, a);
  else hipLaunchKernelGGL(pw_dw_planes_kernel<1>, dim3((unsigned)blocks), dim3(kPwThreads), lds, stream, a);
  int rc = check_launch("pwconv_grad_weight_planes");
  if (rc != SJHIP_OK) return rc;
  const int64_t count = M * N;
  if (count % 4 == 0 && aligned16(workspace) && aligned16(dw))
    hipLaunchKernelGGL(dw_reduce_kernel, dim3((unsigned)((count / 4 + 255) / 256)), dim3(256), 0, stream, workspace, chunks, count, dw);
  else
    hipLaunchKernelGGL(dw_reduce_scalar_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream, workspace, chunks, count, dw);
  return check_launch("pwconv_grad_weight_planes(reduce)");
}

}  // namespace sjhip
