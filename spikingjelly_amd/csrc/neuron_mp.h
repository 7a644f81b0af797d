// Mixed-precision IF / LIF / PLIF with 8-bit floating-point storage.
//
// Reference: the mixed-precision operators of triton_kernel/neuron_kernel/{integrate_and_fire,lif,plif}.py
// (sj::multistep_*_mp_forward / _inference, lif.py:788-956; backward lif.py:1103-1150) with an FP8 storage dtype: x_seq,
// v_init, v_seq and h_seq live in memory as float8_e4m3fn or float8_e5m2, spikes and their gradient in a spike dtype of
// their own (fp32, fp16 or bf16), the recurrence runs in fp32 and only stored values are rounded.  The oracle is the
// reference's own recipe for these operators (test/activation_based/test_triton_neuron.py:212-247): inputs rounded to
// the storage dtype, fp32 arithmetic, outputs rounded to the storage dtype.
//
// One work-item owns 16 neurons (four groups of four, see Tile16): per row four 4-byte accesses to an 8-bit tensor, four
// 8-byte accesses to 16-bit spikes, four 16-byte accesses to an fp32 tensor, each contiguous across the wavefront.  Per neuron-step the forward moves 1 B (x) + spike + 1 B (v_seq) + 1 B (h_seq), a quarter
// of the fp32 kernel's traffic when spikes are 16-bit.  The step arithmetic is neuron_step<float> of the fp32 kernels.
//
// 8-bit conversions must round like torch's `.to(torch.float8_*)` on the CPU: round to nearest even; e4m3fn has no
// infinity and anything that rounds above 448 becomes NaN; e5m2 overflows to infinity like IEEE.  gfx950's packed
// conversion instructions (v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32 and their inverses, OCP formats on this chip, two values
// per instruction) do exactly that in the default (non-saturating) mode and are what the kernels use; the tests compare
// every code, every halfway case, the subnormals and the overflow rule against torch.  encode_f8 below is the same
// conversion in integer arithmetic (about fifteen instructions per value, which made the kernels VALU-bound); it is
// selected with -DSJHIP_F8_SOFTWARE=1.
#pragma once

#include "neuron_bwd.h"
#include "neuron_fwd.h"

#include <initializer_list>

// Rows in flight per work-item in the forward and in the backward.  Measured at T = 16, 2^25 neurons, float8 storage:
// forward 0.514 / 0.527 / 0.537 ms with 2 / 4 / 8 rows, backward 0.83 / 0.81 / 0.87 ms with 1 / 2 / 4.
#ifndef SJHIP_MP_PF
#define SJHIP_MP_PF 2
#endif
#ifndef SJHIP_MP_BWD_PF
#define SJHIP_MP_BWD_PF 2
#endif
#ifndef SJHIP_F8_SOFTWARE
#define SJHIP_F8_SOFTWARE 0
#endif

namespace sjhip {

struct f8e4m3_t { uint8_t bits; };
struct f8e5m2_t { uint8_t bits; };

// EBITS.MBITS minifloat with exponent bias BIAS; FN: no infinities, S.1111.111 is the only NaN
template <int MBITS, int BIAS, bool FN>
__host__ __device__ __forceinline__ uint32_t encode_f8(float f) {
  const uint32_t u = __builtin_bit_cast(uint32_t, f);
  const uint32_t sign = (u >> 24) & 0x80u, mag = u & 0x7fffffffu;
  constexpr int shift = 23 - MBITS;
  constexpr uint32_t min_normal = (uint32_t)(127 + 1 - BIAS) << 23;
  constexpr uint32_t top = FN ? 0x7eu : (0x7bu);        // largest finite code
  constexpr uint32_t over = FN ? 0x7fu : (0x7cu);       // NaN (fn) or infinity
  if (mag >= 0x7f800000u) return sign | ((FN || mag > 0x7f800000u) ? 0x7fu : 0x7cu);
  if (mag < min_normal) {
    // subnormal result: the code is the value in units of the smallest subnormal, rounded to nearest even
    const float units = __builtin_bit_cast(float, mag) * (float)(1u << (BIAS - 1 + MBITS));
    return sign | (uint32_t)__builtin_rintf(units);
  }
  const uint32_t rounded = mag + ((1u << (shift - 1)) - 1u) + ((mag >> shift) & 1u);
  const uint32_t code = (rounded >> shift) - ((uint32_t)(127 - BIAS) << MBITS);
  return sign | (code > top ? over : code);
}

typedef float f32x2 __attribute__((ext_vector_type(2)));

// How the 4 / BYTES elements of one 32-bit word of a tensor of dtype D become floats and back.
template <typename D> struct Codec;
template <> struct Codec<float> {
  static constexpr int BYTES = 4;
  static __device__ __forceinline__ float dec(uint32_t b) { return __builtin_bit_cast(float, b); }
  static __device__ __forceinline__ void dec_word(uint32_t w, float *f) { f[0] = __builtin_bit_cast(float, w); }
  static __device__ __forceinline__ uint32_t enc_word(const float *f) { return __builtin_bit_cast(uint32_t, f[0]); }
};
template <> struct Codec<f16_t> {
  static constexpr int BYTES = 2;
  static __device__ __forceinline__ float dec(uint32_t b) { return Cvt<f16_t>::to_float((uint16_t)b); }
  static __device__ __forceinline__ void dec_word(uint32_t w, float *f) { f[0] = dec(w & 0xffffu); f[1] = dec(w >> 16); }
  static __device__ __forceinline__ uint32_t enc_word(const float *f) {
    return (uint32_t)Cvt<f16_t>::from_float(f[0]) | ((uint32_t)Cvt<f16_t>::from_float(f[1]) << 16);
  }
};
template <> struct Codec<bf16_t> {
  static constexpr int BYTES = 2;
  static __device__ __forceinline__ float dec(uint32_t b) { return Cvt<bf16_t>::to_float((uint16_t)b); }
  static __device__ __forceinline__ void dec_word(uint32_t w, float *f) { f[0] = dec(w & 0xffffu); f[1] = dec(w >> 16); }
  static __device__ __forceinline__ uint32_t enc_word(const float *f) {
    return (uint32_t)Cvt<bf16_t>::from_float(f[0]) | ((uint32_t)Cvt<bf16_t>::from_float(f[1]) << 16);
  }
};
template <> struct Codec<f8e4m3_t> {
  static constexpr int BYTES = 1;
  // S.EEEE.MMM placed in a half as S.0EEEE.MMM0000000 is the same number scaled by 2^-8 (subnormals included)
  static __device__ __forceinline__ float dec(uint32_t b) {
    const uint16_t half = (uint16_t)(((b & 0x80u) << 8) | ((b & 0x7fu) << 7));
    const float f = Cvt<f16_t>::to_float(half) * 256.0f;
    return (b & 0x7fu) == 0x7fu ? __builtin_bit_cast(float, 0x7fc00000u | ((b & 0x80u) << 24)) : f;
  }
  static __device__ __forceinline__ void dec_word(uint32_t w, float *f) {
#if SJHIP_F8_SOFTWARE
    for (int i = 0; i < 4; ++i) f[i] = dec((w >> (8 * i)) & 0xffu);
#else
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    f[0] = lo.x; f[1] = lo.y; f[2] = hi.x; f[3] = hi.y;
#endif
  }
  static __device__ __forceinline__ uint32_t enc_word(const float *f) {
#if SJHIP_F8_SOFTWARE
    return encode_f8<3, 7, true>(f[0]) | (encode_f8<3, 7, true>(f[1]) << 8) | (encode_f8<3, 7, true>(f[2]) << 16) |
           (encode_f8<3, 7, true>(f[3]) << 24);
#else
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w, true);
#endif
  }
};
template <> struct Codec<f8e5m2_t> {
  static constexpr int BYTES = 1;
  // the upper byte of a half
  static __device__ __forceinline__ float dec(uint32_t b) { return Cvt<f16_t>::to_float((uint16_t)(b << 8)); }
  static __device__ __forceinline__ void dec_word(uint32_t w, float *f) {
#if SJHIP_F8_SOFTWARE
    for (int i = 0; i < 4; ++i) f[i] = dec((w >> (8 * i)) & 0xffu);
#else
    const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_bf8((int)w, false), hi = __builtin_amdgcn_cvt_pk_f32_bf8((int)w, true);
    f[0] = lo.x; f[1] = lo.y; f[2] = hi.x; f[3] = hi.y;
#endif
  }
  static __device__ __forceinline__ uint32_t enc_word(const float *f) {
#if SJHIP_F8_SOFTWARE
    return encode_f8<2, 15, false>(f[0]) | (encode_f8<2, 15, false>(f[1]) << 8) | (encode_f8<2, 15, false>(f[2]) << 16) |
           (encode_f8<2, 15, false>(f[3]) << 24);
#else
    int w = __builtin_amdgcn_cvt_pk_bf8_f32(f[0], f[1], 0, false);
    return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(f[2], f[3], w, true);
#endif
  }
};

// A work-item owns 16 neurons as four groups of four: in a wavefront whose first neuron is w0, group g of lane l is
// neurons w0 + 256 g + 4 l .. + 3.  Whatever the element size, one access instruction of the wavefront then covers one
// contiguous run (1 KiB of fp32, 512 B of 16-bit, 256 B of 8-bit values); sixteen consecutive neurons per lane would
// leave the wider tensors with a 32- or 64-byte stride between lanes and four to eight times the cache-line touches.
// `first` is the lane's first neuron (group 0), `groups` how many of its groups lie below N.
struct MpLane {
  int64_t first;
  int groups;
};
__device__ __forceinline__ MpLane mp_lane(int64_t N) {
  const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  MpLane l;
  l.first = wave * 1024 + (int64_t)(threadIdx.x & 63) * 4;
  const int64_t left = N - l.first;
  l.groups = left <= 0 ? 0 : (left > 768 ? 4 : (int)((left + 255) / 256));
  return l;
}

template <int BYTES> struct MpPiece;
template <> struct MpPiece<4> { typedef u32x4 type; };
template <> struct MpPiece<2> { typedef u32x2 type; };
template <> struct MpPiece<1> { typedef uint32_t type; };

template <typename D, bool NT = true> struct Tile16 {
  static constexpr int V = 16;
  static constexpr int BYTES = Codec<D>::BYTES;
  typedef typename MpPiece<BYTES>::type piece_t;  // the four elements of one group
  struct raw_t { piece_t p[4]; };
  static __device__ __forceinline__ const piece_t *at(const void *base, int64_t elem) {
    return (const piece_t *)((const char *)base + elem * BYTES);
  }
  // `row` is the element offset of the row (t * N); groups at or beyond N are neither read nor written
  static __device__ __forceinline__ raw_t load(const void *base, int64_t row, const MpLane &l) {
    raw_t r;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      r.p[g] = piece_t(0);
      if (g < l.groups) r.p[g] = stream_load<NT>(at(base, row + l.first + 256 * g));
    }
    return r;
  }
  static __device__ __forceinline__ raw_t zero() {
    raw_t r;
#pragma unroll
    for (int g = 0; g < 4; ++g) r.p[g] = piece_t(0);
    return r;
  }
  static __device__ __forceinline__ void unpack(const raw_t &r, float (&f)[V]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if constexpr (BYTES == 4) {
        // through a by-value parameter: a bit cast applied directly to a vector element reads element 0 whichever
        // element is named (observed with this compiler)
        f[4 * g] = Codec<D>::dec(r.p[g].x); f[4 * g + 1] = Codec<D>::dec(r.p[g].y);
        f[4 * g + 2] = Codec<D>::dec(r.p[g].z); f[4 * g + 3] = Codec<D>::dec(r.p[g].w);
      } else if constexpr (BYTES == 2) {
        Codec<D>::dec_word(r.p[g].x, &f[4 * g]);
        Codec<D>::dec_word(r.p[g].y, &f[4 * g + 2]);
      } else {
        Codec<D>::dec_word(r.p[g], &f[4 * g]);
      }
    }
  }
  static __device__ __forceinline__ void store(void *base, int64_t row, const MpLane &l, const float (&f)[V]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      piece_t out;
      if constexpr (BYTES == 4) {
        out.x = __builtin_bit_cast(uint32_t, f[4 * g]); out.y = __builtin_bit_cast(uint32_t, f[4 * g + 1]);
        out.z = __builtin_bit_cast(uint32_t, f[4 * g + 2]); out.w = __builtin_bit_cast(uint32_t, f[4 * g + 3]);
      } else if constexpr (BYTES == 2) {
        out.x = Codec<D>::enc_word(&f[4 * g]);
        out.y = Codec<D>::enc_word(&f[4 * g + 2]);
      } else {
        out = Codec<D>::enc_word(&f[4 * g]);
      }
      if (g < l.groups) stream_store<NT>(const_cast<piece_t *>(at(base, row + l.first + 256 * g)), out);
    }
  }
};

// blocks of `block` work-items for N neurons: a wavefront covers 1024 of them
inline int64_t mp_blocks(int64_t N, int block) {
  const int64_t waves = (N + 1023) / 1024;
  return (waves + (block / 64) - 1) / (block / 64);
}

inline bool mp_aligned(std::initializer_list<const void *> ptrs) {
  for (const void *p : ptrs)
    if (p != nullptr && !aligned16(p)) return false;
  return true;
}

}  // namespace sjhip
