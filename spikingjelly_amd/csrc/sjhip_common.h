// Internal helpers shared by the translation units of libsjhip.so: storage-dtype traits,
// 128-bit / element-wise accessors, error text, launch tuning and the optional event profiler.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sjhip.h"

namespace sjhip {

// ----------------------------------------------------------------------------------------------
// Storage dtypes.  fp16 / bf16 travel as raw 16-bit patterns; arithmetic is always fp32.
// ----------------------------------------------------------------------------------------------
struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename S> struct Cvt;

template <> struct Cvt<float> {
  static __host__ __device__ __forceinline__ float round(float f) { return f; }
};

template <> struct Cvt<f16_t> {
  static __host__ __device__ __forceinline__ float to_float(uint16_t b) {
    return (float)__builtin_bit_cast(_Float16, b);
  }
  // round-to-nearest-even, the conversion torch uses for .half()
  static __host__ __device__ __forceinline__ uint16_t from_float(float f) {
    return __builtin_bit_cast(uint16_t, (_Float16)f);
  }
  static __host__ __device__ __forceinline__ float round(float f) { return (float)(_Float16)f; }
};

template <> struct Cvt<bf16_t> {
  static __host__ __device__ __forceinline__ float to_float(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
  }
  // round-to-nearest-even on the upper 16 bits; NaN stays a quiet NaN
  static __host__ __device__ __forceinline__ uint16_t from_float(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
  }
  static __host__ __device__ __forceinline__ float round(float f) { return to_float(from_float(f)); }
};

#ifndef SJHIP_NT_LOAD
#define SJHIP_NT_LOAD 1
#endif
#ifndef SJHIP_NT_STORE
#define SJHIP_NT_STORE 1
#endif

template <typename T> __device__ __forceinline__ T stream_load(const T *p) {
#if SJHIP_NT_LOAD
  return __builtin_nontemporal_load(p);
#else
  return *p;
#endif
}
template <typename T> __device__ __forceinline__ void stream_store(T *p, T v) {
#if SJHIP_NT_STORE
  __builtin_nontemporal_store(v, p);
#else
  *p = v;
#endif
}

// Accessor: how one work-item reads/writes its V consecutive neurons of one row.
// raw_t is what stays in registers between the (early) load and the (late) use.
template <typename S, bool VECTOR> struct Acc;

template <> struct Acc<float, true> {
  static constexpr int V = 4;
  typedef float elem_t;
  typedef f32x4 raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load((const raw_t *)p); }
  static __device__ __forceinline__ raw_t zero() { return (raw_t)(0.f); }
  static __device__ __forceinline__ void unpack(raw_t r, float (&f)[V]) {
    f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w;
  }
  static __device__ __forceinline__ void store(elem_t *p, const float (&f)[V]) {
    raw_t r; r.x = f[0]; r.y = f[1]; r.z = f[2]; r.w = f[3];
    stream_store((raw_t *)p, r);
  }
};
template <> struct Acc<float, false> {
  static constexpr int V = 1;
  typedef float elem_t;
  typedef float raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load(p); }
  static __device__ __forceinline__ raw_t zero() { return 0.f; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&f)[V]) { f[0] = r; }
  static __device__ __forceinline__ void store(elem_t *p, const float (&f)[V]) { stream_store(p, f[0]); }
};
template <typename H> struct Acc16v {
  static constexpr int V = 8;
  typedef uint16_t elem_t;
  typedef u32x4 raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load((const raw_t *)p); }
  static __device__ __forceinline__ raw_t zero() { return (raw_t)(0u); }
  static __device__ __forceinline__ void unpack(raw_t r, float (&f)[V]) {
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = Cvt<H>::to_float((uint16_t)(w[i] & 0xffffu));
      f[2 * i + 1] = Cvt<H>::to_float((uint16_t)(w[i] >> 16));
    }
  }
  static __device__ __forceinline__ void store(elem_t *p, const float (&f)[V]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = (uint32_t)Cvt<H>::from_float(f[2 * i]) | ((uint32_t)Cvt<H>::from_float(f[2 * i + 1]) << 16);
    raw_t r; r.x = w[0]; r.y = w[1]; r.z = w[2]; r.w = w[3];
    stream_store((raw_t *)p, r);
  }
};
template <typename H> struct Acc16s {
  static constexpr int V = 1;
  typedef uint16_t elem_t;
  typedef uint16_t raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load(p); }
  static __device__ __forceinline__ raw_t zero() { return 0; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&f)[V]) { f[0] = Cvt<H>::to_float(r); }
  static __device__ __forceinline__ void store(elem_t *p, const float (&f)[V]) {
    stream_store(p, Cvt<H>::from_float(f[0]));
  }
};
template <> struct Acc<f16_t, true> : Acc16v<f16_t> {};
template <> struct Acc<f16_t, false> : Acc16s<f16_t> {};
template <> struct Acc<bf16_t, true> : Acc16v<bf16_t> {};
template <> struct Acc<bf16_t, false> : Acc16s<bf16_t> {};

// ----------------------------------------------------------------------------------------------
// Host-side services (defined in sjhip_api.hip).
// ----------------------------------------------------------------------------------------------
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int check_launch(const char *what);

struct Tuning {
  int fwd_block;
  int bwd_block;
  int pack_block;
};
const Tuning &tuning();

enum KernelClass { KC_FORWARD = 0, KC_BACKWARD = 1, KC_PLIF_REDUCE = 2, KC_BIT_PACK = 3, KC_BIT_UNPACK = 4, KC_COUNT = 5 };

// Brackets one launch with events when profiling is on; free otherwise.
class ProfileScope {
 public:
  ProfileScope(int kernel_class, hipStream_t stream);
  ~ProfileScope();
 private:
  int kc_;
  hipStream_t stream_;
  hipEvent_t start_;
  bool active_;
};

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Launchers (one per translation unit).
int launch_forward(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                   const void *x_seq, const void *v_init, const float *k_device, void *spike_seq,
                   void *v_seq, void *v_last, void *h_seq, hipStream_t stream);
int launch_backward(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                    const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                    const void *h_seq, const void *v_init,
                    const float *k_device, void *grad_x_seq, void *grad_v_init, float *grad_rtau,
                    float *workspace, hipStream_t stream);
int64_t plif_blocks(int dtype, int64_t N);
int launch_bit_pack(int dtype, int64_t n, const void *src, uint8_t *dst, hipStream_t stream);
int launch_bit_unpack(int dtype, int64_t n, const uint8_t *src, void *dst, hipStream_t stream);

}  // namespace sjhip
