// Internal helpers shared by the translation units of libsjhip.so: storage-dtype traits,
// 128-bit / element-wise accessors, error text, launch tuning and the optional event profiler.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cmath>

#include <type_traits>

#include "sjhip.h"

namespace sjhip {

// ----------------------------------------------------------------------------------------------
// Storage dtypes.  fp16 / bf16 travel as raw 16-bit patterns; arithmetic is always fp32.
// ----------------------------------------------------------------------------------------------
struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };
// The same storage dtypes accessed 8 bytes (four neurons) at a time instead of 16: for kernels whose per-neuron
// on-chip state, not the access width, limits the resident wavefronts (the fp32-state replay backward).
struct f16n_t { uint16_t bits; };
struct bf16n_t { uint16_t bits; };

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename S> struct Cvt;

template <> struct Cvt<float> {
  static __host__ __device__ __forceinline__ float round(float f) { return f; }
};

template <> struct Cvt<f16_t> {
  static constexpr uint16_t kOne = 0x3c00;  // 1.0
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
  static constexpr uint16_t kOne = 0x3f80;  // 1.0
  static __host__ __device__ __forceinline__ float to_float(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
  }
  // round-to-nearest-even on the upper 16 bits; NaN stays a quiet NaN.  On the device this is the
  // hardware conversion (v_cvt_pk_bf16_f32), which rounds the same way.
  static __host__ __device__ __forceinline__ uint16_t from_float(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(uint16_t, (__bf16)f);
#endif
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
  }
  static __host__ __device__ __forceinline__ float round(float f) { return to_float(from_float(f)); }
};

template <> struct Cvt<f16n_t> : Cvt<f16_t> {};
template <> struct Cvt<bf16n_t> : Cvt<bf16_t> {};

// (tensor of dtype R) * (Python scalar) as torch's CPU kernels compute it: the fp32 product is rounded to fp32 and then
// to R.  The register barrier keeps the compiler from fusing the multiply and the conversion into one instruction that
// rounds the exact product once (v_fma_mixlo_f16), which differs from the double rounding in about one result of forty.
template <typename R> __device__ __forceinline__ float scalar_product(float scalar, float t) {
#pragma clang fp contract(off)
  float p = scalar * t;
  if constexpr (!std::is_same<R, float>::value) asm volatile("" : "+v"(p));
  return Cvt<R>::round(p);
}

// Cache policy of one access: NT marks the line as streaming (non-temporal), otherwise default.
// Measured on MI355X: read-mostly kernels (backward, unpack) gain from NT on both loads and stores,
// the write-mostly forward loses with it.
template <bool NT, typename T> __device__ __forceinline__ T stream_load(const T *p) {
  if (NT) return __builtin_nontemporal_load(p);
  return *p;
}
template <bool NT, typename T> __device__ __forceinline__ void stream_store(T *p, T v) {
  if (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// Accessor: how one work-item reads/writes its V consecutive neurons of one row.
// raw_t is what stays in registers between the (early) load and the (late) use.
template <typename S, bool VECTOR, bool NT = true> struct Acc;

template <bool NT> struct Acc<float, true, NT> {
  static constexpr int V = 4;
  typedef float elem_t;
  typedef f32x4 raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load<NT>((const raw_t *)p); }
  static __device__ __forceinline__ raw_t zero() { return (raw_t)(0.f); }
  static __device__ __forceinline__ void unpack(raw_t r, float (&f)[V]) {
    f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w;
  }
  static __device__ __forceinline__ void store(elem_t *p, const float (&f)[V]) {
    raw_t r; r.x = f[0]; r.y = f[1]; r.z = f[2]; r.w = f[3];
    stream_store<NT>((raw_t *)p, r);
  }
  // spikes are exactly 0 or 1: in 16-bit storage the bit pattern is selected instead of converted
  static __device__ __forceinline__ void store_spikes(elem_t *p, const float (&f)[V]) { store(p, f); }
};
template <bool NT> struct Acc<float, false, NT> {
  static constexpr int V = 1;
  typedef float elem_t;
  typedef float raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load<NT>(p); }
  static __device__ __forceinline__ raw_t zero() { return 0.f; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&f)[V]) { f[0] = r; }
  static __device__ __forceinline__ void store(elem_t *p, const float (&f)[V]) { stream_store<NT>(p, f[0]); }
  static __device__ __forceinline__ void store_spikes(elem_t *p, const float (&f)[V]) { store(p, f); }
};
template <typename H, bool NT> struct Acc16v {
  static constexpr int V = 8;
  typedef uint16_t elem_t;
  typedef u32x4 raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load<NT>((const raw_t *)p); }
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
    stream_store<NT>((raw_t *)p, r);
  }
  static __device__ __forceinline__ void store_spikes(elem_t *p, const float (&f)[V]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = (f[2 * i] != 0.0f ? (uint32_t)Cvt<H>::kOne : 0u) | (f[2 * i + 1] != 0.0f ? (uint32_t)Cvt<H>::kOne << 16 : 0u);
    raw_t r; r.x = w[0]; r.y = w[1]; r.z = w[2]; r.w = w[3];
    stream_store<NT>((raw_t *)p, r);
  }
  // fp16 values kept as fp16 in registers (native half arithmetic): the stored bits are the register bits
  static __device__ __forceinline__ void unpack(raw_t r, _Float16 (&f)[V]) {
    static_assert(std::is_same<H, f16_t>::value, "native half registers are for fp16 storage only");
    uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0xffffu));
      f[2 * i + 1] = __builtin_bit_cast(_Float16, (uint16_t)(w[i] >> 16));
    }
  }
  static __device__ __forceinline__ void store(elem_t *p, const _Float16 (&f)[V]) {
    static_assert(std::is_same<H, f16_t>::value, "native half registers are for fp16 storage only");
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = (uint32_t)__builtin_bit_cast(uint16_t, f[2 * i]) | ((uint32_t)__builtin_bit_cast(uint16_t, f[2 * i + 1]) << 16);
    raw_t r; r.x = w[0]; r.y = w[1]; r.z = w[2]; r.w = w[3];
    stream_store<NT>((raw_t *)p, r);
  }
  static __device__ __forceinline__ void store_spikes(elem_t *p, const _Float16 (&f)[V]) { store(p, f); }
};
// four 16-bit neurons per 8-byte access (fp32 arithmetic only)
template <typename H, bool NT> struct Acc16n {
  static constexpr int V = 4;
  typedef uint16_t elem_t;
  typedef u32x2 raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load<NT>((const raw_t *)p); }
  static __device__ __forceinline__ raw_t zero() { return (raw_t)(0u); }
  static __device__ __forceinline__ void unpack(raw_t r, float (&f)[V]) {
    f[0] = Cvt<H>::to_float((uint16_t)(r.x & 0xffffu)); f[1] = Cvt<H>::to_float((uint16_t)(r.x >> 16));
    f[2] = Cvt<H>::to_float((uint16_t)(r.y & 0xffffu)); f[3] = Cvt<H>::to_float((uint16_t)(r.y >> 16));
  }
  static __device__ __forceinline__ void store(elem_t *p, const float (&f)[V]) {
    raw_t r;
    r.x = (uint32_t)Cvt<H>::from_float(f[0]) | ((uint32_t)Cvt<H>::from_float(f[1]) << 16);
    r.y = (uint32_t)Cvt<H>::from_float(f[2]) | ((uint32_t)Cvt<H>::from_float(f[3]) << 16);
    stream_store<NT>((raw_t *)p, r);
  }
};
template <typename H, bool NT> struct Acc16s {
  static constexpr int V = 1;
  typedef uint16_t elem_t;
  typedef uint16_t raw_t;
  static __device__ __forceinline__ raw_t load(const elem_t *p) { return stream_load<NT>(p); }
  static __device__ __forceinline__ raw_t zero() { return 0; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&f)[V]) { f[0] = Cvt<H>::to_float(r); }
  static __device__ __forceinline__ void store(elem_t *p, const float (&f)[V]) {
    stream_store<NT>(p, Cvt<H>::from_float(f[0]));
  }
  static __device__ __forceinline__ void store_spikes(elem_t *p, const float (&f)[V]) {
    stream_store<NT>(p, f[0] != 0.0f ? Cvt<H>::kOne : (uint16_t)0);
  }
  static __device__ __forceinline__ void unpack(raw_t r, _Float16 (&f)[V]) {
    static_assert(std::is_same<H, f16_t>::value, "native half registers are for fp16 storage only");
    f[0] = __builtin_bit_cast(_Float16, r);
  }
  static __device__ __forceinline__ void store(elem_t *p, const _Float16 (&f)[V]) {
    static_assert(std::is_same<H, f16_t>::value, "native half registers are for fp16 storage only");
    stream_store<NT>(p, __builtin_bit_cast(uint16_t, f[0]));
  }
  static __device__ __forceinline__ void store_spikes(elem_t *p, const _Float16 (&f)[V]) { store(p, f); }
};
template <bool NT> struct Acc<f16_t, true, NT> : Acc16v<f16_t, NT> {};
template <bool NT> struct Acc<f16_t, false, NT> : Acc16s<f16_t, NT> {};
template <bool NT> struct Acc<bf16_t, true, NT> : Acc16v<bf16_t, NT> {};
template <bool NT> struct Acc<bf16_t, false, NT> : Acc16s<bf16_t, NT> {};
template <bool NT> struct Acc<f16n_t, true, NT> : Acc16n<f16_t, NT> {};
template <bool NT> struct Acc<f16n_t, false, NT> : Acc16s<f16_t, NT> {};
template <bool NT> struct Acc<bf16n_t, true, NT> : Acc16n<bf16_t, NT> {};
template <bool NT> struct Acc<bf16n_t, false, NT> : Acc16s<bf16_t, NT> {};

// Initial state of this work-item's neurons: its V elements of the [N] tensor, or the one stored element
// for every neuron when the caller passed a broadcast state.
template <typename S, bool VECTOR, bool NT, typename NUM, int V>
__device__ __forceinline__ void load_state(const void *p, int64_t col, bool broadcast, NUM (&v)[V]) {
  typedef Acc<S, VECTOR, NT> A;
  static_assert(A::V == V, "state width");
  if (broadcast) {
    typedef Acc<S, false, false> A1;
    NUM one[1];
    A1::unpack(A1::load((const typename A1::elem_t *)p), one);
#pragma unroll
    for (int j = 0; j < V; ++j) v[j] = one[0];
  } else {
    A::unpack(A::load((const typename A::elem_t *)p + col), v);
  }
}

// The same with the source given as the kernels' `v_init_broadcast` field: 0 = [N] in the storage dtype, 1 = one stored
// element for all, kStateF32 = [N] in fp32 (a checkpoint of a state that is kept in fp32 beside 16-bit storage).
constexpr int kStateF32 = 2;
template <typename S, bool VECTOR, bool NT, typename NUM, int V>
__device__ __forceinline__ void load_state_from(const void *p, int64_t col, int source, NUM (&v)[V]) {
  if (source == kStateF32) {
    const float *q = static_cast<const float *>(p) + col;
    if constexpr (VECTOR && V % 4 == 0) {
#pragma unroll
      for (int i = 0; i < V / 4; ++i) {
        const f32x4 w = stream_load<NT>(reinterpret_cast<const f32x4 *>(q) + i);
        v[4 * i] = (NUM)w.x; v[4 * i + 1] = (NUM)w.y; v[4 * i + 2] = (NUM)w.z; v[4 * i + 3] = (NUM)w.w;
      }
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) v[j] = (NUM)q[j];
    }
    return;
  }
  load_state<S, VECTOR, NT>(p, col, source != 0, v);
}

// ----------------------------------------------------------------------------------------------
// Host-side services (defined in sjhip_api.hip).
// ----------------------------------------------------------------------------------------------
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int check_launch(const char *what);

// Largest block the neuron kernels may be launched with.  Kept small on purpose: the kernels run
// best with about one fat wavefront per SIMD (few resident waves, many loads in flight each), and a
// small bound lets the compiler use several hundred VGPRs for the prefetch buffers.  128 work-items are the
// default; 256 are used with the `spread` column order (see column_block()), where a block's longer contiguous run
// per row measured faster.
#ifndef SJHIP_MAX_BLOCK
#define SJHIP_MAX_BLOCK 256
#endif
// work-items per block of the neuron kernels in the `spread` order when the order is chosen automatically
constexpr int kSpreadBlock = 256;

struct Tuning {
  int fwd_block;
  int bwd_block;
  int fwd_blocks_per_cu;  // 0 = no cap; otherwise dynamic LDS is requested so that at most this many
  int bwd_blocks_per_cu;  // blocks are resident per compute unit
  int replay_blocks_per_cu;  // same for the replay backward (its LDS h buffer already bounds residency)
  int column_spread;         // 0, 1, >= 4: a fixed order, 2: by row stride (resonant_row_stride); see column_block()
};
// dynamic LDS bytes that cap residency at `blocks_per_cu` blocks (0 for no cap)
unsigned occupancy_cap_lds(int blocks_per_cu);
const Tuning &tuning();
// the block-to-column order of the neuron kernels for rows of `row_bytes` (see column_block())
inline int column_spread(int64_t row_bytes, int64_t T);

enum KernelClass { KC_FORWARD = 0, KC_BACKWARD = 1, KC_PLIF_REDUCE = 2, KC_BIT_PACK = 3, KC_BIT_UNPACK = 4,
                   KC_SSA_FORWARD = 5, KC_SSA_BACKWARD = 6, KC_PW_GEMM = 7, KC_PW_GRAD_WEIGHT = 8, KC_BN_STATS = 9,
                   KC_BN_LIF_FORWARD = 10, KC_BN_LIF_BACKWARD = 11, KC_BN_GRAD_INPUT = 12, KC_STREAM_PROBE = 13, KC_MFMA_PROBE = 14, KC_COUNT = 15 };

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

// Which columns a block works on.  Blocks are handed to the eight XCDs round-robin (block b runs on XCD b % 8), so
// by default every XCD takes every eighth block-sized chunk of a row.  Measured on [16, 2^25 + K] fp32 (forward plus
// replaying backward, ms): that order is the fastest for almost every row length (2.22 to 2.30 over K = 0 ... 8192 in
// steps of 256 and powers of two up to 2^24) except where the row stride in bytes is a multiple of 4 KiB whose bits 12
// and 20 have odd parity (K = 1024, 3072, 5120, 7168, 262144, 266240: 2.61 to 2.93; K = 263168, both bits set: 2.24).
// Rows of one column then alternate between the two values of an address bit the memory system hashes from bits 12 and
// 20, and an XCD that otherwise stays on one side of it is sent to both.  A plain four-stream copy shows none of this;
// it takes the 32 to 64 concurrent row streams of these kernels.  `spread` gives each XCD one contiguous eighth of the
// columns instead: slower than the default at friendly strides (2.85 against 2.65 on the benchmark step) and
// insensitive to the stride (2.87 at K = 1024 against 3.57); the backward over several pieces uses it.  With 256
// work-items per block (4 KiB of a row per block and step instead of 2) the spread order loses nothing at the strides
// where bit 12 is the odd one (forward + backward kernels, ms: K = 0 default order 2.62; spread with 256: K = 0 2.66,
// K = 1024 2.68, K = 3072 2.70; spread with 128: 2.81 at K = 1024); where bit 20 is the odd one (K = 262 144,
// 266 240) it stays at 3.10 with either block size (3.14 in the default order).
// A third order deals the XCDs runs of kColumnRun consecutive blocks in turn (XCD x takes run x, 8 + x, ...).  At the
// resonant strides it is as good as the contiguous eighths where bit 12 is the odd one and better where bit 20 is
// (forward + backward kernels, ms, K = 262 144: 3.13 eighths, 2.89 runs; K = 266 240: 3.07 and 2.87; K = 1024: 2.70
// and 2.67; K = 0, for comparison: 2.60 in the default order), with 256 work-items per block in the first case and 128
// in the second (forward at K = 262 144: 1.27 ms with 128, 1.39 with 256; at K = 1024: 1.38 and 1.21).  At friendly
// strides the runs are no better than the default order and for some worse (backward at N = 2^25 + 4096: 1.57
// against 1.44 ms), so the default stays.
inline bool resonant_row_stride(int64_t bytes) {
  return (bytes & 4095) == 0 && (((bytes >> 12) ^ (bytes >> 20)) & 1) != 0;
}
inline bool resonant_bit_20(int64_t bytes) { return ((bytes >> 20) & 1) != 0; }
constexpr int kColumnRun = 256;
// The `spread` argument of column_block() for T rows of `row_bytes`: 0 the default order, 1 contiguous eighths, larger
// values runs of that many blocks.  Tuning key "column_spread": 0 and 1 force those orders, 4 and more force runs of
// that many blocks, 2 (default) chooses: contiguous eighths for small tensors whose rows are a multiple of 256 KiB apart
// (at least four rows of at most 256 MiB together), runs of kColumnRun blocks for the resonant strides, the default
// order otherwise.  Measured (forward / backward, us; default order -> eighths): fp32 [16, 2^22] 165 / 214 -> 163 / 177,
// fp32 [16, 2^21] 99 / 109 -> 87 / 90, fp32 [8, 2^23] 167 / 198 -> 161 / 180, bf16 [8, 2^23] 73 / 108 -> 65 / 102, bf16 [4, 2^24]
// 83 / 94 -> 66 / 91, fp16 [32, 49 * 2^17] inference 153 -> 145.  The other way: larger tensors (fp32 [16, 2^23] 292 / 370 ->
// 316 / 369, [16, 2^24] 579 / 702 -> 626 / 739, [4, 2^25] 318 / 352 -> 331 / 369), rows that are not such a multiple apart (fp32
// [16, 147 * 2^15] 182 / 228 -> 228 / 245, [4, 147 * 2^15] 51 / 52 -> 55 / 58) and single rows (fp32 [1, 2^24] 45 -> 53).
inline int column_spread(int64_t row_bytes, int64_t T) {
  const int mode = tuning().column_spread;
  if (mode != 2) return mode;
  if ((row_bytes & ((int64_t(1) << 18) - 1)) == 0 && T >= 4 && T * row_bytes <= (int64_t(256) << 20)) return 1;
  return resonant_row_stride(row_bytes) ? kColumnRun : 0;
}
// work-items per block that go with column_spread() when it chose the order by itself
inline int spread_block(int64_t row_bytes) { return resonant_bit_20(row_bytes) ? 128 : kSpreadBlock; }
#ifdef __HIPCC__
__device__ __forceinline__ unsigned column_block(int spread) {
  const unsigned b = blockIdx.x;
  if (!spread) return b;
  if (spread > 1) {
    const unsigned g = (unsigned)spread, x = b % 8u, i = b / 8u;
    const unsigned full = gridDim.x / (8u * g) * (8u * g);  // blocks beyond the last full round of runs keep their number
    return b < full ? ((i / g) * 8u + x) * g + i % g : b;
  }
  const unsigned per = gridDim.x / 8u;
  return b < per * 8u ? (b % 8u) * per + b / 8u : b;
}
#endif

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// True when x / f == x * (1 / f) bit for bit for every x: f is a power of two far from the ends of the exponent
// range, so both are the same exact scaling and a subnormal result rounds identically.
static inline bool exact_reciprocal(float f) {
  int e;
  return std::isfinite(f) && f > 0.0f && std::frexp(f, &e) == 0.5f && f <= 0x1p100f && f >= 0x1p-100f;
}

// A long sequence handled as consecutive pieces of `chunk` steps inside one launch: the forward leaves the state after
// every piece but the last in `checkpoints` ([pieces - 1][N], storage dtype), the replaying backward starts each piece
// from there and keeps the gradient of a piece's initial state in registers for the piece before it.
struct PieceArgs {
  void *checkpoints;
  int64_t chunk;
  int64_t pieces;
  int checkpoints_f32;  // the checkpoints hold fp32 (16-bit storage whose state is kept in fp32)
};
// whether a checkpoint of the state is an fp32 row rather than one in the storage dtype
inline bool checkpoints_are_f32(int dtype, uint32_t flags) { return dtype != SJHIP_F32 && (flags & SJHIP_FLAG_FP32_STATE) != 0; }

// Launchers (one per translation unit).
int launch_forward(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                   const void *x_seq, const void *v_init, const float *k_device, void *spike_seq,
                   void *v_seq, void *v_last, void *h_seq, hipStream_t stream);
int launch_stbif_forward(int dtype, uint32_t flags, int64_t T, int64_t N, const void *x_seq, const void *q_init,
                         const void *acc_q_init, const float *q_threshold, const float *pos_max, const float *neg_min,
                         void *out_seq, void *q_final, void *acc_q_final, void *cur_output, int32_t *work_flag,
                         hipStream_t stream);
int launch_aaif_forward(int dtype, uint32_t flags, int64_t T, int64_t N, const void *x_seq, const void *v_init,
                        const float *v_threshold, int64_t threshold_count, const float *v_offset, int64_t offset_count,
                        int64_t channel_size, int64_t inner_size, float v_reset, void *spike_seq, void *v_seq,
                        void *v_last, hipStream_t stream);
int launch_izhikevich_forward(int dtype, const sjhip_izhikevich_params &p, int64_t T, int64_t N, const void *x_seq,
                              const void *v_init, const void *w_init, void *spike_seq, void *v_seq, void *w_seq,
                              void *v_last, void *w_last, void *h_seq, hipStream_t stream);
int launch_izhikevich_backward(int dtype, const sjhip_izhikevich_params &p, int64_t T, int64_t N,
                               const void *grad_spike_seq, const void *grad_v_seq, const void *grad_w_seq,
                               const void *grad_v_last, const void *grad_w_last, const void *h_seq, const void *v_init,
                               void *grad_x_seq, void *grad_v_init, void *grad_w_init, hipStream_t stream);
int launch_forward_mp(int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                      const void *x_seq, const void *v_init, const float *k_device, void *spike_seq, void *v_seq,
                      void *v_last, void *h_seq, hipStream_t stream);
int launch_backward_mp(int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                       const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last, const void *h_seq,
                       const void *v_init, const float *k_device, void *grad_x_seq, void *grad_v_init,
                       float *grad_rtau, float *workspace, hipStream_t stream);
int launch_izhikevich_backward_replay(int dtype, const sjhip_izhikevich_params &p, int64_t T, int64_t N,
                                      const void *x_seq, const void *v_init, const void *w_init,
                                      const void *grad_spike_seq, const void *grad_v_seq, const void *grad_w_seq,
                                      const void *grad_v_last, const void *grad_w_last, void *grad_x_seq,
                                      void *grad_v_init, void *grad_w_init, hipStream_t stream);
int launch_backward(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                    const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                    const void *h_seq, const void *v_init,
                    const float *k_device, void *grad_x_seq, void *grad_v_init, float *grad_rtau,
                    float *workspace, hipStream_t stream);
int launch_forward_pieces(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N, int64_t chunk,
                          const void *x_seq, const void *v_init, const float *k_device, void *spike_seq, void *v_seq,
                          void *v_last, void *checkpoints, hipStream_t stream);
int launch_backward_recompute_pieces(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N, int64_t chunk,
                                     const void *x_seq, const void *v_init, const float *k_device, const void *checkpoints,
                                     const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                                     void *grad_x_seq, void *grad_v_init, float *grad_rtau, float *workspace,
                                     hipStream_t stream);
int launch_forward_packed(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                          const void *x_seq, const void *v_init, const float *k_device, uint8_t *spike_bits,
                          void *v_seq, void *v_last, hipStream_t stream);
// block size (128 or 64 lanes) whose parked h fits in LDS for a sequence of T steps; 0 if none
int recompute_block(int dtype, int64_t T, bool round_each);
bool recompute_supported(int dtype, int64_t T, int64_t N);
bool recompute_preferred(int dtype, int64_t T, int64_t N, bool round_each);
int launch_backward_recompute(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                              const void *x_seq, const void *v_init, const float *k_device,
                              const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                              void *grad_x_seq, void *grad_v_init, float *grad_rtau, float *workspace,
                              hipStream_t stream);
int64_t plif_blocks(int dtype, int64_t N);
bool ssa_supported(int dtype, int cph, int64_t L);
int launch_ssa_lif(bool backward, int neuron, const sjhip_neuron_params &p, int64_t T, int64_t B, int heads, int cph, int64_t L,
                   float scale, const uint8_t *qkv_bits, const float *v_init, float *spikes, float *h_seq, float *v_last,
                   const float *grad_spikes, const float *grad_v_last, float *grad_qkv, float *grad_v_init,
                   hipStream_t stream);
int launch_ssa(bool backward, int dtype, int64_t samples, int heads, int cph, int64_t L, float scale, const void *qkv,
               const uint8_t *qkv_bits, const void *grad_out, void *out, void *grad_qkv, hipStream_t stream);
int launch_bit_pack(int dtype, int64_t n, const void *src, uint8_t *dst, hipStream_t stream);
int launch_bit_unpack(int dtype, int64_t n, const uint8_t *src, void *dst, hipStream_t stream);
int launch_stream_probe(int reads, int writes, int nontemporal, int64_t floats_per_stream, const float *const *in,
                        float *const *out, hipStream_t stream);
int64_t mfma_probe_blocks(int wavefronts_per_simd);
int launch_mfma_probe(int operands, int wavefronts_per_simd, int iterations, float *sink, int64_t sink_floats, hipStream_t stream);
int64_t pwconv_planes_elems(int64_t rows, int64_t cols);
int launch_pwconv_split_weight(const float *w, int64_t rows, int64_t cols, int transpose, uint16_t *planes, hipStream_t stream);
int launch_pwconv_split_weight_f16(const float *w, int64_t rows, int64_t cols, int transpose, uint16_t *planes, float *amax_reset,
                                   int64_t amax_floats, hipStream_t stream);
int launch_pwconv_amax(const float *x, int64_t S, int64_t per_sample, float *amax, hipStream_t stream);
int launch_pwconv_gemm(const uint16_t *a_planes, int a_terms, int64_t M, int64_t K, const float *b, int b_terms,
                       const float *b_amax, int64_t S, int64_t L, float *c, float *stats, hipStream_t stream, bool b_bits = false);
int64_t pwconv_gemm_stats_rows(int64_t K, int64_t S, int64_t L);
int64_t pwconv_dw_workspace_floats(int64_t M, int64_t N, int64_t S);
int launch_pwconv_grad_weight(const float *dy, int dy_terms, const float *dy_amax, const float *x, int x_terms,
                              const float *x_amax, int64_t S, int64_t M, int64_t N, int64_t L, float *dw, float *workspace,
                              hipStream_t stream, bool x_bits = false);
int64_t pwconv_plane_ld(int64_t S, int64_t L);
int launch_pwconv_split_planes(const float *x, int64_t S, int64_t C, int64_t L, int terms, const float *amax, uint16_t *planes,
                               hipStream_t stream);
int64_t pwconv_gemm_planes_stats_rows(int64_t S, int64_t L);
int launch_pwconv_gemm_planes(const uint16_t *a_planes, int64_t M, int64_t K, const uint16_t *b_planes, int b_terms,
                              const float *b_amax, int64_t S, int64_t L, float *c, float *stats, hipStream_t stream);
int64_t pwconv_dw_planes_workspace_floats(int64_t M, int64_t N, int64_t S, int64_t L);
int launch_pwconv_grad_weight_planes(const uint16_t *dy_planes, const float *dy_amax, const uint16_t *x_planes, int x_terms,
                                     const float *x_amax, int64_t S, int64_t M, int64_t N, int64_t L, float *dw,
                                     float *workspace, hipStream_t stream);
int launch_bn_stats(const float *y, int64_t S, int64_t C, int64_t L, float *partial, hipStream_t stream);
int launch_bn_finalize(const float *partial, int64_t rows, int64_t count, int64_t C, const float *gamma, const float *beta, float eps,
                       float momentum, float *running_mean, float *running_var, float *scale, float *shift, float *mean,
                       float *invstd, int64_t *batches_tracked, hipStream_t stream);
// (k_device: PLIF's k = sigmoid(w) in device memory, else nullptr; grad_k + k_workspace: where dL/dk goes, PLIF only)
int launch_bn_lif_forward(int neuron, const sjhip_neuron_params &p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                          const float *scale, const float *shift, const float *v_init, const float *k_device, float *spike_seq,
                          uint8_t *spike_bits, float *v_last, hipStream_t stream);
int64_t bn_lif_backward_k_workspace_floats(int64_t B, int64_t C, int64_t L);
int launch_bn_lif_backward(int neuron, const sjhip_neuron_params &p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                           const float *scale, const float *shift, const float *v_init, const float *k_device,
                           const float *grad_spike_seq, const float *grad_v_last, float *grad_z, float *grad_v_init, float *partial,
                           float *grad_k, float *k_workspace, hipStream_t stream);
int launch_bn_backward_finalize(const float *partial, int64_t T, int64_t B, int64_t C, int64_t L, int training, const float *gamma,
                                const float *mean, const float *invstd, float *dgamma, float *dbeta, float *coef,
                                float *amax_reset, hipStream_t stream);
int launch_bn_grad_input(const float *g, const float *y, const float *coef, int64_t S, int64_t C, int64_t L, float *dy, float *amax,
                         hipStream_t stream);

}  // namespace sjhip
