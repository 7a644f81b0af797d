// Spike bit-packing: 8 binary spikes -> 1 byte, LSB first over the flattened tensor, and back.
//
// Layout follows the reference (triton_kernel/compress.py:19-44, 47-111; cuda_kernel/tensor_cache.py:16-93):
// byte j bit i holds element 8j+i, the last byte is zero-padded.  An element counts as a spike when it
// is non-zero (what `.to(torch.bool)` does in the reference's torch path: -0.0 is no spike, NaN is).
//
// Unlike the reference kernels (eight stride-8 scalar accesses per byte) every lane moves one 128-bit
// vector of consecutive elements, so a wavefront reads/writes 1 KiB contiguous per instruction; the
// 4-bit results of fp32 lanes are paired with one lane shuffle.  Each work-item handles PACK_R vectors
// so several loads are in flight.  What does not fill a whole vector (and unaligned buffers) goes
// through the element-wise kernels.
#include "sjhip_common.h"

namespace sjhip {

namespace {

constexpr int PACK_R = 4;

template <int ESIZE> __device__ __forceinline__ uint32_t spike_bits(u32x4 r);
template <> __device__ __forceinline__ uint32_t spike_bits<4>(u32x4 r) {
  return ((r.x & 0x7fffffffu) ? 1u : 0u) | ((r.y & 0x7fffffffu) ? 2u : 0u) | ((r.z & 0x7fffffffu) ? 4u : 0u) |
         ((r.w & 0x7fffffffu) ? 8u : 0u);
}
template <> __device__ __forceinline__ uint32_t spike_bits<2>(u32x4 r) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
  uint32_t b = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    b |= ((w[i] & 0x00007fffu) ? 1u : 0u) << (2 * i);
    b |= ((w[i] & 0x7fff0000u) ? 1u : 0u) << (2 * i + 1);
  }
  return b;
}
template <> __device__ __forceinline__ uint32_t spike_bits<1>(u32x4 r) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
  uint32_t b = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) b |= ((w[i] >> (8 * j)) & 0xffu ? 1u : 0u) << (4 * i + j);
  }
  return b;
}

// items = number of whole 16-byte vectors; for ESIZE 4 it is even so shuffle partners share fate.
template <int ESIZE>
__global__ void __launch_bounds__(256) pack_vector_kernel(const u32x4 *__restrict__ src, uint8_t *__restrict__ dst,
                                                          int64_t items) {
  const int64_t base = (int64_t)blockIdx.x * blockDim.x * PACK_R + threadIdx.x;
  u32x4 r[PACK_R];
#pragma unroll
  for (int i = 0; i < PACK_R; ++i) {
    const int64_t item = base + (int64_t)i * blockDim.x;
    r[i] = (item < items) ? stream_load<true>(src + item) : (u32x4)(0u);
  }
#pragma unroll
  for (int i = 0; i < PACK_R; ++i) {
    const int64_t item = base + (int64_t)i * blockDim.x;
    const uint32_t bits = spike_bits<ESIZE>(r[i]);
    if (ESIZE == 4) {
      const uint32_t other = __shfl_xor(bits, 1, 64);
      if (item < items && (threadIdx.x & 1) == 0) dst[item >> 1] = (uint8_t)(bits | (other << 4));
    } else if (ESIZE == 2) {
      if (item < items) dst[item] = (uint8_t)bits;
    } else {
      if (item < items) reinterpret_cast<uint16_t *>(dst)[item] = (uint16_t)bits;
    }
  }
}

template <int ESIZE> __device__ __forceinline__ bool elem_nonzero(const void *src, int64_t i);
template <> __device__ __forceinline__ bool elem_nonzero<4>(const void *src, int64_t i) {
  return (static_cast<const uint32_t *>(src)[i] & 0x7fffffffu) != 0;
}
template <> __device__ __forceinline__ bool elem_nonzero<2>(const void *src, int64_t i) {
  return (static_cast<const uint16_t *>(src)[i] & 0x7fffu) != 0;
}
template <> __device__ __forceinline__ bool elem_nonzero<1>(const void *src, int64_t i) {
  return static_cast<const uint8_t *>(src)[i] != 0;
}

// one work-item per output byte in [byte_begin, byte_end)
template <int ESIZE>
__global__ void __launch_bounds__(256) pack_scalar_kernel(const void *__restrict__ src, uint8_t *__restrict__ dst,
                                                          int64_t byte_begin, int64_t byte_end, int64_t n) {
  const int64_t j = byte_begin + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= byte_end) return;
  uint32_t b = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int64_t e = 8 * j + i;
    if (e < n && elem_nonzero<ESIZE>(src, e)) b |= 1u << i;
  }
  dst[j] = (uint8_t)b;
}

// `one` = bit pattern of 1 in the output dtype (fp32 0x3f800000, fp16 0x3c00, bf16 0x3f80, u8 0x01)
template <int ESIZE>
__global__ void __launch_bounds__(256) unpack_vector_kernel(const uint8_t *__restrict__ src, u32x4 *__restrict__ dst,
                                                            int64_t items, uint32_t one) {
  const int64_t base = (int64_t)blockIdx.x * blockDim.x * PACK_R + threadIdx.x;
#pragma unroll
  for (int i = 0; i < PACK_R; ++i) {
    const int64_t item = base + (int64_t)i * blockDim.x;
    if (item >= items) continue;
    uint32_t w[4];
    if (ESIZE == 4) {
      const uint32_t bits = (uint32_t)src[item >> 1] >> (4 * (int)(item & 1));
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = ((bits >> j) & 1u) ? one : 0u;
    } else if (ESIZE == 2) {
      const uint32_t bits = src[item];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        w[j] = (((bits >> (2 * j)) & 1u) ? one : 0u) | (((bits >> (2 * j + 1)) & 1u) ? (one << 16) : 0u);
    } else {
      const uint32_t bits = reinterpret_cast<const uint16_t *>(src)[item];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t x = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) x |= ((bits >> (4 * j + q)) & 1u) << (8 * q);
        w[j] = x * one;
      }
    }
    u32x4 r; r.x = w[0]; r.y = w[1]; r.z = w[2]; r.w = w[3];
    stream_store<true>(dst + item, r);
  }
}

// one work-item per output element in [elem_begin, n)
template <int ESIZE>
__global__ void __launch_bounds__(256) unpack_scalar_kernel(const uint8_t *__restrict__ src, void *__restrict__ dst,
                                                            int64_t elem_begin, int64_t n, uint32_t one) {
  const int64_t e = elem_begin + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  const uint32_t bit = (src[e >> 3] >> (e & 7)) & 1u;
  const uint32_t val = bit ? one : 0u;
  if (ESIZE == 4) static_cast<uint32_t *>(dst)[e] = val;
  else if (ESIZE == 2) static_cast<uint16_t *>(dst)[e] = (uint16_t)val;
  else static_cast<uint8_t *>(dst)[e] = (uint8_t)val;
}

int elem_size(int dtype) {
  switch (dtype) {
    case SJHIP_F32: return 4;
    case SJHIP_F16: case SJHIP_BF16: return 2;
    case SJHIP_U8: return 1;
    default: return 0;
  }
}

uint32_t one_pattern(int dtype) {
  switch (dtype) {
    case SJHIP_F32: return 0x3f800000u;
    case SJHIP_F16: return 0x3c00u;
    case SJHIP_BF16: return 0x3f80u;
    default: return 0x01u;
  }
}

template <int ESIZE>
int pack_typed(int64_t n, const void *src, uint8_t *dst, hipStream_t stream) {
  constexpr int V = 16 / ESIZE;              // elements per 128-bit vector
  constexpr int GROUP = V < 8 ? 8 : V;       // elements that fill whole bytes and whole vectors
  const int block = 256;
  const bool vec_ok = aligned16(src) && ((reinterpret_cast<uintptr_t>(dst) & 1u) == 0);
  const int64_t n_main = vec_ok ? (n / GROUP) * GROUP : 0;
  const int64_t total_bytes = (n + 7) / 8;
  ProfileScope prof(KC_BIT_PACK, stream);
  if (n_main > 0) {
    const int64_t items = n_main / V;
    const int64_t blocks = (items + (int64_t)block * PACK_R - 1) / ((int64_t)block * PACK_R);
    if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bit_pack: n=%lld", (long long)n);
    hipLaunchKernelGGL((pack_vector_kernel<ESIZE>), dim3((unsigned)blocks), dim3(block), 0, stream,
                       static_cast<const u32x4 *>(src), dst, items);
    int rc = check_launch("bit_pack");
    if (rc != SJHIP_OK) return rc;
  }
  const int64_t byte_begin = n_main / 8;
  if (byte_begin < total_bytes) {
    const int64_t rest = total_bytes - byte_begin;
    const int64_t blocks = (rest + block - 1) / block;
    if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bit_pack: n=%lld", (long long)n);
    hipLaunchKernelGGL((pack_scalar_kernel<ESIZE>), dim3((unsigned)blocks), dim3(block), 0, stream, src, dst,
                       byte_begin, total_bytes, n);
    return check_launch("bit_pack(tail)");
  }
  return SJHIP_OK;
}

template <int ESIZE>
int unpack_typed(int64_t n, const uint8_t *src, void *dst, uint32_t one, hipStream_t stream) {
  constexpr int V = 16 / ESIZE;
  constexpr int GROUP = V < 8 ? 8 : V;
  const int block = 256;
  const bool vec_ok = aligned16(dst) && ((reinterpret_cast<uintptr_t>(src) & 1u) == 0);
  const int64_t n_main = vec_ok ? (n / GROUP) * GROUP : 0;
  ProfileScope prof(KC_BIT_UNPACK, stream);
  if (n_main > 0) {
    const int64_t items = n_main / V;
    const int64_t blocks = (items + (int64_t)block * PACK_R - 1) / ((int64_t)block * PACK_R);
    if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bit_unpack: n=%lld", (long long)n);
    hipLaunchKernelGGL((unpack_vector_kernel<ESIZE>), dim3((unsigned)blocks), dim3(block), 0, stream, src,
                       static_cast<u32x4 *>(dst), items, one);
    int rc = check_launch("bit_unpack");
    if (rc != SJHIP_OK) return rc;
  }
  if (n_main < n) {
    const int64_t rest = n - n_main;
    const int64_t blocks = (rest + block - 1) / block;
    if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "bit_unpack: n=%lld", (long long)n);
    hipLaunchKernelGGL((unpack_scalar_kernel<ESIZE>), dim3((unsigned)blocks), dim3(block), 0, stream, src, dst,
                       n_main, n, one);
    return check_launch("bit_unpack(tail)");
  }
  return SJHIP_OK;
}

}  // namespace

int launch_bit_pack(int dtype, int64_t n, const void *src, uint8_t *dst, hipStream_t stream) {
  switch (elem_size(dtype)) {
    case 4: return pack_typed<4>(n, src, dst, stream);
    case 2: return pack_typed<2>(n, src, dst, stream);
    case 1: return pack_typed<1>(n, src, dst, stream);
    default: return fail(SJHIP_ERR_INVALID, "bit_pack: dtype %d", dtype);
  }
}

int launch_bit_unpack(int dtype, int64_t n, const uint8_t *src, void *dst, hipStream_t stream) {
  const uint32_t one = one_pattern(dtype);
  switch (elem_size(dtype)) {
    case 4: return unpack_typed<4>(n, src, dst, one, stream);
    case 2: return unpack_typed<2>(n, src, dst, one, stream);
    case 1: return unpack_typed<1>(n, src, dst, one, stream);
    default: return fail(SJHIP_ERR_INVALID, "bit_unpack: dtype %d", dtype);
  }
}

}  // namespace sjhip
