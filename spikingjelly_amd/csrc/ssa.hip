// Spiking self-attention contraction  out = scale * (V K^T) Q  and its backward, on MFMA.
//
// Layout and order follow the reference (layer/attention.py:346-353, `_ssa_kernel_torch`): qkv is
// [TB, 3, H, Cph, L] (q, k, v of one sample stacked on dim 1; each head a row-major [Cph, L] tile of
// binary spikes), S = V K^T is [Cph, Cph] (contraction over the L tokens), out = scale * S Q is
// [TB, H, Cph, L].  One wavefront owns one (sample, head) problem:
//   * the three tiles are staged once through LDS as bf16 (0/1 are exact), rows padded with zeros;
//   * S = V K^T runs on v_mfma_f32_32x32x16_bf16, fp32 accumulation -- exact integers <= L;
//   * S goes through LDS (accumulator layout -> operand layout) as bf16, exact because L <= 256;
//   * out = S Q on the same bf16 MFMA; sums are integers <= Cph * L < 2^24, so the fp32 result is the
//     exact integer and `scale` (a power of two in the reference, 0.125) is applied once.
// Hence the forward equals an int64 matmul of the spikes times scale, bit for bit, in fp32 output,
// and after one rounding in 16-bit output (what torch's bf16 matmuls also produce).
//
// The backward has real-valued operands (grad_out, dS), so it uses the fp32 MFMA
// (v_mfma_f32_32x32x2_f32): dS = scale * dO Q^T, dQ = scale * S^T dO, dV = dS K, dK = dS^T V,
// with S recomputed on the bf16 MFMA as in the forward.
//
// The k index of both MFMA operands uses the same lane -> k mapping, so only the row/column mapping of
// the operands and the accumulator layout (row = 8*(r/4) + 4*(lane/32) + r%4, col = lane%32 for
// accumulator register r) matter.
#include "sjhip_common.h"

#include <mutex>

namespace sjhip {

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint16_t u16x8 __attribute__((ext_vector_type(8)));

constexpr unsigned kSsaMaxLds = 159u * 1024u;

struct SsaArgs {
  const void *qkv;
  const void *grad_out;
  void *out;
  void *grad_qkv;
  int64_t problems;  // TB * heads
  int heads;
  int cph;    // channels per head (<= 64); tiles are zero-padded to 32 or 64 rows in LDS
  int L;      // tokens
  int Lp;     // LDS row stride (elements) of the bf16 tiles
  int Lq;     // LDS row stride (floats) of the grad_out tile
  float scale;
};

template <typename S> struct Io;
template <> struct Io<float> {
  typedef float elem_t;
  static __device__ __forceinline__ float get(const elem_t *p, int64_t i) { return p[i]; }
  static __device__ __forceinline__ void put(elem_t *p, int64_t i, float v) { p[i] = v; }
};
template <> struct Io<f16_t> {
  typedef uint16_t elem_t;
  static __device__ __forceinline__ float get(const elem_t *p, int64_t i) { return Cvt<f16_t>::to_float(p[i]); }
  static __device__ __forceinline__ void put(elem_t *p, int64_t i, float v) { p[i] = Cvt<f16_t>::from_float(v); }
};
template <> struct Io<bf16_t> {
  typedef uint16_t elem_t;
  static __device__ __forceinline__ float get(const elem_t *p, int64_t i) { return Cvt<bf16_t>::to_float(p[i]); }
  static __device__ __forceinline__ void put(elem_t *p, int64_t i, float v) { p[i] = Cvt<bf16_t>::from_float(v); }
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

// global [rows, L] tile -> LDS bf16 [rows][Lp], columns L..Lp-1 zeroed
template <typename S>
__device__ __forceinline__ void stage_bf16(const typename Io<S>::elem_t *src, uint16_t *dst, int rows, int rows_pad,
                                           int L, int Lp) {
  const int lane = threadIdx.x;
  for (int idx = lane; idx < rows_pad * Lp; idx += 64) {
    const int r = idx / Lp, c = idx - r * Lp;
    dst[idx] = (c < L && r < rows) ? Cvt<bf16_t>::from_float(Io<S>::get(src, (int64_t)r * L + c)) : (uint16_t)0;
  }
}

// global [rows, L] tile -> LDS fp32 [rows][Lq], padded with zeros
template <typename S>
__device__ __forceinline__ void stage_f32(const typename Io<S>::elem_t *src, float *dst, int rows, int rows_pad, int L,
                                          int Lq) {
  const int lane = threadIdx.x;
  for (int idx = lane; idx < rows_pad * Lq; idx += 64) {
    const int r = idx / Lq, c = idx - r * Lq;
    dst[idx] = (c < L && r < rows) ? Io<S>::get(src, (int64_t)r * L + c) : 0.0f;
  }
}

// S block (mi, ni) = V[mi*32.., :] K[ni*32.., :]^T over the padded token axis, bf16 MFMA
__device__ __forceinline__ f32x16 gemm_vkt(const uint16_t *v_lds, const uint16_t *k_lds, int mi, int ni, int Lp, int Lk) {
  const int lane = threadIdx.x;
  const uint16_t *ap = v_lds + (mi * 32 + (lane & 31)) * Lp + 8 * (lane >> 5);
  const uint16_t *bp = k_lds + (ni * 32 + (lane & 31)) * Lp + 8 * (lane >> 5);
  f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < Lk; k0 += 16) {
    const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u16x8 *>(ap + k0));
    const bf16x8 b = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u16x8 *>(bp + k0));
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
  }
  return acc;
}

// accumulator register r of this lane sits at (row, col) of its 32x32 block
__device__ __forceinline__ int acc_row(int r) { return 8 * (r >> 2) + 4 * ((int)threadIdx.x >> 5) + (r & 3); }
__device__ __forceinline__ int acc_col() { return (int)threadIdx.x & 31; }

template <typename S, int MC>
__global__ void __launch_bounds__(64) ssa_forward_kernel(const SsaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ssa_lds[];
  typedef typename Io<S>::elem_t E;
  constexpr int CPH = 32 * MC;
  const int L = a.L, Lp = a.Lp;
  const int Lk = (L + 15) & ~15;
  constexpr int LS = CPH + 8;  // row stride of the bf16 S tile
  uint16_t *q_lds = reinterpret_cast<uint16_t *>(ssa_lds);
  uint16_t *k_lds = q_lds + CPH * Lp;
  uint16_t *v_lds = k_lds + CPH * Lp;
  uint16_t *s_lds = v_lds + CPH * Lp;

  const int64_t p = blockIdx.x;
  const int64_t sample = p / a.heads, head = p - sample * a.heads;
  const int cph = a.cph;
  const int64_t tile = (int64_t)cph * L;
  const E *qkv = static_cast<const E *>(a.qkv);
  const E *qg = qkv + ((sample * 3 + 0) * a.heads + head) * tile;
  const E *kg = qkv + ((sample * 3 + 1) * a.heads + head) * tile;
  const E *vg = qkv + ((sample * 3 + 2) * a.heads + head) * tile;
  stage_bf16<S>(qg, q_lds, cph, CPH, L, Lp);
  stage_bf16<S>(kg, k_lds, cph, CPH, L, Lp);
  stage_bf16<S>(vg, v_lds, cph, CPH, L, Lp);
  __syncthreads();

  // S = V K^T, exact integers <= L <= 256 -> bf16 in LDS, operand layout for the second product
#pragma unroll
  for (int mi = 0; mi < MC; ++mi) {
#pragma unroll
    for (int ni = 0; ni < MC; ++ni) {
      const f32x16 acc = gemm_vkt(v_lds, k_lds, mi, ni, Lp, Lk);
#pragma unroll
      for (int r = 0; r < 16; ++r)
        s_lds[(mi * 32 + acc_row(r)) * LS + ni * 32 + acc_col()] = Cvt<bf16_t>::from_float(acc[r]);
    }
  }
  __syncthreads();

  // out[c1, l] = scale * sum_c2 S[c1, c2] Q[c2, l]
  const int lane = threadIdx.x;
  E *og = static_cast<E *>(a.out) + p * tile;
  const int ntiles = (L + 31) / 32;
  for (int nt = 0; nt < ntiles; ++nt) {
#pragma unroll
    for (int mi = 0; mi < MC; ++mi) {
      f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int k0 = 0; k0 < CPH; k0 += 16) {
        const bf16x8 av = __builtin_bit_cast(
            bf16x8, *reinterpret_cast<const u16x8 *>(s_lds + (mi * 32 + (lane & 31)) * LS + k0 + 8 * (lane >> 5)));
        u16x8 bw;
#pragma unroll
        for (int j = 0; j < 8; ++j) bw[j] = q_lds[(k0 + 8 * (lane >> 5) + j) * Lp + nt * 32 + (lane & 31)];
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, __builtin_bit_cast(bf16x8, bw), acc, 0, 0, 0);
      }
      const int col = nt * 32 + acc_col();
      if (col < L) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = mi * 32 + acc_row(r);
          if (row < cph) Io<S>::put(og, (int64_t)row * L + col, acc[r] * a.scale);
        }
      }
    }
  }
}

// D[m, n] (+)= sum_k A(m, k) B(k, n) on the fp32 MFMA, K stepping by 2; fa(m, k) / fb(k, n) fetch operands
template <typename FA, typename FB>
__device__ __forceinline__ f32x16 gemm_f32(int K, FA fa, FB fb) {
  const int lane = threadIdx.x;
  const int mn = lane & 31, kh = lane >> 5;
  f32x16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  for (int k0 = 0; k0 < K; k0 += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa(mn, k0 + kh), fb(k0 + kh, mn), acc, 0, 0, 0);
  return acc;
}

template <typename S, int MC>
__global__ void __launch_bounds__(64) ssa_backward_kernel(const SsaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ssa_lds[];
  typedef typename Io<S>::elem_t E;
  constexpr int CPH = 32 * MC;
  constexpr int LS = CPH + 1;  // row stride of the fp32 S / dS tiles
  const int L = a.L, Lp = a.Lp, Lq = a.Lq;
  const int Lk = (L + 15) & ~15;
  const int L2 = (L + 1) & ~1;
  float *do_lds = reinterpret_cast<float *>(ssa_lds);
  float *s_lds = do_lds + CPH * Lq;
  float *ds_lds = s_lds + CPH * LS;
  uint16_t *q_lds = reinterpret_cast<uint16_t *>(ds_lds + CPH * LS);
  uint16_t *k_lds = q_lds + CPH * Lp;
  uint16_t *v_lds = k_lds + CPH * Lp;

  const int64_t p = blockIdx.x;
  const int64_t sample = p / a.heads, head = p - sample * a.heads;
  const int cph = a.cph;
  const int64_t tile = (int64_t)cph * L;
  const E *qkv = static_cast<const E *>(a.qkv);
  const int64_t qoff = ((sample * 3 + 0) * a.heads + head) * tile;
  const int64_t koff = ((sample * 3 + 1) * a.heads + head) * tile;
  const int64_t voff = ((sample * 3 + 2) * a.heads + head) * tile;
  stage_bf16<S>(qkv + qoff, q_lds, cph, CPH, L, Lp);
  stage_bf16<S>(qkv + koff, k_lds, cph, CPH, L, Lp);
  stage_bf16<S>(qkv + voff, v_lds, cph, CPH, L, Lp);
  stage_f32<S>(static_cast<const E *>(a.grad_out) + p * tile, do_lds, cph, CPH, L, Lq);
  __syncthreads();

  const float scale = a.scale;
  // S = V K^T (exact) and dS = scale * dO Q^T, both [CPH, CPH], into LDS
#pragma unroll
  for (int mi = 0; mi < MC; ++mi) {
#pragma unroll
    for (int ni = 0; ni < MC; ++ni) {
      const f32x16 s_acc = gemm_vkt(v_lds, k_lds, mi, ni, Lp, Lk);
      const f32x16 ds_acc = gemm_f32(
          L2, [&](int m, int k) { return do_lds[(mi * 32 + m) * Lq + k]; },
          [&](int k, int n) { return bf16_bits_to_float(q_lds[(ni * 32 + n) * Lp + k]); });
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int idx = (mi * 32 + acc_row(r)) * LS + ni * 32 + acc_col();
        s_lds[idx] = s_acc[r];
        ds_lds[idx] = ds_acc[r] * scale;
      }
    }
  }
  __syncthreads();

  E *gq = static_cast<E *>(a.grad_qkv);
  const int ntiles = (L + 31) / 32;
  for (int nt = 0; nt < ntiles; ++nt) {
    const int col = nt * 32 + acc_col();
#pragma unroll
    for (int mi = 0; mi < MC; ++mi) {
      // dQ[c2, l] = scale * sum_c1 S[c1, c2] dO[c1, l]
      const f32x16 dq = gemm_f32(
          CPH, [&](int m, int k) { return s_lds[k * LS + mi * 32 + m]; },
          [&](int k, int n) { return do_lds[k * Lq + nt * 32 + n]; });
      // dV[c1, l] = sum_c2 dS[c1, c2] K[c2, l]
      const f32x16 dv = gemm_f32(
          CPH, [&](int m, int k) { return ds_lds[(mi * 32 + m) * LS + k]; },
          [&](int k, int n) { return bf16_bits_to_float(k_lds[k * Lp + nt * 32 + n]); });
      // dK[c2, l] = sum_c1 dS[c1, c2] V[c1, l]
      const f32x16 dk = gemm_f32(
          CPH, [&](int m, int k) { return ds_lds[k * LS + mi * 32 + m]; },
          [&](int k, int n) { return bf16_bits_to_float(v_lds[k * Lp + nt * 32 + n]); });
      if (col < L) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = mi * 32 + acc_row(r);
          if (row >= cph) continue;
          const int64_t o = (int64_t)row * L + col;
          Io<S>::put(gq, qoff + o, dq[r] * scale);
          Io<S>::put(gq, koff + o, dk[r]);
          Io<S>::put(gq, voff + o, dv[r]);
        }
      }
    }
  }
}

int lds_row_bf16(int L) { return ((L + 31) & ~31) + 8; }
int lds_row_f32(int L) { return ((L + 31) & ~31) + 4; }

int padded_rows(int cph) { return cph <= 32 ? 32 : 64; }
unsigned forward_lds(int cph, int L) {
  const int c = padded_rows(cph);
  return (unsigned)((3 * c * lds_row_bf16(L) + c * (c + 8)) * 2);
}
unsigned backward_lds(int cph, int L) {
  const int c = padded_rows(cph);
  return (unsigned)(3 * c * lds_row_bf16(L) * 2 + (c * lds_row_f32(L) + 2 * c * (c + 1)) * 4);
}

template <typename K>
int launch_with_lds(K kernel, const SsaArgs &a, unsigned lds, hipStream_t stream, std::once_flag &once, hipError_t &attr_rc,
                    const char *what) {
  std::call_once(once, [&]() {
    attr_rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)kSsaMaxLds);
    (void)hipGetLastError();
  });
  if (lds > 64u * 1024u && attr_rc != hipSuccess)
    return fail(SJHIP_ERR_LAUNCH, "%s: cannot raise the dynamic LDS limit: %s", what, hipGetErrorString(attr_rc));
  hipLaunchKernelGGL(kernel, dim3((unsigned)a.problems), dim3(64), lds, stream, a);
  return check_launch(what);
}

template <typename S, int MC>
int launch_fwd(const SsaArgs &a, hipStream_t stream) {
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  return launch_with_lds(ssa_forward_kernel<S, MC>, a, forward_lds(a.cph, a.L), stream, once, attr_rc, "ssa_forward");
}
template <typename S, int MC>
int launch_bwd(const SsaArgs &a, hipStream_t stream) {
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  return launch_with_lds(ssa_backward_kernel<S, MC>, a, backward_lds(a.cph, a.L), stream, once, attr_rc, "ssa_backward");
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
               const void *grad_out, void *out, void *grad_qkv, hipStream_t stream) {
  if (!ssa_supported(dtype, cph, L))
    return fail(SJHIP_ERR_UNSUPPORTED, "ssa: dtype %d, %d channels per head, %lld tokens is not supported "
                "(needs at most 64 channels per head, at most 256 tokens, and the tiles of one head fitting in LDS)", dtype, cph, (long long)L);
  if (samples < 1 || heads < 1 || samples * heads > 0x7fffffffLL)
    return fail(SJHIP_ERR_INVALID, "ssa: samples=%lld heads=%d", (long long)samples, heads);
  SsaArgs a;
  a.qkv = qkv; a.grad_out = grad_out; a.out = out; a.grad_qkv = grad_qkv;
  a.problems = samples * heads; a.heads = heads; a.cph = cph; a.L = (int)L;
  a.Lp = lds_row_bf16((int)L); a.Lq = lds_row_f32((int)L); a.scale = scale;
  ProfileScope prof(backward ? KC_SSA_BACKWARD : KC_SSA_FORWARD, stream);
  switch (dtype) {
    case SJHIP_F32: return launch_dtype<float>(a, backward, stream);
    case SJHIP_F16: return launch_dtype<f16_t>(a, backward, stream);
    default: return launch_dtype<bf16_t>(a, backward, stream);
  }
}

}  // namespace sjhip
