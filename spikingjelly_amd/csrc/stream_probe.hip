// Plain streaming kernels that measure what the memory system gives to the access mixes of the neuron kernels:
// R read streams and W write streams of fp32, one 16-byte access per work-item and stream, nothing else.  They are the
// ceilings the neuron kernels' bandwidth is compared with (a forward with v_seq moves 1 read : 2 writes, a training
// forward that also saves h_seq 1 : 3, a backward 3 : 1), measured on the same device in the same run.
#include "sjhip_common.h"

namespace sjhip {

namespace {

struct ProbeArgs {
  const f32x4 *in[4];
  f32x4 *out[4];
  int64_t quads;  // 16-byte words per stream
};

template <int R, int W, bool NT> __global__ void __launch_bounds__(256) stream_probe_kernel(const ProbeArgs a) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= a.quads) return;
  f32x4 sum = (f32x4)(1.0f);
#pragma unroll
  for (int r = 0; r < R; ++r) sum += stream_load<NT>(a.in[r] + i);
  if (W == 0) {
    // keep the loads alive without writing: the stored value would need a sum no input produces
    if (sum.x == 1.2345e38f) a.out[0][i] = sum;
  } else {
#pragma unroll
    for (int w = 0; w < W; ++w) stream_store<NT>(a.out[w] + i, sum);
  }
}

// Matrix-core probe: a wavefront issues 16 v_mfma_f32_32x32x16_f16 per iteration (four operand pairs on four independent
// accumulators, so no instruction waits for another) and nothing else; one block of four wavefronts per SIMD slot.
// What it sustains depends on the operands, because the chip lowers its clock under the matrix cores' power draw.
typedef _Float16 probe_f16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
__device__ __forceinline__ uint32_t probe_hash(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}
__global__ void __launch_bounds__(256) mfma_probe_kernel(int operands, int iterations, float *sink) {
  probe_f16x8 a[4], b[4];
#pragma unroll
  for (int s = 0; s < 4; ++s)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float va = 0.0f, vb = 0.0f;
      if (operands != 0) {  // uniform in [-1, 1), different for every lane, element and operand
        va = (float)(probe_hash(blockIdx.x * 977u + threadIdx.x * 31u + s * 8u + i) & 0xffffu) / 32768.0f - 1.0f;
        vb = (float)(probe_hash(blockIdx.x * 613u + threadIdx.x * 17u + s * 8u + i + 99u) & 0xffffu) / 32768.0f - 1.0f;
      }
      a[s][i] = (_Float16)va;
      b[s][i] = (_Float16)vb;
    }
  probe_f32x16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[s], b[(s + i) & 3], acc[i], 0, 0, 0);
  }
  float x = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) x += acc[i][r];
  if (threadIdx.x == 0) sink[blockIdx.x] = x;  // keeps the products alive
}

template <int R, int W> int launch_probe(const ProbeArgs &a, bool nt, hipStream_t stream) {
  const int64_t blocks = (a.quads + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "stream_probe: %lld words", (long long)a.quads);
  ProfileScope prof(KC_STREAM_PROBE, stream);
  if (nt) hipLaunchKernelGGL((stream_probe_kernel<R, W, true>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  else hipLaunchKernelGGL((stream_probe_kernel<R, W, false>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
  return check_launch("stream_probe");
}

}  // namespace

int launch_stream_probe(int reads, int writes, int nontemporal, int64_t floats_per_stream, const float *const *in,
                        float *const *out, hipStream_t stream) {
  if (reads < 0 || reads > 3 || writes < 0 || writes > 3 || reads + writes == 0)
    return fail(SJHIP_ERR_INVALID, "stream_probe: %d reads, %d writes (0..3 each, not both 0)", reads, writes);
  if (floats_per_stream < 4 || floats_per_stream % 4 != 0) return fail(SJHIP_ERR_INVALID, "stream_probe: %lld floats per stream must be a positive multiple of 4", (long long)floats_per_stream);
  ProbeArgs a;
  for (int i = 0; i < 4; ++i) { a.in[i] = nullptr; a.out[i] = nullptr; }
  for (int r = 0; r < reads; ++r) {
    if (!in || !in[r] || !aligned16(in[r])) return fail(SJHIP_ERR_INVALID, "stream_probe: input %d is NULL or not 16-byte aligned", r);
    a.in[r] = reinterpret_cast<const f32x4 *>(in[r]);
  }
  const int outs = writes > 0 ? writes : 1;  // a read-only probe still takes one (never written) output pointer
  for (int w = 0; w < outs; ++w) {
    if (!out || !out[w] || !aligned16(out[w])) return fail(SJHIP_ERR_INVALID, "stream_probe: output %d is NULL or not 16-byte aligned", w);
    a.out[w] = reinterpret_cast<f32x4 *>(out[w]);
  }
  a.quads = floats_per_stream / 4;
  const bool nt = nontemporal != 0;
  switch (reads * 4 + writes) {
    case 1 * 4 + 0: return launch_probe<1, 0>(a, nt, stream);
    case 2 * 4 + 0: return launch_probe<2, 0>(a, nt, stream);
    case 3 * 4 + 0: return launch_probe<3, 0>(a, nt, stream);
    case 0 * 4 + 1: return launch_probe<0, 1>(a, nt, stream);
    case 0 * 4 + 2: return launch_probe<0, 2>(a, nt, stream);
    case 0 * 4 + 3: return launch_probe<0, 3>(a, nt, stream);
    case 1 * 4 + 1: return launch_probe<1, 1>(a, nt, stream);
    case 1 * 4 + 2: return launch_probe<1, 2>(a, nt, stream);
    case 1 * 4 + 3: return launch_probe<1, 3>(a, nt, stream);
    case 2 * 4 + 1: return launch_probe<2, 1>(a, nt, stream);
    case 3 * 4 + 1: return launch_probe<3, 1>(a, nt, stream);
    default: return fail(SJHIP_ERR_UNSUPPORTED, "stream_probe: mix %d reads : %d writes is not instantiated", reads, writes);
  }
}

int64_t mfma_probe_blocks(int wavefronts_per_simd) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
  return (int64_t)cus * wavefronts_per_simd;
}

int launch_mfma_probe(int operands, int wavefronts_per_simd, int iterations, float *sink, int64_t sink_floats, hipStream_t stream) {
  if (operands < 0 || operands > 1 || wavefronts_per_simd < 1 || wavefronts_per_simd > 8 || iterations < 1 || iterations > (1 << 24))
    return fail(SJHIP_ERR_INVALID, "mfma_probe: operands %d (0 zeros, 1 random), %d wavefronts per SIMD (1..8), %d iterations (1..2^24)", operands, wavefronts_per_simd, iterations);
  const int64_t blocks = mfma_probe_blocks(wavefronts_per_simd);
  if (!sink || sink_floats < blocks) return fail(SJHIP_ERR_INVALID, "mfma_probe: sink holds %lld floats, %lld blocks write one each", (long long)sink_floats, (long long)blocks);
  ProfileScope prof(KC_MFMA_PROBE, stream);
  hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, operands, iterations, sink);
  return check_launch("mfma_probe");
}

}  // namespace sjhip
