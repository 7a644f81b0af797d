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

}  // namespace sjhip
