// Host launcher of the multi-step backward kernels and of the PLIF dL/dk reduction.
#include "neuron_bwd.h"

#include <cmath>

namespace sjhip {

// Fixed-order final sum of the per-block partials: lane i adds partials[i], [i+1024], ... in fp64,
// then a binary tree over the 1024 lanes through LDS.  Same order on every run.
__global__ void __launch_bounds__(1024) plif_reduce_kernel(const float *partials, int64_t count,
                                                            const float *k_device, float k_host,
                                                            int decay_input, float *out) {
  __shared__ double tree[1024];
  double sum = 0.0;
  for (int64_t i = threadIdx.x; i < count; i += 1024) sum += (double)partials[i];
  tree[threadIdx.x] = sum;
  __syncthreads();
  for (int stride = 512; stride > 0; stride >>= 1) {
    if ((int)threadIdx.x < stride) tree[threadIdx.x] += tree[threadIdx.x + stride];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    double total = tree[0];
    if (decay_input) total /= (double)(k_device ? *k_device : k_host);
    out[0] = (float)total;
  }
}

namespace {

template <typename S, int MODE>
void launch_mode(const BwdArgs &a, bool vector, dim3 grid, dim3 threads, unsigned lds, hipStream_t stream) {
  if (vector) hipLaunchKernelGGL((backward_kernel<S, true, MODE>), grid, threads, lds, stream, a);
  else hipLaunchKernelGGL((backward_kernel<S, false, MODE>), grid, threads, lds, stream, a);
}

template <typename S>
int launch_typed(BwdArgs &a, bool vector, int mode, float *grad_k_out, hipStream_t stream) {
  const bool plif = mode == BWD_PLIF;
  const int block = tuning().bwd_block;
  const int V = vector ? Acc<S, true, true>::V : 1;
  const int64_t items = (a.N + V - 1) / V;
  const int64_t blocks = (items + block - 1) / block;
  if (blocks > 0x7fffffffLL) return fail(SJHIP_ERR_TOO_LARGE, "backward: N=%lld needs %lld blocks", (long long)a.N, (long long)blocks);
  const dim3 grid((unsigned)blocks), threads(block);
  const unsigned lds = occupancy_cap_lds(tuning().bwd_blocks_per_cu);
  {
    ProfileScope prof(KC_BACKWARD, stream);
    if (a.T <= kShortSequence) {
      if (mode == BWD_PLIF) launch_mode<S, BWD_PLIF | BWD_SHORT>(a, vector, grid, threads, lds, stream);
      else if (mode == BWD_QIF) launch_mode<S, BWD_QIF | BWD_SHORT>(a, vector, grid, threads, lds, stream);
      else launch_mode<S, BWD_PLAIN | BWD_SHORT>(a, vector, grid, threads, lds, stream);
    } else if (mode == BWD_PLIF) launch_mode<S, BWD_PLIF>(a, vector, grid, threads, lds, stream);
    else if (mode == BWD_QIF) launch_mode<S, BWD_QIF>(a, vector, grid, threads, lds, stream);
    else launch_mode<S, BWD_PLAIN>(a, vector, grid, threads, lds, stream);
    int rc = check_launch("backward");
    if (rc != SJHIP_OK) return rc;
  }
  if (plif && !a.atomic_reduce) return launch_plif_reduce(a, blocks, grad_k_out, stream);
  return SJHIP_OK;
}

}  // namespace

int launch_plif_reduce(const BwdArgs &a, int64_t blocks, float *grad_k_out, hipStream_t stream) {
  ProfileScope prof(KC_PLIF_REDUCE, stream);
  hipLaunchKernelGGL(plif_reduce_kernel, dim3(1), dim3(1024), 0, stream, (const float *)a.partials, blocks,
                     a.k_device, a.k, a.decay_input, grad_k_out);
  return check_launch("plif_reduce");
}

int64_t plif_blocks(int dtype, int64_t N) {
  (void)dtype;
  // upper bound for every block size (>= 64 lanes) and access width the launcher may pick
  return (N + 63) / 64;
}

int launch_backward(int neuron, int dtype, const sjhip_neuron_params &p, int64_t T, int64_t N,
                    const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                    const void *h_seq, const void *v_init,
                    const float *k_device, void *grad_x_seq, void *grad_v_init, float *grad_rtau,
                    float *workspace, hipStream_t stream) {
  BwdArgs a;
  int rc = build_bwd_args(a, neuron, dtype, p, T, N, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, v_init, k_device,
                          grad_x_seq, grad_v_init, grad_rtau, workspace);
  if (rc != SJHIP_OK) return rc;
  const int mode = neuron == SJHIP_NEURON_PLIF ? BWD_PLIF : ((neuron == SJHIP_NEURON_QIF || neuron == SJHIP_NEURON_EIF) ? BWD_QIF : BWD_PLAIN);

  const int esize = dtype == SJHIP_F32 ? 4 : 2;
  const int V = 16 / esize;
  const bool vector = (N % V == 0) && aligned16(grad_spike_seq) && aligned16(h_seq) && aligned16(grad_x_seq) &&
                      (grad_v_init == nullptr || aligned16(grad_v_init)) && (grad_v_seq == nullptr || aligned16(grad_v_seq)) &&
                      (grad_v_last == nullptr || aligned16(grad_v_last)) &&
                      (v_init == nullptr || a.v_init_broadcast || aligned16(v_init));

  switch (dtype) {
    case SJHIP_F32: return launch_typed<float>(a, vector, mode, grad_rtau, stream);
    case SJHIP_F16: return launch_typed<f16_t>(a, vector, mode, grad_rtau, stream);
    case SJHIP_BF16: return launch_typed<bf16_t>(a, vector, mode, grad_rtau, stream);
    default: return fail(SJHIP_ERR_INVALID, "backward: dtype %d", dtype);
  }
}

}  // namespace sjhip
