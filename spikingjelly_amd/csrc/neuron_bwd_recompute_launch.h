// Kernel launch of the recompute backward for one storage dtype; included by the per-dtype
// translation units so the three sets of kernels compile in parallel.
#pragma once

#include <mutex>

#include "neuron_bwd_recompute.h"

namespace sjhip {

// LDS per compute unit on gfx950 is 160 KiB; 1 KiB is left for the statically allocated reduction words
constexpr unsigned kRecomputeMaxLds = 159u * 1024u;

template <typename S, bool ROUND_EACH, int MODE>
int launch_kernel(const FwdArgs &f, const BwdArgs &b, int block, unsigned lds, int64_t blocks, hipStream_t stream) {
  auto kernel = backward_recompute_kernel<S, ROUND_EACH, MODE>;
  // a block may use more than the default 64 KiB of dynamic LDS only after this opt-in (once per kernel)
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [&]() {
    attr_rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)kRecomputeMaxLds);
    (void)hipGetLastError();  // a refusal is reported below, only if the launch really needs the larger limit
  });
  if (lds > 64u * 1024u && attr_rc != hipSuccess)
    return fail(SJHIP_ERR_LAUNCH, "backward(recompute): cannot raise the dynamic LDS limit: %s", hipGetErrorString(attr_rc));
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(block), lds, stream, f, b);
  return check_launch("backward(recompute)");
}

template <typename S, bool ROUND_EACH, int MODE>
int launch_pieces_kernel(const FwdArgs &f, const BwdArgs &b, const PieceArgs &p, int block, unsigned lds, int64_t blocks,
                         hipStream_t stream) {
  auto kernel = backward_recompute_pieces_kernel<S, ROUND_EACH, MODE>;
  // pieces of 16 steps stay below the default 64 KiB of dynamic LDS; longer pieces (17 steps and more at 256 lanes,
  // 33 and more at 128) do not and need the same opt-in as launch_kernel
  static std::once_flag once;
  static hipError_t attr_rc = hipSuccess;
  std::call_once(once, [&]() {
    attr_rc = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)kRecomputeMaxLds);
    (void)hipGetLastError();
  });
  if (lds > kRecomputeMaxLds)
    return fail(SJHIP_ERR_UNSUPPORTED, "backward(recompute, pieces): %u bytes of LDS per block exceed %u", lds, kRecomputeMaxLds);
  if (lds > 64u * 1024u && attr_rc != hipSuccess)
    return fail(SJHIP_ERR_LAUNCH, "backward(recompute, pieces): cannot raise the dynamic LDS limit: %s", hipGetErrorString(attr_rc));
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(block), lds, stream, f, b, p);
  return check_launch("backward(recompute, pieces)");
}

template <typename S, bool ROUND_EACH>
int launch_mode(const FwdArgs &f, const BwdArgs &b, int mode, int block, unsigned lds, int64_t blocks, hipStream_t stream,
                const PieceArgs *pieces) {
  if (pieces) {
    if (mode == BWD_PLIF) return launch_pieces_kernel<S, ROUND_EACH, BWD_PLIF>(f, b, *pieces, block, lds, blocks, stream);
    if (mode == BWD_QIF) return launch_pieces_kernel<S, ROUND_EACH, BWD_QIF>(f, b, *pieces, block, lds, blocks, stream);
    return launch_pieces_kernel<S, ROUND_EACH, BWD_PLAIN>(f, b, *pieces, block, lds, blocks, stream);
  }
  if (b.T <= kShortSequence) {
    if (mode == BWD_PLIF) return launch_kernel<S, ROUND_EACH, BWD_PLIF | BWD_SHORT>(f, b, block, lds, blocks, stream);
    if (mode == BWD_QIF) return launch_kernel<S, ROUND_EACH, BWD_QIF | BWD_SHORT>(f, b, block, lds, blocks, stream);
    return launch_kernel<S, ROUND_EACH, BWD_PLAIN | BWD_SHORT>(f, b, block, lds, blocks, stream);
  }
  if (mode == BWD_PLIF) return launch_kernel<S, ROUND_EACH, BWD_PLIF>(f, b, block, lds, blocks, stream);
  if (mode == BWD_QIF) return launch_kernel<S, ROUND_EACH, BWD_QIF>(f, b, block, lds, blocks, stream);
  return launch_kernel<S, ROUND_EACH, BWD_PLAIN>(f, b, block, lds, blocks, stream);
}

template <typename S>
int launch_recompute_dtype(const FwdArgs &f, const BwdArgs &b, bool round_each, int mode, int block, unsigned lds,
                           int64_t blocks, hipStream_t stream, const PieceArgs *pieces) {
  // the 8-byte access tags exist for fp32 state only
  if constexpr (std::is_same<S, f16_t>::value || std::is_same<S, bf16_t>::value) {
    if (round_each) return launch_mode<S, true>(f, b, mode, block, lds, blocks, stream, pieces);
  }
  return launch_mode<S, false>(f, b, mode, block, lds, blocks, stream, pieces);
}

}  // namespace sjhip
