// C ABI of libsjhip.so (declared in include/sjhip.h): argument validation, thread-local error
// text, launch tuning and the optional event profiler.  No entry point allocates device memory or
// synchronises the host (sjhip_profile_read excepted, which waits for the events it reports on).
#include "sjhip_common.h"

#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

namespace sjhip {

namespace {

thread_local char g_error[512] = "";

struct TuningStore {
  std::atomic<int> fwd_block{128};
  std::atomic<int> bwd_block{128};
  // Measured on MI355X at T=16, N=33.5M fp32: 2 blocks of 128 per compute unit (one wavefront per
  // SIMD) with 8 rows prefetched beat full occupancy by 7 % forward and 7 % backward.
  std::atomic<int> fwd_blocks_per_cu{2};
  std::atomic<int> bwd_blocks_per_cu{2};
  // The replay backward has two phases per wavefront (recompute h, then BPTT) and needs more waves
  // in flight to overlap them: uncapped (8 waves per CU at T=16 fp32) measured 15 % faster than 2 blocks.
  std::atomic<int> replay_blocks_per_cu{0};
  std::atomic<int> column_spread{2};
};
TuningStore g_tuning;

struct EventPair {
  hipEvent_t start, stop;
  int kc;
};
std::mutex g_prof_mutex;
std::atomic<int> g_prof_on{0};
std::vector<EventPair> g_prof_pending;
int64_t g_prof_count[KC_COUNT] = {0};
double g_prof_ms[KC_COUNT] = {0};
constexpr size_t kMaxPending = 4096;

// caller holds g_prof_mutex
void drain_pending() {
  for (EventPair &e : g_prof_pending) {
    float ms = 0.0f;
    if (hipEventSynchronize(e.stop) == hipSuccess && hipEventElapsedTime(&ms, e.start, e.stop) == hipSuccess) {
      g_prof_count[e.kc] += 1;
      g_prof_ms[e.kc] += (double)ms;
    }
    (void)hipEventDestroy(e.start);
    (void)hipEventDestroy(e.stop);
  }
  g_prof_pending.clear();
}

}  // namespace

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(SJHIP_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return SJHIP_OK;
}

const Tuning &tuning() {
  thread_local Tuning t;
  t.fwd_block = g_tuning.fwd_block.load(std::memory_order_relaxed);
  t.bwd_block = g_tuning.bwd_block.load(std::memory_order_relaxed);
  t.fwd_blocks_per_cu = g_tuning.fwd_blocks_per_cu.load(std::memory_order_relaxed);
  t.bwd_blocks_per_cu = g_tuning.bwd_blocks_per_cu.load(std::memory_order_relaxed);
  t.replay_blocks_per_cu = g_tuning.replay_blocks_per_cu.load(std::memory_order_relaxed);
  t.column_spread = g_tuning.column_spread.load(std::memory_order_relaxed);
  return t;
}

unsigned occupancy_cap_lds(int blocks_per_cu) {
  // gfx950 has 160 KiB of LDS per compute unit and a block may ask for at most 64 KiB of it:
  // asking for floor(160 KiB / n) (in 512-byte granules) lets exactly n blocks be resident.
  if (blocks_per_cu <= 0) return 0;
  const unsigned total = 160u * 1024u;
  unsigned bytes = (total / (unsigned)blocks_per_cu) & ~511u;
  if (bytes > 64u * 1024u) bytes = 64u * 1024u;
  return bytes;
}

ProfileScope::ProfileScope(int kernel_class, hipStream_t stream)
    : kc_(kernel_class), stream_(stream), start_(nullptr), active_(false) {
  if (!g_prof_on.load(std::memory_order_relaxed)) return;
  if (hipEventCreate(&start_) != hipSuccess) return;
  if (hipEventRecord(start_, stream_) != hipSuccess) { (void)hipEventDestroy(start_); return; }
  active_ = true;
}

ProfileScope::~ProfileScope() {
  if (!active_) return;
  hipEvent_t stop;
  if (hipEventCreate(&stop) != hipSuccess) { (void)hipEventDestroy(start_); return; }
  (void)hipEventRecord(stop, stream_);
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  g_prof_pending.push_back(EventPair{start_, stop, kc_});
  if (g_prof_pending.size() >= kMaxPending) drain_pending();
}

}  // namespace sjhip

using namespace sjhip;

// Workspace of sjhip_neuron_backward_static: the per-block partial sums of the PLIF dL/dk reduction, held in
// the code object instead of in memory a caller allocated.  4 MiB on every GPU the library runs on, for as long as the
// process lives.  In host code the array's name is only a handle for hipGetSymbolAddress; kernels get the address
// that call returned.
constexpr int64_t kStaticWorkspaceFloats = int64_t(1) << 20;
static_assert(kStaticWorkspaceFloats * 64 == SJHIP_STATIC_WORKSPACE_MAX_NEURONS, "plif_blocks() counts one partial per 64 neurons at most");
static __device__ __align__(256) float scratch[kStaticWorkspaceFloats];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float *g_scratch_ptr[kMaxDevices] = {nullptr};
// Every call on a device shares that device's array, so two calls whose kernels overlap would corrupt each other's
// partial sums.  Calls on one stream are ordered; a call on another stream is refused while the last call's work has not
// finished.  `g_scratch_done` is recorded behind every launch that uses the array (made once per device, beside the
// address look-up); a stream that is being captured into a graph records and checks nothing (the caller orders the
// graph's replays).
hipEvent_t g_scratch_done[kMaxDevices] = {nullptr};
hipStream_t g_scratch_stream[kMaxDevices] = {nullptr};
bool g_scratch_used[kMaxDevices] = {false};

bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

// Device address of `scratch` on the current device, looked up once per device; refuses a call on `stream` while a call
// made on another stream of the device is still running.
int static_workspace(const char *what, hipStream_t stream, float **out, int *device) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(SJHIP_ERR_LAUNCH, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(SJHIP_ERR_UNSUPPORTED, "%s: device ordinal %d", what, dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    float *ptr = nullptr;
    e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return fail(SJHIP_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) on device %d: %s", what, dev, hipGetErrorString(e));
    e = hipEventCreateWithFlags(&g_scratch_done[dev], hipEventDisableTiming);
    if (e != hipSuccess) return fail(SJHIP_ERR_LAUNCH, "%s: hipEventCreateWithFlags on device %d: %s", what, dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  if (g_scratch_used[dev] && g_scratch_stream[dev] != stream && !stream_is_capturing(stream)) {
    e = hipEventQuery(g_scratch_done[dev]);
    if (e == hipErrorNotReady)
      return fail(SJHIP_ERR_INVALID, "%s: the built-in workspace of device %d is in use by a call on another stream that has not "
                  "finished; order the calls (one stream, or an event between them)", what, dev);
    if (e != hipSuccess) (void)hipGetLastError();
  }
  *out = g_scratch_ptr[dev];
  *device = dev;
  return SJHIP_OK;
}

// After the launch that uses the array: remember the stream and when its work ends.
void static_workspace_launched(int dev, hipStream_t stream) {
  if (stream_is_capturing(stream)) return;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (hipEventRecord(g_scratch_done[dev], stream) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  g_scratch_stream[dev] = stream;
  g_scratch_used[dev] = true;
}

bool valid_dtype_fp(int dtype) { return dtype == SJHIP_F32 || dtype == SJHIP_F16 || dtype == SJHIP_BF16; }

// ILIF: the count limit must be a positive integer that every storage dtype holds exactly (bf16: up to 256)
int check_levels(const char *what, int neuron, const sjhip_neuron_params &p, bool backward) {
  if (neuron == SJHIP_NEURON_EIF && (!(p.a0 > 0.0f) || !std::isfinite(p.a0)))
    return fail(SJHIP_ERR_INVALID, "%s: EIF delta_T=%g must be positive", what, (double)p.a0);
  if (neuron != SJHIP_NEURON_ILIF) {
    if (backward && p.sg_id == SJHIP_SG_MULTI_LEVEL) return fail(SJHIP_ERR_INVALID, "%s: the multi-level surrogate belongs to ILIF", what);
    return SJHIP_OK;
  }
  if (!(p.level_max >= 1.0f) || p.level_max > 256.0f || p.level_max != std::floor(p.level_max))
    return fail(SJHIP_ERR_INVALID, "%s: ILIF level_max=%g must be an integer in [1, 256]", what, (double)p.level_max);
  if (!(p.v_threshold > 0.0f) || !std::isfinite(p.v_threshold))
    return fail(SJHIP_ERR_INVALID, "%s: ILIF v_threshold=%g must be positive", what, (double)p.v_threshold);
  if (backward) {
    if (p.sg_id != SJHIP_SG_MULTI_LEVEL) return fail(SJHIP_ERR_INVALID, "%s: ILIF needs the multi-level surrogate, got id %d", what, p.sg_id);
    if (!(p.grad_min <= p.grad_max)) return fail(SJHIP_ERR_INVALID, "%s: ILIF gradient window [%g, %g]", what, (double)p.grad_min, (double)p.grad_max);
  }
  return SJHIP_OK;
}

int check_shape(const char *what, int64_t T, int64_t N) {
  if (T < 1 || N < 1) return fail(SJHIP_ERR_INVALID, "%s: T=%lld N=%lld must be >= 1", what, (long long)T, (long long)N);
  if (T > (int64_t(1) << 62) / N) return fail(SJHIP_ERR_TOO_LARGE, "%s: T*N overflows", what);
  return SJHIP_OK;
}

}  // namespace

extern "C" {

int sjhip_abi_version(void) { return SJHIP_ABI_VERSION; }

const char *sjhip_last_error(void) { return g_error; }

int sjhip_neuron_forward(int neuron, int dtype, const sjhip_neuron_params *p, int64_t T, int64_t N,
                         const void *x_seq, const void *v_init, const float *rtau_device, void *spike_seq,
                         void *v_seq, void *v_last, void *h_seq, void *stream) {
  if (!p) return fail(SJHIP_ERR_INVALID, "forward: params is NULL");
  if (neuron < SJHIP_NEURON_IF || neuron > SJHIP_NEURON_EIF) return fail(SJHIP_ERR_INVALID, "forward: neuron %d", neuron);
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "forward: dtype %d", dtype);
  int rc = check_shape("forward", T, N);
  if (rc != SJHIP_OK) return rc;
  if (!x_seq || !v_init || !spike_seq) return fail(SJHIP_ERR_INVALID, "forward: NULL tensor");
  if (!v_seq && !v_last) return fail(SJHIP_ERR_INVALID, "forward: neither v_seq nor v_last given");
  rc = check_levels("forward", neuron, *p, false);
  if (rc != SJHIP_OK) return rc;
  if (neuron == SJHIP_NEURON_PLIF && !rtau_device) return fail(SJHIP_ERR_INVALID, "forward: PLIF needs rtau_device");
  return launch_forward(neuron, dtype, *p, T, N, x_seq, v_init, rtau_device, spike_seq, v_seq, v_last, h_seq,
                        static_cast<hipStream_t>(stream));
}

int sjhip_neuron_forward_packed(int neuron, int dtype, const sjhip_neuron_params *p, int64_t T, int64_t N,
                                const void *x_seq, const void *v_init, const float *rtau_device, uint8_t *spike_bits,
                                void *v_seq, void *v_last, void *stream) {
  if (!p) return fail(SJHIP_ERR_INVALID, "forward_packed: params is NULL");
  if (neuron < SJHIP_NEURON_IF || neuron > SJHIP_NEURON_EIF) return fail(SJHIP_ERR_INVALID, "forward_packed: neuron %d", neuron);
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "forward_packed: dtype %d", dtype);
  int rc = check_shape("forward_packed", T, N);
  if (rc != SJHIP_OK) return rc;
  if (!x_seq || !v_init || !spike_bits) return fail(SJHIP_ERR_INVALID, "forward_packed: NULL tensor");
  if (!v_seq && !v_last) return fail(SJHIP_ERR_INVALID, "forward_packed: neither v_seq nor v_last given");
  if (neuron == SJHIP_NEURON_ILIF) return fail(SJHIP_ERR_UNSUPPORTED, "forward_packed: ILIF fires counts, not bits");
  if (neuron == SJHIP_NEURON_PLIF && !rtau_device) return fail(SJHIP_ERR_INVALID, "forward_packed: PLIF needs rtau_device");
  return launch_forward_packed(neuron, dtype, *p, T, N, x_seq, v_init, rtau_device, spike_bits, v_seq, v_last,
                               static_cast<hipStream_t>(stream));
}

int64_t sjhip_plif_workspace_floats(int dtype, int64_t N) {
  if (N < 1) return 0;
  return plif_blocks(dtype, N);
}

namespace {
// everything sjhip_neuron_backward checks except the workspace
int check_backward(int neuron, int dtype, const sjhip_neuron_params *p, int64_t T, int64_t N, const void *grad_spike_seq,
                   const void *h_seq, const void *v_init, const float *rtau_device, void *grad_x_seq, void *grad_v_init,
                   float *grad_rtau) {
  if (!p) return fail(SJHIP_ERR_INVALID, "backward: params is NULL");
  if (neuron < SJHIP_NEURON_IF || neuron > SJHIP_NEURON_EIF) return fail(SJHIP_ERR_INVALID, "backward: neuron %d", neuron);
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "backward: dtype %d", dtype);
  if (p->sg_id < SJHIP_SG_SIGMOID || p->sg_id > SJHIP_SG_MULTI_LEVEL) return fail(SJHIP_ERR_UNSUPPORTED, "backward: surrogate id %d", p->sg_id);
  int rc = check_shape("backward", T, N);
  if (rc != SJHIP_OK) return rc;
  if (!h_seq || !grad_x_seq) return fail(SJHIP_ERR_INVALID, "backward: NULL tensor");
  rc = check_levels("backward", neuron, *p, true);
  if (rc != SJHIP_OK) return rc;
  if ((neuron == SJHIP_NEURON_QIF || neuron == SJHIP_NEURON_EIF) && grad_v_init && !v_init)
    return fail(SJHIP_ERR_INVALID, "backward: QIF / EIF need v_init for grad_v_init");
  if (neuron == SJHIP_NEURON_PLIF && (!v_init || !grad_rtau || !rtau_device))
    return fail(SJHIP_ERR_INVALID, "backward: PLIF needs v_init, rtau_device and grad_rtau");
  return SJHIP_OK;
}
}  // namespace

int sjhip_neuron_backward(int neuron, int dtype, const sjhip_neuron_params *p, int64_t T, int64_t N,
                          const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                          const void *h_seq, const void *v_init,
                          const float *rtau_device, void *grad_x_seq, void *grad_v_init, float *grad_rtau,
                          float *workspace, void *stream) {
  int rc = check_backward(neuron, dtype, p, T, N, grad_spike_seq, h_seq, v_init, rtau_device, grad_x_seq, grad_v_init, grad_rtau);
  if (rc != SJHIP_OK) return rc;
  if (neuron == SJHIP_NEURON_PLIF && !(p->flags & SJHIP_FLAG_ATOMIC_REDUCE) && !workspace)
    return fail(SJHIP_ERR_INVALID, "backward: PLIF needs a workspace unless SJHIP_FLAG_ATOMIC_REDUCE");
  return launch_backward(neuron, dtype, *p, T, N, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, v_init, rtau_device, grad_x_seq,
                         grad_v_init, grad_rtau, workspace, static_cast<hipStream_t>(stream));
}

int sjhip_neuron_backward_static(int neuron, int dtype, const sjhip_neuron_params *p, int64_t T, int64_t N,
                                 const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                                 const void *h_seq, const void *v_init, const float *rtau_device, void *grad_x_seq,
                                 void *grad_v_init, float *grad_rtau, void *stream) {
  int rc = check_backward(neuron, dtype, p, T, N, grad_spike_seq, h_seq, v_init, rtau_device, grad_x_seq, grad_v_init, grad_rtau);
  if (rc != SJHIP_OK) return rc;
  float *workspace = nullptr;
  int device = 0;
  if (neuron == SJHIP_NEURON_PLIF && !(p->flags & SJHIP_FLAG_ATOMIC_REDUCE)) {
    if (plif_blocks(dtype, N) > kStaticWorkspaceFloats)
      return fail(SJHIP_ERR_TOO_LARGE, "backward(static): N=%lld needs %lld partial sums, the built-in workspace holds %lld "
                  "(N <= %lld); use sjhip_neuron_backward with a workspace of the caller's", (long long)N,
                  (long long)plif_blocks(dtype, N), (long long)kStaticWorkspaceFloats, (long long)(kStaticWorkspaceFloats * 64));
    rc = static_workspace("backward(static)", static_cast<hipStream_t>(stream), &workspace, &device);
    if (rc != SJHIP_OK) return rc;
  }
  rc = launch_backward(neuron, dtype, *p, T, N, grad_spike_seq, grad_v_seq, grad_v_last, h_seq, v_init, rtau_device, grad_x_seq,
                       grad_v_init, grad_rtau, workspace, static_cast<hipStream_t>(stream));
  if (rc == SJHIP_OK && workspace) static_workspace_launched(device, static_cast<hipStream_t>(stream));
  return rc;
}

namespace {
int check_mp(const char *what, int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params *p, int64_t T,
             int64_t N) {
  if (!p) return fail(SJHIP_ERR_INVALID, "%s: params is NULL", what);
  if (neuron < SJHIP_NEURON_IF || neuron > SJHIP_NEURON_PLIF) return fail(SJHIP_ERR_UNSUPPORTED, "%s: neuron %d (IF, LIF and PLIF only)", what, neuron);
  if (storage_dtype != SJHIP_F8E4M3 && storage_dtype != SJHIP_F8E5M2)
    return fail(SJHIP_ERR_INVALID, "%s: storage dtype %d is not an 8-bit float", what, storage_dtype);
  if (!valid_dtype_fp(spike_dtype)) return fail(SJHIP_ERR_INVALID, "%s: spike dtype %d", what, spike_dtype);
  return check_shape(what, T, N);
}
}  // namespace

int sjhip_neuron_forward_mp(int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params *p, int64_t T,
                            int64_t N, const void *x_seq, const void *v_init, const float *rtau_device, void *spike_seq,
                            void *v_seq, void *v_last, void *h_seq, void *stream) {
  int rc = check_mp("forward(mp)", neuron, storage_dtype, spike_dtype, p, T, N);
  if (rc != SJHIP_OK) return rc;
  if (!x_seq || !v_init || !spike_seq) return fail(SJHIP_ERR_INVALID, "forward(mp): NULL tensor");
  if (!v_seq && !v_last) return fail(SJHIP_ERR_INVALID, "forward(mp): neither v_seq nor v_last given");
  if (neuron == SJHIP_NEURON_PLIF && !rtau_device) return fail(SJHIP_ERR_INVALID, "forward(mp): PLIF needs rtau_device");
  return launch_forward_mp(neuron, storage_dtype, spike_dtype, *p, T, N, x_seq, v_init, rtau_device, spike_seq, v_seq,
                           v_last, h_seq, static_cast<hipStream_t>(stream));
}

int sjhip_neuron_backward_mp(int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params *p, int64_t T,
                             int64_t N, const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                             const void *h_seq, const void *v_init, const float *rtau_device, void *grad_x_seq,
                             void *grad_v_init, float *grad_rtau, float *workspace, void *stream) {
  int rc = check_mp("backward(mp)", neuron, storage_dtype, spike_dtype, p, T, N);
  if (rc != SJHIP_OK) return rc;
  if (p->sg_id < SJHIP_SG_SIGMOID || p->sg_id > SJHIP_SG_ERF) return fail(SJHIP_ERR_UNSUPPORTED, "backward(mp): surrogate id %d", p->sg_id);
  if (!grad_spike_seq || !h_seq || !grad_x_seq) return fail(SJHIP_ERR_INVALID, "backward(mp): NULL tensor");
  if (neuron == SJHIP_NEURON_PLIF) {
    if (!v_init || !grad_rtau || !rtau_device) return fail(SJHIP_ERR_INVALID, "backward(mp): PLIF needs v_init, rtau_device and grad_rtau");
    if (!(p->flags & SJHIP_FLAG_ATOMIC_REDUCE) && !workspace) return fail(SJHIP_ERR_INVALID, "backward(mp): PLIF needs a workspace unless SJHIP_FLAG_ATOMIC_REDUCE");
  }
  return launch_backward_mp(neuron, storage_dtype, spike_dtype, *p, T, N, grad_spike_seq, grad_v_seq, grad_v_last, h_seq,
                            v_init, rtau_device, grad_x_seq, grad_v_init, grad_rtau, workspace,
                            static_cast<hipStream_t>(stream));
}

int sjhip_recompute_supported(int dtype, int64_t T, int64_t N) {
  if (!valid_dtype_fp(dtype) || T < 1 || N < 1) return 0;
  return recompute_supported(dtype, T, N) ? 1 : 0;
}

int sjhip_recompute_preferred(int dtype, int64_t T, int64_t N, uint32_t flags) {
  if (!valid_dtype_fp(dtype) || T < 1 || N < 1) return 0;
  const bool round_each = dtype != SJHIP_F32 && !(flags & SJHIP_FLAG_FP32_STATE);
  return recompute_preferred(dtype, T, N, round_each) ? 1 : 0;
}

int sjhip_neuron_backward_recompute(int neuron, int dtype, const sjhip_neuron_params *p, int64_t T, int64_t N,
                                    const void *x_seq, const void *v_init, const float *rtau_device,
                                    const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                                    void *grad_x_seq, void *grad_v_init, float *grad_rtau, float *workspace,
                                    void *stream) {
  if (!p) return fail(SJHIP_ERR_INVALID, "backward(recompute): params is NULL");
  if (neuron < SJHIP_NEURON_IF || neuron > SJHIP_NEURON_EIF) return fail(SJHIP_ERR_INVALID, "backward(recompute): neuron %d", neuron);
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "backward(recompute): dtype %d", dtype);
  if (p->sg_id < SJHIP_SG_SIGMOID || p->sg_id > SJHIP_SG_MULTI_LEVEL) return fail(SJHIP_ERR_UNSUPPORTED, "backward(recompute): surrogate id %d", p->sg_id);
  int rc = check_shape("backward(recompute)", T, N);
  if (rc != SJHIP_OK) return rc;
  if (!x_seq || !v_init || !grad_x_seq) return fail(SJHIP_ERR_INVALID, "backward(recompute): NULL tensor");
  rc = check_levels("backward(recompute)", neuron, *p, true);
  if (rc != SJHIP_OK) return rc;
  if (neuron == SJHIP_NEURON_PLIF) {
    if (!grad_rtau || !rtau_device) return fail(SJHIP_ERR_INVALID, "backward(recompute): PLIF needs rtau_device and grad_rtau");
    if (!(p->flags & SJHIP_FLAG_ATOMIC_REDUCE) && !workspace) return fail(SJHIP_ERR_INVALID, "backward(recompute): PLIF needs a workspace unless SJHIP_FLAG_ATOMIC_REDUCE");
  }
  return launch_backward_recompute(neuron, dtype, *p, T, N, x_seq, v_init, rtau_device, grad_spike_seq, grad_v_seq,
                                   grad_v_last, grad_x_seq, grad_v_init, grad_rtau, workspace,
                                   static_cast<hipStream_t>(stream));
}

int64_t sjhip_replay_pieces(int64_t T, int64_t chunk) { return (T < 1 || chunk < 1) ? 0 : (T + chunk - 1) / chunk; }

int sjhip_neuron_forward_pieces(int neuron, int dtype, const sjhip_neuron_params *p, int64_t T, int64_t N, int64_t chunk,
                                const void *x_seq, const void *v_init, const float *rtau_device, void *spike_seq,
                                void *v_seq, void *v_last, void *checkpoints, void *stream) {
  if (!p) return fail(SJHIP_ERR_INVALID, "forward(pieces): params is NULL");
  if (neuron < SJHIP_NEURON_IF || neuron > SJHIP_NEURON_EIF) return fail(SJHIP_ERR_INVALID, "forward(pieces): neuron %d", neuron);
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "forward(pieces): dtype %d", dtype);
  int rc = check_shape("forward(pieces)", T, N);
  if (rc != SJHIP_OK) return rc;
  if (chunk < 1) return fail(SJHIP_ERR_INVALID, "forward(pieces): chunk %lld", (long long)chunk);
  if (!x_seq || !v_init || !spike_seq) return fail(SJHIP_ERR_INVALID, "forward(pieces): NULL tensor");
  if (!v_seq && !v_last) return fail(SJHIP_ERR_INVALID, "forward(pieces): neither v_seq nor v_last given");
  if (T > chunk && !checkpoints) return fail(SJHIP_ERR_INVALID, "forward(pieces): %lld pieces need checkpoints", (long long)sjhip_replay_pieces(T, chunk));
  rc = check_levels("forward(pieces)", neuron, *p, false);
  if (rc != SJHIP_OK) return rc;
  if (neuron == SJHIP_NEURON_PLIF && !rtau_device) return fail(SJHIP_ERR_INVALID, "forward(pieces): PLIF needs rtau_device");
  return launch_forward_pieces(neuron, dtype, *p, T, N, chunk, x_seq, v_init, rtau_device, spike_seq, v_seq, v_last, checkpoints,
                               static_cast<hipStream_t>(stream));
}

int sjhip_neuron_backward_recompute_pieces(int neuron, int dtype, const sjhip_neuron_params *p, int64_t T, int64_t N,
                                           int64_t chunk, const void *x_seq, const void *v_init, const float *rtau_device,
                                           const void *checkpoints, const void *grad_spike_seq, const void *grad_v_seq,
                                           const void *grad_v_last, void *grad_x_seq, void *grad_v_init, float *grad_rtau,
                                           float *workspace, void *stream) {
  if (!p) return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): params is NULL");
  if (neuron < SJHIP_NEURON_IF || neuron > SJHIP_NEURON_EIF) return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): neuron %d", neuron);
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): dtype %d", dtype);
  if (p->sg_id < SJHIP_SG_SIGMOID || p->sg_id > SJHIP_SG_MULTI_LEVEL) return fail(SJHIP_ERR_UNSUPPORTED, "backward(recompute, pieces): surrogate id %d", p->sg_id);
  int rc = check_shape("backward(recompute, pieces)", T, N);
  if (rc != SJHIP_OK) return rc;
  if (chunk < 1) return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): chunk %lld", (long long)chunk);
  if (!x_seq || !v_init || !grad_x_seq) return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): NULL tensor");
  if (T > chunk && !checkpoints) return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): several pieces need checkpoints");
  rc = check_levels("backward(recompute, pieces)", neuron, *p, true);
  if (rc != SJHIP_OK) return rc;
  if (neuron == SJHIP_NEURON_PLIF) {
    if (!grad_rtau || !rtau_device) return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): PLIF needs rtau_device and grad_rtau");
    if (!(p->flags & SJHIP_FLAG_ATOMIC_REDUCE) && !workspace) return fail(SJHIP_ERR_INVALID, "backward(recompute, pieces): PLIF needs a workspace unless SJHIP_FLAG_ATOMIC_REDUCE");
  }
  return launch_backward_recompute_pieces(neuron, dtype, *p, T, N, chunk, x_seq, v_init, rtau_device, checkpoints, grad_spike_seq,
                                          grad_v_seq, grad_v_last, grad_x_seq, grad_v_init, grad_rtau, workspace,
                                          static_cast<hipStream_t>(stream));
}

int sjhip_stbif_forward(int dtype, uint32_t flags, int64_t T, int64_t N, const void *x_seq, const void *q_init,
                        const void *acc_q_init, const float *q_threshold, const float *pos_max, const float *neg_min,
                        void *out_seq, void *q_final, void *acc_q_final, void *cur_output, int32_t *work_flag,
                        void *stream) {
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "stbif_forward: dtype %d", dtype);
  if (flags & ~(SJHIP_FLAG_FP32_STATE | SJHIP_FLAG_Q_BROADCAST | SJHIP_FLAG_ACC_BROADCAST))
    return fail(SJHIP_ERR_INVALID, "stbif_forward: flags 0x%x", flags);
  int rc = check_shape("stbif_forward", T, N);
  if (rc != SJHIP_OK) return rc;
  if (!x_seq || !q_init || !acc_q_init || !out_seq || !q_final || !acc_q_final || !cur_output)
    return fail(SJHIP_ERR_INVALID, "stbif_forward: NULL tensor");
  if (!q_threshold || !pos_max || !neg_min) return fail(SJHIP_ERR_INVALID, "stbif_forward: NULL scalar address");
  return launch_stbif_forward(dtype, flags, T, N, x_seq, q_init, acc_q_init, q_threshold, pos_max, neg_min, out_seq,
                              q_final, acc_q_final, cur_output, work_flag, static_cast<hipStream_t>(stream));
}

namespace {
int check_izhikevich(const char *what, int dtype, const sjhip_izhikevich_params *p, int64_t T, int64_t N, bool backward) {
  if (!p) return fail(SJHIP_ERR_INVALID, "%s: params is NULL", what);
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "%s: dtype %d", what, dtype);
  if (!(p->tau > 0.0f) || !std::isfinite(p->tau) || !(p->tau_w > 0.0f) || !std::isfinite(p->tau_w))
    return fail(SJHIP_ERR_INVALID, "%s: tau=%g tau_w=%g must be positive", what, (double)p->tau, (double)p->tau_w);
  if (backward && (p->sg_id < SJHIP_SG_SIGMOID || p->sg_id > SJHIP_SG_ERF))
    return fail(SJHIP_ERR_UNSUPPORTED, "%s: surrogate id %d", what, p->sg_id);
  const uint32_t known = SJHIP_FLAG_SOFT_RESET | SJHIP_FLAG_DETACH_RESET | SJHIP_FLAG_FP32_STATE |
                         SJHIP_FLAG_V_INIT_BROADCAST | SJHIP_FLAG_W_INIT_BROADCAST;
  if (p->flags & ~known) return fail(SJHIP_ERR_INVALID, "%s: flags 0x%x", what, p->flags);
  return check_shape(what, T, N);
}
}  // namespace

int sjhip_izhikevich_forward(int dtype, const sjhip_izhikevich_params *p, int64_t T, int64_t N, const void *x_seq,
                             const void *v_init, const void *w_init, void *spike_seq, void *v_seq, void *w_seq,
                             void *v_last, void *w_last, void *h_seq, void *stream) {
  int rc = check_izhikevich("izhikevich_forward", dtype, p, T, N, false);
  if (rc != SJHIP_OK) return rc;
  if (!x_seq || !v_init || !w_init || !spike_seq || !v_last || !w_last)
    return fail(SJHIP_ERR_INVALID, "izhikevich_forward: NULL tensor");
  return launch_izhikevich_forward(dtype, *p, T, N, x_seq, v_init, w_init, spike_seq, v_seq, w_seq, v_last, w_last, h_seq,
                                   static_cast<hipStream_t>(stream));
}

int sjhip_izhikevich_backward(int dtype, const sjhip_izhikevich_params *p, int64_t T, int64_t N,
                              const void *grad_spike_seq, const void *grad_v_seq, const void *grad_w_seq,
                              const void *grad_v_last, const void *grad_w_last, const void *h_seq, const void *v_init,
                              void *grad_x_seq, void *grad_v_init, void *grad_w_init, void *stream) {
  int rc = check_izhikevich("izhikevich_backward", dtype, p, T, N, true);
  if (rc != SJHIP_OK) return rc;
  if (!grad_spike_seq || !h_seq || !grad_x_seq) return fail(SJHIP_ERR_INVALID, "izhikevich_backward: NULL tensor");
  if (grad_v_init && !v_init) return fail(SJHIP_ERR_INVALID, "izhikevich_backward: grad_v_init needs v_init");
  return launch_izhikevich_backward(dtype, *p, T, N, grad_spike_seq, grad_v_seq, grad_w_seq, grad_v_last, grad_w_last, h_seq,
                                    v_init, grad_x_seq, grad_v_init, grad_w_init, static_cast<hipStream_t>(stream));
}

int sjhip_izhikevich_backward_replay(int dtype, const sjhip_izhikevich_params *p, int64_t T, int64_t N, const void *x_seq,
                                     const void *v_init, const void *w_init, const void *grad_spike_seq,
                                     const void *grad_v_seq, const void *grad_w_seq, const void *grad_v_last,
                                     const void *grad_w_last, void *grad_x_seq, void *grad_v_init, void *grad_w_init,
                                     void *stream) {
  int rc = check_izhikevich("izhikevich_backward(replay)", dtype, p, T, N, true);
  if (rc != SJHIP_OK) return rc;
  if (!x_seq || !v_init || !w_init || !grad_spike_seq || !grad_x_seq)
    return fail(SJHIP_ERR_INVALID, "izhikevich_backward(replay): NULL tensor");
  return launch_izhikevich_backward_replay(dtype, *p, T, N, x_seq, v_init, w_init, grad_spike_seq, grad_v_seq, grad_w_seq,
                                           grad_v_last, grad_w_last, grad_x_seq, grad_v_init, grad_w_init,
                                           static_cast<hipStream_t>(stream));
}

int sjhip_aaif_forward(int dtype, uint32_t flags, int64_t T, int64_t N, const void *x_seq, const void *v_init,
                       const float *v_threshold, int64_t threshold_count, const float *v_offset, int64_t offset_count,
                       int64_t channel_size, int64_t inner_size, float v_reset, void *spike_seq, void *v_seq,
                       void *v_last, void *stream) {
  if (!valid_dtype_fp(dtype)) return fail(SJHIP_ERR_INVALID, "aaif_forward: dtype %d", dtype);
  if (flags & ~(SJHIP_FLAG_SOFT_RESET | SJHIP_FLAG_FP32_STATE | SJHIP_FLAG_V_INIT_BROADCAST))
    return fail(SJHIP_ERR_INVALID, "aaif_forward: flags 0x%x", flags);
  int rc = check_shape("aaif_forward", T, N);
  if (rc != SJHIP_OK) return rc;
  if (!x_seq || !v_init || !spike_seq || !v_threshold || !v_offset) return fail(SJHIP_ERR_INVALID, "aaif_forward: NULL tensor");
  if (!v_seq && !v_last) return fail(SJHIP_ERR_INVALID, "aaif_forward: neither v_seq nor v_last given");
  if (channel_size < 1 || inner_size < 1 || channel_size > N || inner_size > N)
    return fail(SJHIP_ERR_INVALID, "aaif_forward: channel_size=%lld inner_size=%lld for N=%lld", (long long)channel_size,
                (long long)inner_size, (long long)N);
  if ((threshold_count != 1 && threshold_count != channel_size) || (offset_count != 1 && offset_count != channel_size))
    return fail(SJHIP_ERR_INVALID, "aaif_forward: %lld thresholds and %lld offsets for %lld channels",
                (long long)threshold_count, (long long)offset_count, (long long)channel_size);
  return launch_aaif_forward(dtype, flags, T, N, x_seq, v_init, v_threshold, threshold_count, v_offset, offset_count,
                             channel_size, inner_size, v_reset, spike_seq, v_seq, v_last, static_cast<hipStream_t>(stream));
}

int sjhip_bit_pack(int dtype, int64_t n, const void *src, uint8_t *dst, void *stream) {
  if (n < 0) return fail(SJHIP_ERR_INVALID, "bit_pack: n=%lld", (long long)n);
  if (n == 0) return SJHIP_OK;
  if (!src || !dst) return fail(SJHIP_ERR_INVALID, "bit_pack: NULL buffer");
  return launch_bit_pack(dtype, n, src, dst, static_cast<hipStream_t>(stream));
}

int sjhip_bit_unpack(int dtype, int64_t n, const uint8_t *src, void *dst, void *stream) {
  if (n < 0) return fail(SJHIP_ERR_INVALID, "bit_unpack: n=%lld", (long long)n);
  if (n == 0) return SJHIP_OK;
  if (!src || !dst) return fail(SJHIP_ERR_INVALID, "bit_unpack: NULL buffer");
  return launch_bit_unpack(dtype, n, src, dst, static_cast<hipStream_t>(stream));
}

int sjhip_ssa_supported(int dtype, int channels_per_head, int64_t tokens) {
  return ssa_supported(dtype, channels_per_head, tokens) ? 1 : 0;
}

int sjhip_ssa_forward(int dtype, int64_t samples, int heads, int channels_per_head, int64_t tokens, float scale,
                      const void *qkv, void *out, void *stream) {
  if (!qkv || !out) return fail(SJHIP_ERR_INVALID, "ssa_forward: NULL tensor");
  return launch_ssa(false, dtype, samples, heads, channels_per_head, tokens, scale, qkv, nullptr, nullptr, out, nullptr,
                    static_cast<hipStream_t>(stream));
}

int sjhip_ssa_forward_packed(int dtype, int64_t samples, int heads, int channels_per_head, int64_t tokens, float scale,
                             const uint8_t *qkv_bits, void *out, void *stream) {
  if (!qkv_bits || !out) return fail(SJHIP_ERR_INVALID, "ssa_forward_packed: NULL tensor");
  return launch_ssa(false, dtype, samples, heads, channels_per_head, tokens, scale, nullptr, qkv_bits, nullptr, out, nullptr,
                    static_cast<hipStream_t>(stream));
}

int sjhip_ssa_backward_packed(int dtype, int64_t samples, int heads, int channels_per_head, int64_t tokens, float scale,
                              const uint8_t *qkv_bits, const void *grad_out, void *grad_qkv, void *stream) {
  if (!qkv_bits || !grad_out || !grad_qkv) return fail(SJHIP_ERR_INVALID, "ssa_backward_packed: NULL tensor");
  return launch_ssa(true, dtype, samples, heads, channels_per_head, tokens, scale, nullptr, qkv_bits, grad_out, nullptr,
                    grad_qkv, static_cast<hipStream_t>(stream));
}

int sjhip_ssa_backward(int dtype, int64_t samples, int heads, int channels_per_head, int64_t tokens, float scale,
                       const void *qkv, const void *grad_out, void *grad_qkv, void *stream) {
  if (!qkv || !grad_out || !grad_qkv) return fail(SJHIP_ERR_INVALID, "ssa_backward: NULL tensor");
  return launch_ssa(true, dtype, samples, heads, channels_per_head, tokens, scale, qkv, nullptr, grad_out, nullptr, grad_qkv,
                    static_cast<hipStream_t>(stream));
}

int sjhip_ssa_lif_forward_packed(int neuron, const sjhip_neuron_params *p, int64_t T, int64_t B, int heads, int channels_per_head,
                                 int64_t tokens, float scale, const uint8_t *qkv_bits, const float *v_init, float *spike_seq,
                                 float *h_seq, float *v_last, void *stream) {
  if (!p) return fail(SJHIP_ERR_INVALID, "ssa_lif_forward: params is NULL");
  if (!qkv_bits || !v_init || !spike_seq) return fail(SJHIP_ERR_INVALID, "ssa_lif_forward: NULL tensor");
  return launch_ssa_lif(false, neuron, *p, T, B, heads, channels_per_head, tokens, scale, qkv_bits, v_init, spike_seq, h_seq,
                        v_last, nullptr, nullptr, nullptr, nullptr, static_cast<hipStream_t>(stream));
}

int sjhip_ssa_lif_backward_packed(int neuron, const sjhip_neuron_params *p, int64_t T, int64_t B, int heads,
                                  int channels_per_head, int64_t tokens, float scale, const uint8_t *qkv_bits,
                                  const float *h_seq, const float *grad_spike_seq, const float *grad_v_last, float *grad_qkv,
                                  float *grad_v_init, void *stream) {
  if (!p) return fail(SJHIP_ERR_INVALID, "ssa_lif_backward: params is NULL");
  if (!qkv_bits || !h_seq || !grad_qkv) return fail(SJHIP_ERR_INVALID, "ssa_lif_backward: NULL tensor");
  if (p->sg_id < SJHIP_SG_SIGMOID || p->sg_id > SJHIP_SG_ERF) return fail(SJHIP_ERR_UNSUPPORTED, "ssa_lif_backward: surrogate id %d", p->sg_id);
  return launch_ssa_lif(true, neuron, *p, T, B, heads, channels_per_head, tokens, scale, qkv_bits, nullptr,
                        nullptr, const_cast<float *>(h_seq), nullptr, grad_spike_seq, grad_v_last, grad_qkv, grad_v_init,
                        static_cast<hipStream_t>(stream));
}

int sjhip_stream_probe(int reads, int writes, int nontemporal, int64_t floats_per_stream, const float *const *in,
                       float *const *out, void *stream) {
  return launch_stream_probe(reads, writes, nontemporal, floats_per_stream, in, out, static_cast<hipStream_t>(stream));
}

int64_t sjhip_mfma_probe_blocks(int wavefronts_per_simd) {
  return wavefronts_per_simd >= 1 && wavefronts_per_simd <= 8 ? mfma_probe_blocks(wavefronts_per_simd) : 0;
}

int sjhip_mfma_probe(int operands, int wavefronts_per_simd, int iterations, float *sink, int64_t sink_floats, void *stream) {
  return launch_mfma_probe(operands, wavefronts_per_simd, iterations, sink, sink_floats, static_cast<hipStream_t>(stream));
}

int64_t sjhip_pwconv_planes_elems(int64_t rows, int64_t cols) {
  if (rows < 1 || cols < 1) return 0;
  return pwconv_planes_elems(rows, cols);
}

int sjhip_pwconv_split_weight(const float *w, int64_t rows, int64_t cols, int transpose, uint16_t *planes, void *stream) {
  if (!w || !planes) return fail(SJHIP_ERR_INVALID, "pwconv_split_weight: NULL buffer");
  if (rows < 1 || cols < 1) return fail(SJHIP_ERR_INVALID, "pwconv_split_weight: %lld x %lld", (long long)rows, (long long)cols);
  return launch_pwconv_split_weight(w, rows, cols, transpose, planes, static_cast<hipStream_t>(stream));
}

int sjhip_pwconv_gemm(const uint16_t *a_planes, int a_terms, int64_t M, int64_t K, const float *b, int b_terms, int64_t S,
                      int64_t L, float *c, void *stream) {
  if (!a_planes || !b || !c) return fail(SJHIP_ERR_INVALID, "pwconv_gemm: NULL buffer");
  if (M < 1 || K < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_gemm: M=%lld K=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)K, (long long)S, (long long)L);
  if (S > (int64_t(1) << 40) / L) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm: S*L overflows");
  if (a_terms < 1 || a_terms > 3) return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_gemm: %d weight terms (1 to 3 bf16 terms; fp16 planes belong to sjhip_pwconv_gemm_f16)", a_terms);
  return launch_pwconv_gemm(a_planes, a_terms, M, K, b, b_terms, nullptr, S, L, c, nullptr, static_cast<hipStream_t>(stream));
}

int64_t sjhip_pwconv_gemm_stats_rows(int64_t K, int64_t S, int64_t L) {
  if (K < 1 || S < 1 || L < 1 || S > (int64_t(1) << 40) / L) return 0;
  return pwconv_gemm_stats_rows(K, S, L);
}

int sjhip_pwconv_gemm_stats(const uint16_t *a_planes, int a_terms, int64_t M, int64_t K, const float *b, int b_terms, int64_t S,
                            int64_t L, float *c, float *partial, void *stream) {
  if (!a_planes || !b || !c || !partial) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_stats: NULL buffer");
  if (M < 1 || K < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_stats: M=%lld K=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)K, (long long)S, (long long)L);
  if (S > (int64_t(1) << 40) / L) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm_stats: S*L overflows");
  if (a_terms < 1 || a_terms > 3) return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_gemm_stats: %d weight terms (1 to 3 bf16 terms; fp16 planes belong to sjhip_pwconv_gemm_f16)", a_terms);
  return launch_pwconv_gemm(a_planes, a_terms, M, K, b, b_terms, nullptr, S, L, c, partial, static_cast<hipStream_t>(stream));
}

int64_t sjhip_pwconv_grad_weight_workspace_floats(int64_t M, int64_t N, int64_t S) {
  if (M < 1 || N < 1 || S < 1) return 0;
  return pwconv_dw_workspace_floats(M, N, S);
}

int sjhip_pwconv_grad_weight(const float *dy, int dy_terms, const float *x, int x_terms, int64_t S, int64_t M, int64_t N,
                             int64_t L, float *dw, float *workspace, void *stream) {
  if (!dy || !x || !dw || !workspace) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight: NULL buffer");
  if (M < 1 || N < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight: M=%lld N=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)N, (long long)S, (long long)L);
  if (dy_terms < 1 || dy_terms > 3) return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_grad_weight: %d gradient terms (1 to 3 bf16 terms)", dy_terms);
  return launch_pwconv_grad_weight(dy, dy_terms, nullptr, x, x_terms, nullptr, S, M, N, L, dw, workspace, static_cast<hipStream_t>(stream));
}

int64_t sjhip_pwconv_amax_floats(int64_t S) { return S < 0 ? 0 : SJHIP_PW_AMAX_FLOATS + SJHIP_PW_AMAX_SAMPLE_WORDS * S; }

int sjhip_pwconv_split_weight_f16(const float *w, int64_t rows, int64_t cols, int transpose, uint16_t *planes, float *amax_reset,
                                  int64_t amax_reset_samples, void *stream) {
  if (!w || !planes) return fail(SJHIP_ERR_INVALID, "pwconv_split_weight_f16: NULL buffer");
  if (rows < 1 || cols < 1) return fail(SJHIP_ERR_INVALID, "pwconv_split_weight_f16: %lld x %lld", (long long)rows, (long long)cols);
  if (!aligned16(planes)) return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_split_weight_f16: the planes must be 16-byte aligned");
  if (amax_reset && amax_reset_samples < 0) return fail(SJHIP_ERR_INVALID, "pwconv_split_weight_f16: amax_reset_samples=%lld", (long long)amax_reset_samples);
  return launch_pwconv_split_weight_f16(w, rows, cols, transpose, planes, amax_reset, SJHIP_PW_AMAX_FLOATS + SJHIP_PW_AMAX_SAMPLE_WORDS * amax_reset_samples,
                                        static_cast<hipStream_t>(stream));
}

int sjhip_pwconv_amax(const float *x, int64_t S, int64_t per_sample, float *amax, void *stream) {
  if (!x || !amax) return fail(SJHIP_ERR_INVALID, "pwconv_amax: NULL buffer");
  if (S < 1 || per_sample < 1 || S > (int64_t(1) << 40) / per_sample)
    return fail(SJHIP_ERR_INVALID, "pwconv_amax: S=%lld samples of per_sample=%lld elements", (long long)S, (long long)per_sample);
  return launch_pwconv_amax(x, S, per_sample, amax, static_cast<hipStream_t>(stream));
}

int sjhip_pwconv_gemm_f16(const uint16_t *a_planes, int64_t M, int64_t K, const float *b, int b_terms, const float *b_amax,
                          int64_t S, int64_t L, float *c, float *partial, void *stream) {
  if (!a_planes || !b || !c) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_f16: NULL buffer");
  if (M < 1 || K < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_f16: M=%lld K=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)K, (long long)S, (long long)L);
  if (S > (int64_t(1) << 40) / L) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm_f16: S*L overflows");
  if (b_terms != 1 && b_terms != 2) return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_gemm_f16: %d activation terms (1 or 2)", b_terms);
  if (b_terms == 2 && !b_amax) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_f16: two activation terms need the largest magnitude from sjhip_pwconv_amax");
  if (b_terms == 2 && !aligned16(b_amax)) return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_gemm_f16: the amax buffer must be 16-byte aligned");
  return launch_pwconv_gemm(a_planes, SJHIP_PW_F16 | 2, M, K, b, b_terms, b_terms == 2 ? b_amax : nullptr, S, L, c, partial,
                            static_cast<hipStream_t>(stream));
}

int sjhip_pwconv_grad_weight_f16(const float *dy, const float *dy_amax, const float *x, int x_terms, const float *x_amax,
                                 int64_t S, int64_t M, int64_t N, int64_t L, float *dw, float *workspace, void *stream) {
  if (!dy || !dy_amax || !x || !dw || !workspace) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight_f16: NULL buffer");
  if (M < 1 || N < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight_f16: M=%lld N=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)N, (long long)S, (long long)L);
  if (x_terms != 1 && x_terms != 2) return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_grad_weight_f16: %d activation terms (1 or 2)", x_terms);
  if (x_terms == 2 && !x_amax) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight_f16: two activation terms need the largest magnitude from sjhip_pwconv_amax");
  if (!aligned16(dy_amax) || (x_terms == 2 && !aligned16(x_amax)))
    return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_grad_weight_f16: the amax buffers must be 16-byte aligned");
  return launch_pwconv_grad_weight(dy, SJHIP_PW_F16 | 2, dy_amax, x, x_terms, x_terms == 2 ? x_amax : nullptr, S, M, N, L, dw,
                                   workspace, static_cast<hipStream_t>(stream));
}

int sjhip_pwconv_gemm_f16_bits(const uint16_t *a_planes, int64_t M, int64_t K, const uint8_t *b_bits, int64_t S, int64_t L,
                               float *c, float *partial, void *stream) {
  if (!a_planes || !b_bits || !c) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_f16_bits: NULL buffer");
  if (M < 1 || K < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_f16_bits: M=%lld K=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)K, (long long)S, (long long)L);
  if (S > (int64_t(1) << 40) / L) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm_f16_bits: S*L overflows");
  return launch_pwconv_gemm(a_planes, SJHIP_PW_F16 | 2, M, K, reinterpret_cast<const float *>(b_bits), 1, nullptr, S, L, c, partial,
                            static_cast<hipStream_t>(stream), true);
}

int sjhip_pwconv_grad_weight_f16_bits(const float *dy, const float *dy_amax, const uint8_t *x_bits, int64_t S, int64_t M,
                                      int64_t N, int64_t L, float *dw, float *workspace, void *stream) {
  if (!dy || !dy_amax || !x_bits || !dw || !workspace) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight_f16_bits: NULL buffer");
  if (M < 1 || N < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight_f16_bits: M=%lld N=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)N, (long long)S, (long long)L);
  if (!aligned16(dy_amax)) return fail(SJHIP_ERR_UNSUPPORTED, "pwconv_grad_weight_f16_bits: the amax buffer must be 16-byte aligned");
  return launch_pwconv_grad_weight(dy, SJHIP_PW_F16 | 2, dy_amax, reinterpret_cast<const float *>(x_bits), 1, nullptr, S, M, N, L, dw,
                                   workspace, static_cast<hipStream_t>(stream), true);
}

int64_t sjhip_pwconv_plane_elems(int64_t S, int64_t C, int64_t L, int terms) {
  if (S < 1 || C < 1 || L < 1 || terms < 1 || terms > 2 || S > (int64_t(1) << 40) / L) return 0;
  return terms * C * pwconv_plane_ld(S, L);
}

int sjhip_pwconv_split_planes(const float *x, int64_t S, int64_t C, int64_t L, int terms, const float *amax, uint16_t *planes,
                              void *stream) {
  if (!x || !planes) return fail(SJHIP_ERR_INVALID, "pwconv_split_planes: NULL buffer");
  if (S < 1 || C < 1 || L < 1 || S > (int64_t(1) << 40) / L) return fail(SJHIP_ERR_INVALID, "pwconv_split_planes: S=%lld C=%lld L=%lld", (long long)S, (long long)C, (long long)L);
  return launch_pwconv_split_planes(x, S, C, L, terms, amax, planes, static_cast<hipStream_t>(stream));
}

int64_t sjhip_pwconv_gemm_planes_stats_rows(int64_t S, int64_t L) {
  if (S < 1 || L < 1 || S > (int64_t(1) << 40) / L) return 0;
  return pwconv_gemm_planes_stats_rows(S, L);
}

int sjhip_pwconv_gemm_planes(const uint16_t *a_planes, int64_t M, int64_t K, const uint16_t *b_planes, int b_terms,
                             const float *b_amax, int64_t S, int64_t L, float *c, float *partial, void *stream) {
  if (!a_planes || !b_planes || !c) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_planes: NULL buffer");
  if (M < 1 || K < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_gemm_planes: M=%lld K=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)K, (long long)S, (long long)L);
  if (S > (int64_t(1) << 40) / L) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_gemm_planes: S*L overflows");
  return launch_pwconv_gemm_planes(a_planes, M, K, b_planes, b_terms, b_amax, S, L, c, partial, static_cast<hipStream_t>(stream));
}

int64_t sjhip_pwconv_grad_weight_planes_workspace_floats(int64_t M, int64_t N, int64_t S, int64_t L) {
  if (M < 1 || N < 1 || S < 1 || L < 1 || S > (int64_t(1) << 40) / L) return 0;
  return pwconv_dw_planes_workspace_floats(M, N, S, L);
}

int sjhip_pwconv_grad_weight_planes(const uint16_t *dy_planes, const float *dy_amax, const uint16_t *x_planes, int x_terms,
                                    const float *x_amax, int64_t S, int64_t M, int64_t N, int64_t L, float *dw, float *workspace,
                                    void *stream) {
  if (!dy_planes || !x_planes || !dw || !workspace) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight_planes: NULL buffer");
  if (M < 1 || N < 1 || S < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "pwconv_grad_weight_planes: M=%lld N=%lld S=%lld L=%lld must be >= 1", (long long)M, (long long)N, (long long)S, (long long)L);
  if (S > (int64_t(1) << 40) / L) return fail(SJHIP_ERR_TOO_LARGE, "pwconv_grad_weight_planes: S*L overflows");
  return launch_pwconv_grad_weight_planes(dy_planes, dy_amax, x_planes, x_terms, x_amax, S, M, N, L, dw, workspace,
                                          static_cast<hipStream_t>(stream));
}

int sjhip_bn_stats(const float *y, int64_t S, int64_t C, int64_t L, float *partial, void *stream) {
  if (!y || !partial) return fail(SJHIP_ERR_INVALID, "bn_stats: NULL buffer");
  return launch_bn_stats(y, S, C, L, partial, static_cast<hipStream_t>(stream));
}

int sjhip_bn_finalize(const float *partial, int64_t S, int64_t C, int64_t L, const float *gamma, const float *beta, float eps,
                      float momentum, float *running_mean, float *running_var, float *scale, float *shift, float *mean,
                      float *invstd, int64_t *batches_tracked, void *stream) {
  if (!scale || !shift || !mean || !invstd) return fail(SJHIP_ERR_INVALID, "bn_finalize: NULL output");
  if (partial && (S < 1 || L < 1)) return fail(SJHIP_ERR_INVALID, "bn_finalize: S=%lld L=%lld", (long long)S, (long long)L);
  return launch_bn_finalize(partial, S, S * L, C, gamma, beta, eps, momentum, running_mean, running_var, scale, shift, mean, invstd,
                            batches_tracked, static_cast<hipStream_t>(stream));
}

int sjhip_bn_finalize_rows(const float *partial, int64_t rows, int64_t count, int64_t C, const float *gamma, const float *beta,
                           float eps, float momentum, float *running_mean, float *running_var, float *scale, float *shift,
                           float *mean, float *invstd, int64_t *batches_tracked, void *stream) {
  if (!partial || !scale || !shift || !mean || !invstd) return fail(SJHIP_ERR_INVALID, "bn_finalize_rows: NULL buffer");
  if (rows < 1 || count < 1) return fail(SJHIP_ERR_INVALID, "bn_finalize_rows: rows=%lld count=%lld", (long long)rows, (long long)count);
  return launch_bn_finalize(partial, rows, count, C, gamma, beta, eps, momentum, running_mean, running_var, scale, shift, mean,
                            invstd, batches_tracked, static_cast<hipStream_t>(stream));
}

int sjhip_bn_lif_forward(int neuron, const sjhip_neuron_params *p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                         const float *scale, const float *shift, const float *v_init, float *spike_seq, uint8_t *spike_bits,
                         float *v_last, void *stream) {
  if (!p || !y || !scale || !shift || !v_init || (spike_seq == nullptr) == (spike_bits == nullptr))
    return fail(SJHIP_ERR_INVALID, "bn_lif_forward: NULL buffer, or not exactly one of spike_seq / spike_bits");
  return launch_bn_lif_forward(neuron, *p, T, B, C, L, y, scale, shift, v_init, nullptr, spike_seq, spike_bits, v_last,
                               static_cast<hipStream_t>(stream));
}

int sjhip_bn_lif_backward(int neuron, const sjhip_neuron_params *p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                          const float *scale, const float *shift, const float *v_init, const float *grad_spike_seq,
                          const float *grad_v_last, float *grad_z, float *grad_v_init, float *partial, void *stream) {
  if (!p || !y || !scale || !shift || !v_init || !grad_spike_seq || !grad_z || !partial)
    return fail(SJHIP_ERR_INVALID, "bn_lif_backward: NULL buffer");
  return launch_bn_lif_backward(neuron, *p, T, B, C, L, y, scale, shift, v_init, nullptr, grad_spike_seq, grad_v_last, grad_z,
                                grad_v_init, partial, nullptr, nullptr, static_cast<hipStream_t>(stream));
}

int sjhip_bn_plif_forward(const sjhip_neuron_params *p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                          const float *scale, const float *shift, const float *v_init, const float *k_device, float *spike_seq,
                          uint8_t *spike_bits, float *v_last, void *stream) {
  if (!p || !y || !scale || !shift || !v_init || !k_device || (spike_seq == nullptr) == (spike_bits == nullptr))
    return fail(SJHIP_ERR_INVALID, "bn_plif_forward: NULL buffer, or not exactly one of spike_seq / spike_bits");
  return launch_bn_lif_forward(SJHIP_NEURON_PLIF, *p, T, B, C, L, y, scale, shift, v_init, k_device, spike_seq, spike_bits, v_last,
                               static_cast<hipStream_t>(stream));
}

int64_t sjhip_bn_plif_backward_workspace_floats(int64_t B, int64_t C, int64_t L) {
  return bn_lif_backward_k_workspace_floats(B, C, L);
}

int sjhip_bn_plif_backward(const sjhip_neuron_params *p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                           const float *scale, const float *shift, const float *v_init, const float *k_device,
                           const float *grad_spike_seq, const float *grad_v_last, float *grad_z, float *grad_v_init,
                           float *partial, float *grad_k, float *workspace, void *stream) {
  if (!p || !y || !scale || !shift || !v_init || !k_device || !grad_spike_seq || !grad_z || !partial || !grad_k || !workspace)
    return fail(SJHIP_ERR_INVALID, "bn_plif_backward: NULL buffer");
  return launch_bn_lif_backward(SJHIP_NEURON_PLIF, *p, T, B, C, L, y, scale, shift, v_init, k_device, grad_spike_seq, grad_v_last,
                                grad_z, grad_v_init, partial, grad_k, workspace, static_cast<hipStream_t>(stream));
}

int sjhip_bn_backward_finalize(const float *partial, int64_t T, int64_t B, int64_t C, int64_t L, int training, const float *gamma,
                               const float *mean, const float *invstd, float *dgamma, float *dbeta, float *coef, float *amax_reset,
                               void *stream) {
  if (!partial || !mean || !invstd || !coef) return fail(SJHIP_ERR_INVALID, "bn_backward_finalize: NULL buffer");
  if (T < 1 || B < 1 || L < 1) return fail(SJHIP_ERR_INVALID, "bn_backward_finalize: T=%lld B=%lld L=%lld", (long long)T, (long long)B, (long long)L);
  return launch_bn_backward_finalize(partial, T, B, C, L, training, gamma, mean, invstd, dgamma, dbeta, coef, amax_reset,
                                     static_cast<hipStream_t>(stream));
}

int sjhip_bn_grad_input(const float *g, const float *y, const float *coef, int64_t S, int64_t C, int64_t L, float *dy, void *stream) {
  if (!g || !y || !coef || !dy) return fail(SJHIP_ERR_INVALID, "bn_grad_input: NULL buffer");
  return launch_bn_grad_input(g, y, coef, S, C, L, dy, nullptr, static_cast<hipStream_t>(stream));
}

int sjhip_bn_grad_input_amax(const float *g, const float *y, const float *coef, int64_t S, int64_t C, int64_t L, float *dy,
                             float *amax, void *stream) {
  if (!g || !y || !coef || !dy || !amax) return fail(SJHIP_ERR_INVALID, "bn_grad_input_amax: NULL buffer");
  return launch_bn_grad_input(g, y, coef, S, C, L, dy, amax, static_cast<hipStream_t>(stream));
}

int sjhip_set_tuning(const char *key, int value) {
  if (!key) return fail(SJHIP_ERR_INVALID, "set_tuning: NULL key");
  const bool block_ok = (value == 64 || value == 128 || value == 256 || value == 512) && value <= SJHIP_MAX_BLOCK;
  if (!strcmp(key, "fwd_block")) { if (!block_ok) return fail(SJHIP_ERR_INVALID, "set_tuning: fwd_block=%d", value); g_tuning.fwd_block = value; return SJHIP_OK; }
  if (!strcmp(key, "bwd_block")) { if (!block_ok) return fail(SJHIP_ERR_INVALID, "set_tuning: bwd_block=%d", value); g_tuning.bwd_block = value; return SJHIP_OK; }
  const bool cap_ok = value >= 0 && value <= 64;
  if (!strcmp(key, "fwd_blocks_per_cu")) { if (!cap_ok) return fail(SJHIP_ERR_INVALID, "set_tuning: fwd_blocks_per_cu=%d", value); g_tuning.fwd_blocks_per_cu = value; return SJHIP_OK; }
  if (!strcmp(key, "bwd_blocks_per_cu")) { if (!cap_ok) return fail(SJHIP_ERR_INVALID, "set_tuning: bwd_blocks_per_cu=%d", value); g_tuning.bwd_blocks_per_cu = value; return SJHIP_OK; }
  if (!strcmp(key, "replay_blocks_per_cu")) { if (!cap_ok) return fail(SJHIP_ERR_INVALID, "set_tuning: replay_blocks_per_cu=%d", value); g_tuning.replay_blocks_per_cu = value; return SJHIP_OK; }
  if (!strcmp(key, "column_spread")) { if (value < 0 || value == 3 || value > 65536) return fail(SJHIP_ERR_INVALID, "set_tuning: column_spread=%d", value); g_tuning.column_spread = value; return SJHIP_OK; }
  return fail(SJHIP_ERR_INVALID, "set_tuning: unknown key '%s'", key);
}

int sjhip_get_tuning(const char *key) {
  if (!key) return fail(SJHIP_ERR_INVALID, "get_tuning: NULL key");
  if (!strcmp(key, "fwd_block")) return g_tuning.fwd_block;
  if (!strcmp(key, "bwd_block")) return g_tuning.bwd_block;
  if (!strcmp(key, "fwd_blocks_per_cu")) return g_tuning.fwd_blocks_per_cu;
  if (!strcmp(key, "bwd_blocks_per_cu")) return g_tuning.bwd_blocks_per_cu;
  if (!strcmp(key, "replay_blocks_per_cu")) return g_tuning.replay_blocks_per_cu;
  if (!strcmp(key, "column_spread")) return g_tuning.column_spread;
  return fail(SJHIP_ERR_INVALID, "get_tuning: unknown key '%s'", key);
}

int sjhip_profile_enable(int on) {
  g_prof_on.store(on ? 1 : 0);
  return SJHIP_OK;
}

int sjhip_profile_reset(void) {
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  drain_pending();
  for (int i = 0; i < KC_COUNT; ++i) { g_prof_count[i] = 0; g_prof_ms[i] = 0.0; }
  return SJHIP_OK;
}

int sjhip_profile_read(int which, int64_t *launches, double *total_ms) {
  if (which < 0 || which >= KC_COUNT) return fail(SJHIP_ERR_INVALID, "profile_read: class %d", which);
  std::lock_guard<std::mutex> lock(g_prof_mutex);
  drain_pending();
  if (launches) *launches = g_prof_count[which];
  if (total_ms) *total_ms = g_prof_ms[which];
  return SJHIP_OK;
}

}  // extern "C"
