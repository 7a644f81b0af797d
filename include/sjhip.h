/*
 * sjhip.h -- C ABI of libsjhip.so: multi-step spiking-neuron kernels for
 * AMD MI355X (gfx950), hand-written HIP.
 *
 * Every entry point is asynchronous on the HIP stream it is given, owns no
 * device memory, never synchronises the host and never throws: it returns
 * SJHIP_OK (0) or a negative sjhip_status and leaves a thread-local message
 * for sjhip_last_error().  All tensors are dense row-major [T, N] views
 * ("time outer, neurons contiguous") of device memory owned by the caller.
 *
 * Reference interfaces these entry points stand in for (paths relative to the
 * SpikingJelly source tree):
 *   sjhip_neuron_forward   <- torch.ops.sj.cupy_multistep_{if,lif,plif}_forward
 *                             spikingjelly/activation_based/cuda_kernel/neuron_kernel/multi_step/lif.py:144-192,
 *                             plif.py:288-386, integrate_and_fire.py:76-147; and
 *                             torch.ops.sj.multistep_{if,lif,plif}_{forward,inference}
 *                             spikingjelly/activation_based/triton_kernel/neuron_kernel/lif.py:673-763
 *                             QIF: torch.ops.sj.cupy_multistep_qif_forward and its backward,
 *                             cuda_kernel/neuron_kernel/multi_step/qif.py:21-277, 628-701
 *                             EIF: torch.ops.sj.cupy_multistep_eif_forward and its backward,
 *                             cuda_kernel/neuron_kernel/multi_step/eif.py
 *                             ILIF: torch.ops.sj.multistep_ilif_forward{,_no_grad} and its backward,
 *                             triton_kernel/neuron_kernel/ilif.py:37-235, 241-462, 556-726
 *   sjhip_neuron_forward_packed <- the same forward ops followed by BitSpikeCompressor.compress,
 *                             spikingjelly/activation_based/memopt/compress.py:332-385
 *   sjhip_neuron_backward  <- torch.ops.sj.cupy_multistep_{if,lif,plif}_backward
 *                             multi_step/lif.py:228-282, plif.py:389-470, integrate_and_fire.py:150-200;
 *                             BPTT body multi_step/base.py:137-409
 *   sjhip_plif_workspace_floats / grad_rtau reduction
 *                          <- shared-memory tree + atomicAdd in multi_step/plif.py:107-237 and the
 *                             per-neuron partials + torch.sum of triton_kernel/neuron_kernel/plif.py:340-378,1180-1203
 *   sjhip_bit_pack/unpack  <- bit_spike_compress / bit_spike_decompress,
 *                             spikingjelly/activation_based/triton_kernel/compress.py:114-221 (torch fallback :19-44),
 *                             and float2bool/bool2float of cuda_kernel/tensor_cache.py:16-93
 */
#ifndef SJHIP_H_
#define SJHIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SJHIP_ABI_VERSION 7

typedef enum sjhip_status {
  SJHIP_OK = 0,
  SJHIP_ERR_INVALID = -1,     /* bad enum / flag / NULL / size / alignment */
  SJHIP_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for */
  SJHIP_ERR_LAUNCH = -3,      /* HIP reported an error at launch */
  SJHIP_ERR_TOO_LARGE = -4    /* size beyond a documented limit */
} sjhip_status;

/* Neuron model: charge equation applied before fire/reset. */
typedef enum sjhip_neuron {
  SJHIP_NEURON_IF = 0,  /* h = v + x                                  (functional/neuron.py:310)   */
  SJHIP_NEURON_LIF = 1, /* h = v + (x - (v - vr)) / tau  or  v - (v - vr)/tau + x   (:849-852)     */
  SJHIP_NEURON_PLIF = 2, /* h = v + (x - (v - vr)) * k    or  v - (v - vr)*k + x     (:1290-1295)   */
  SJHIP_NEURON_QIF = 3, /* h = v + (x + a0 (v - v_rest) (v - v_c)) / tau          (functional/neuron.py:397) */
  SJHIP_NEURON_EIF = 5, /* exponential integrate-and-fire (functional/neuron.py:483-485):
                           h = v + (x + v_rest - v + delta_T exp((v - theta_rh) / delta_T)) / tau; theta_rh travels in
                           the field v_c and delta_T (> 0) in the field a0.  exp() is the device library's, accurate
                           to 1 ulp but not bit-identical to a host libm: h agrees with a CPU run to rounding, a
                           spike may differ where h lands within that distance of v_threshold. */
  SJHIP_NEURON_ILIF = 4 /* integer-valued LIF (functional/neuron.py:1097-1099): h = v - v/tau + x (the LIF charge
                           without input decay and with v_reset = None), fires the count
                           c = rint(clamp(h / v_th, 0, level_max)) instead of a binary spike and resets softly by
                           c v_th.  spike_seq holds c.  Always a soft reset; the flags DECAY_INPUT and SOFT_RESET
                           are ignored.  Backward needs sg_id = SJHIP_SG_MULTI_LEVEL. */
} sjhip_neuron;

/* Storage dtype of every [T,N] / [N] tensor of one call. */
typedef enum sjhip_dtype {
  SJHIP_F32 = 0,
  SJHIP_F16 = 1,
  SJHIP_BF16 = 2,
  SJHIP_U8 = 3, /* bit_pack / bit_unpack only */
  SJHIP_F8E4M3 = 4, /* float8_e4m3fn, storage dtype of the *_mp entry points only */
  SJHIP_F8E5M2 = 5  /* float8_e5m2, likewise */
} sjhip_dtype;

/* Surrogate gradient used by the backward pass (forward is always Heaviside).
 * Ids follow triton_kernel/surrogate_kernel.py:26-34. */
typedef enum sjhip_surrogate {
  SJHIP_SG_SIGMOID = 0,
  SJHIP_SG_ATAN = 1,
  SJHIP_SG_PIECEWISE_QUADRATIC = 2,
  SJHIP_SG_PIECEWISE_EXP = 3,
  SJHIP_SG_SOFT_SIGN = 4,
  SJHIP_SG_SUPER_SPIKE = 5,
  SJHIP_SG_ERF = 6,
  SJHIP_SG_MULTI_LEVEL = 7 /* ILIF only (quantize.py:580-598): straight-through window on z = h / v_th,
                              dc/dz = [grad_min <= z <= grad_max]; sg_alpha is unused */
} sjhip_surrogate;

/* Bit flags. */
#define SJHIP_FLAG_DECAY_INPUT 0x01u  /* LIF/PLIF: input is scaled by 1/tau */
#define SJHIP_FLAG_SOFT_RESET 0x02u   /* v = h - s*v_th ; otherwise hard reset to v_reset */
#define SJHIP_FLAG_DETACH_RESET 0x04u /* backward: no gradient through the reset branch */
#define SJHIP_FLAG_FP32_STATE 0x10u   /* 16-bit storage: keep v and all arithmetic in fp32, round only
                                         what is stored (the reference's mixed-precision ops,
                                         triton_kernel/neuron_kernel/lif.py:787-870).  Without it 16-bit
                                         storage rounds after every arithmetic op, like the torch backend. */
#define SJHIP_FLAG_RECIPROCAL_TAU 0x20u /* LIF: multiply by fl(1/tau) instead of dividing by tau (what the
                                           CuPy/Triton kernels and torch-on-GPU do); default is the IEEE
                                           division of the torch CPU backend. */
#define SJHIP_FLAG_ATOMIC_REDUCE 0x80u /* PLIF backward: one atomicAdd per block into grad_rtau (caller
                                          zeroes it) instead of the deterministic two-pass reduction */

#define SJHIP_FLAG_V_INIT_BROADCAST 0x100u /* v_init points to ONE element that every neuron starts from (a
                                              module state that is still its scalar reset value): no [N]
                                              tensor has to be filled and read */
#define SJHIP_FLAG_GRAD_STORAGE 0x1000u /* sjhip_neuron_backward_mp: grad_x_seq and grad_v_init are written in the
                                           storage dtype instead of fp32 (0x200 - 0x800 are taken further down) */

/* Scalars of one neuron layer.  `tau` is tau for LIF and the reciprocal k = sigmoid(w) for PLIF
 * (ignored for IF).  `v_reset` is ignored for IF soft reset and is the charge-equation offset
 * (0 when the module has v_reset=None) otherwise. */
typedef struct sjhip_neuron_params {
  float tau;
  float v_threshold;
  float v_reset;
  float sg_alpha;   /* backward only */
  int32_t sg_id;    /* backward only, sjhip_surrogate */
  uint32_t flags;
  float v_rest;     /* QIF and EIF */
  float v_c;        /* QIF: critical voltage; EIF: theta_rh */
  float a0;         /* QIF: a0; EIF: delta_T */
  float level_max;  /* ILIF only: largest spike count D, an integer >= 1 */
  float grad_min;   /* ILIF only, backward: lower end of the gradient window on h / v_th */
  float grad_max;   /* ILIF only, backward: upper end (grad_min <= grad_max) */
} sjhip_neuron_params;

/* ABI version of the loaded library (== SJHIP_ABI_VERSION it was built with). */
int sjhip_abi_version(void);

/* Thread-local text of the last error returned on this thread ("" if none). */
const char *sjhip_last_error(void);

/*
 * Forward over T steps for N neurons.
 *   x_seq     [T,N] in            v_init  [N] in ([1] with SJHIP_FLAG_V_INIT_BROADCAST)
 *   spike_seq [T,N] out (0/1 in the storage dtype; ILIF: the count 0..level_max)
 *   v_seq     [T,N] out, membrane potential after reset at every step; NULL = do not write
 *   v_last    [N] out, membrane potential after the last step; NULL = do not write
 *             (at least one of v_seq / v_last must be given)
 *   h_seq     [T,N] out, membrane potential before reset, saved for backward; NULL = do not write
 *   rtau_device  PLIF only (required there, SJHIP_ERR_INVALID without it; NULL for the other neurons): device
 *             address of one fp32 holding k = sigmoid(w), read by the kernel in place of p->tau so that no host
 *             synchronisation is needed to fetch it
 * T >= 1, N >= 1, T*N < 2^62.  128-bit accesses are used when N is a multiple of 16/sizeof(dtype)
 * and every pointer is 16-byte aligned; otherwise an element-wise kernel runs.
 */
int sjhip_neuron_forward(int neuron, int dtype, const sjhip_neuron_params *p,
                         int64_t T, int64_t N,
                         const void *x_seq, const void *v_init, const float *rtau_device,
                         void *spike_seq, void *v_seq, void *v_last, void *h_seq,
                         void *stream);

/*
 * Inference forward that writes the spikes bit-packed instead of as a dense tensor: the fused form of
 * sjhip_neuron_forward followed by sjhip_bit_pack, i.e. of a kernel-backend neuron feeding the reference's
 * BitSpikeCompressor (spikingjelly/activation_based/memopt/compress.py:332-385 on top of
 * triton_kernel/compress.py:114-166).  Per neuron-step it moves sizeof(dtype) + 1/8 bytes instead of
 * 2 sizeof(dtype) for the forward plus sizeof(dtype) + 1/8 for the pack.
 *   spike_bits  [(T*N)/8] bytes out: byte j bit i = spike of flattened element 8 j + i (LSB first), exactly
 *               what sjhip_bit_pack writes for the dense [T,N] spike tensor
 *   other arguments as sjhip_neuron_forward (no h_seq: this is an inference entry point)
 * N must be a multiple of 8 so that every time step starts on a byte (SJHIP_ERR_UNSUPPORTED otherwise).
 */
int sjhip_neuron_forward_packed(int neuron, int dtype, const sjhip_neuron_params *p,
                                int64_t T, int64_t N,
                                const void *x_seq, const void *v_init, const float *rtau_device,
                                uint8_t *spike_bits, void *v_seq, void *v_last,
                                void *stream);

/* Number of floats of caller-provided workspace the PLIF backward needs for N neurons of `dtype`
 * (per-block partial sums of the deterministic reduction). */
int64_t sjhip_plif_workspace_floats(int dtype, int64_t N);

/*
 * Backward (BPTT) over T steps.
 *   grad_spike_seq [T,N] in, or NULL for zeros (a loss on the membrane potential alone): nothing is read then
 *   grad_v_seq     [T,N] in, gradient w.r.t. v_seq, or NULL
 *   grad_v_last    [N] in, gradient w.r.t. v_last (enters at t = T-1), or NULL
 *   h_seq          [T,N] in (from forward)
 *   v_init         [N] in ([1] with SJHIP_FLAG_V_INIT_BROADCAST), PLIF only (NULL otherwise): v before step 0
 *   grad_x_seq     [T,N] out
 *   grad_v_init    [N] out, or NULL when the caller does not need the gradient of the initial state
 *   grad_rtau      1 float out, PLIF only: dL/dk, k = sigmoid(w)
 *   workspace      sjhip_plif_workspace_floats() floats, PLIF without SJHIP_FLAG_ATOMIC_REDUCE
 */
int sjhip_neuron_backward(int neuron, int dtype, const sjhip_neuron_params *p,
                          int64_t T, int64_t N,
                          const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                          const void *h_seq,
                          const void *v_init, const float *rtau_device,
                          void *grad_x_seq, void *grad_v_init,
                          float *grad_rtau, float *workspace,
                          void *stream);

/*
 * sjhip_neuron_backward with the PLIF workspace inside the library: for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference,
 * whose operators allocate their outputs and partial sums through torch / CuPy on every call.  Same arguments and
 * results as sjhip_neuron_backward minus `workspace`: the per-block partial sums of dL/dk go to a 4 MiB array that is
 * part of the library's code object (one copy per GPU, held until the process ends), so the call reaches no
 * hipMalloc / hipFree.  PLIF without SJHIP_FLAG_ATOMIC_REDUCE accepts N <= SJHIP_STATIC_WORKSPACE_MAX_NEURONS and
 * returns SJHIP_ERR_TOO_LARGE beyond; other neurons use no workspace and are passed through.  The stream's device must
 * be the current device.  Every call on one GPU shares that GPU's array: calls on one stream are ordered and need no
 * clearing in between (each launch writes every partial it later sums); a call on another stream of the GPU while the
 * last call's work has not finished is refused with SJHIP_ERR_INVALID (an event recorded behind every launch that uses
 * the array, created once per GPU, tells), so order such calls with one stream or an event.  A stream that is being
 * captured into a graph is neither checked nor recorded: the caller orders the replays of graphs that use the array.
 */
#define SJHIP_STATIC_WORKSPACE_MAX_NEURONS (INT64_C(1) << 26)
int sjhip_neuron_backward_static(int neuron, int dtype, const sjhip_neuron_params *p,
                                 int64_t T, int64_t N,
                                 const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                                 const void *h_seq,
                                 const void *v_init, const float *rtau_device,
                                 void *grad_x_seq, void *grad_v_init,
                                 float *grad_rtau,
                                 void *stream);

/*
 * Backward that needs no h_seq: it replays the forward from x_seq and v_init (bit-identical h, kept
 * in LDS) and then runs the same BPTT.  A forward whose backward will use this entry point can be
 * called with h_seq = NULL, which saves its largest write.  Same argument meaning as
 * sjhip_neuron_backward with (x_seq, v_init) in place of h_seq; `p` carries the forward flags too
 * (SJHIP_FLAG_FP32_STATE, SJHIP_FLAG_RECIPROCAL_TAU).  Requires sjhip_recompute_supported() and
 * 16-byte aligned tensors; returns SJHIP_ERR_UNSUPPORTED / SJHIP_ERR_INVALID otherwise.
 * Stands in for the same reference backward ops as sjhip_neuron_backward; the reference has no
 * recomputing variant (its kernels always read the saved h_seq, multi_step/base.py:137-409).
 */
int sjhip_neuron_backward_recompute(int neuron, int dtype, const sjhip_neuron_params *p,
                                    int64_t T, int64_t N,
                                    const void *x_seq, const void *v_init, const float *rtau_device,
                                    const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                                    void *grad_x_seq, void *grad_v_init,
                                    float *grad_rtau, float *workspace,
                                    void *stream);

/*
 * The replay for sequences of any length, in one launch each way.  The sequence is cut into pieces of `chunk` steps
 * (the last may be shorter; sjhip_replay_pieces(T, chunk) of them).  sjhip_neuron_forward_pieces is
 * sjhip_neuron_forward with h_seq = NULL that also leaves the state after every piece but the last in
 * `checkpoints` [pieces - 1][N] (storage dtype, see below; may be NULL when T <= chunk).  sjhip_neuron_backward_recompute_pieces
 * is sjhip_neuron_backward_recompute that walks the pieces from the last to the first: each is replayed from its
 * checkpoint into an LDS buffer of `chunk` steps (so chunk, not T, must satisfy sjhip_recompute_supported) and walked
 * back; the gradient of a piece's initial state stays in registers (fp32) for the piece before it.  Results: spikes,
 * states and checkpoints are bit-identical to sjhip_neuron_forward's; gradients are those of the walk over the whole
 * sequence (in fp32 storage also those of sjhip_neuron_backward_recompute applied piece by piece with grad_v_init
 * handed on as grad_v_last).  N must be a multiple of the 128-bit
 * vector width and every tensor 16-byte aligned.  With 16-bit storage and SJHIP_FLAG_FP32_STATE the checkpoints are
 * fp32 rows ([pieces - 1][N] floats: a checkpoint in the storage dtype would round the state).  The saved state per
 * neuron is 1 / chunk of an h_seq; chunk = 16 keeps
 * five or more blocks resident per compute unit, which is where the single-piece kernel runs fastest.  No counterpart
 * in the reference (its kernels always read the saved h_seq, multi_step/base.py:137-409).
 */
int64_t sjhip_replay_pieces(int64_t T, int64_t chunk);
int sjhip_neuron_forward_pieces(int neuron, int dtype, const sjhip_neuron_params *p,
                                int64_t T, int64_t N, int64_t chunk,
                                const void *x_seq, const void *v_init, const float *rtau_device,
                                void *spike_seq, void *v_seq, void *v_last, void *checkpoints,
                                void *stream);
int sjhip_neuron_backward_recompute_pieces(int neuron, int dtype, const sjhip_neuron_params *p,
                                           int64_t T, int64_t N, int64_t chunk,
                                           const void *x_seq, const void *v_init, const float *rtau_device,
                                           const void *checkpoints,
                                           const void *grad_spike_seq, const void *grad_v_seq, const void *grad_v_last,
                                           void *grad_x_seq, void *grad_v_init,
                                           float *grad_rtau, float *workspace,
                                           void *stream);

/* 1 if sjhip_neuron_backward_recompute can serve [T,N] of `dtype` (N a multiple of the 128-bit vector
 * width and T steps of h fitting in LDS: T <= 159), else 0. */
int sjhip_recompute_supported(int dtype, int64_t T, int64_t N);

/* 1 if, beyond being supported, the replay is expected to beat a saved h_seq: its LDS footprint grows with T and
 * below four resident wavefronts per compute unit (T > 39) reading h_seq is faster.  `flags` as in
 * sjhip_neuron_params (only SJHIP_FLAG_FP32_STATE matters).  A policy hint for callers; both paths stay valid. */
int sjhip_recompute_preferred(int dtype, int64_t T, int64_t N, uint32_t flags);

/*
 * ST-BIF, the signed ternary integrate-and-fire neuron of SpikeZIP's QANN-to-SNN conversion; inference only (the
 * reference implements no backward either).  Stands in for torch.ops.sj.multi_step_stbif / single_step_stbif,
 * spikingjelly/activation_based/triton_kernel/neuron_kernel/stbif.py:94-137, 258-316, 337-399, and computes the torch
 * backend's functional.stbif_step (functional/neuron.py:3234-3247) for every step:
 *     q += x / s;  acc = round(acc);  pos = (q - 1 >= 0) & (acc < pos_max);  neg = (q < 0) & (acc > neg_min);
 *     cur = pos - neg;  acc += cur;  q = pos ? q - 1 : (neg ? q + 1 : q);  out = cur * s
 *   x_seq       [T,N] in
 *   q_init      [N] in, quantisation residual ([1] with SJHIP_FLAG_Q_BROADCAST; a fresh neuron starts from 0.5)
 *   acc_q_init  [N] in, integer released so far ([1] with SJHIP_FLAG_ACC_BROADCAST; a fresh neuron starts from 0)
 *   q_threshold, pos_max, neg_min   device addresses of one fp32 each: the quantiser scale s and the bounds of acc;
 *               they are rounded to `dtype` before use, like `.to(x)` in the reference
 *   out_seq     [T,N] out: -s, 0 or +s
 *   q_final, acc_q_final, cur_output   [N] out: the states after the last step and its ternary output
 *   work_flag   one int32, or NULL: set to 1 when any input or any output of the call is non-zero, never cleared
 *               (the caller zeroes it; STBIFNeuron.is_work)
 * flags: SJHIP_FLAG_FP32_STATE (16-bit storage: fp32 arithmetic, stored values rounded -- the Triton kernel;
 * without it every op is rounded like torch on half tensors) and the two broadcast flags.
 */
#define SJHIP_FLAG_Q_BROADCAST 0x200u
#define SJHIP_FLAG_ACC_BROADCAST 0x400u
int sjhip_stbif_forward(int dtype, uint32_t flags, int64_t T, int64_t N,
                        const void *x_seq, const void *q_init, const void *acc_q_init,
                        const float *q_threshold, const float *pos_max, const float *neg_min,
                        void *out_seq, void *q_final, void *acc_q_final, void *cur_output,
                        int32_t *work_flag, void *stream);

/*
 * IF / LIF / PLIF with 8-bit floating-point storage (mixed precision).  Stands in for the reference's
 * torch.ops.sj.multistep_{if,lif,plif}_mp_forward / _mp_inference and their backward with an FP8 storage dtype,
 * spikingjelly/activation_based/triton_kernel/neuron_kernel/lif.py:788-956, 1103-1150 (plif.py:834-879,
 * integrate_and_fire.py likewise): x_seq, v_init, v_seq, v_last, h_seq, grad_v_seq and grad_v_last are
 * `storage_dtype` (SJHIP_F8E4M3 or SJHIP_F8E5M2), spike_seq and grad_spike_seq are `spike_dtype` (SJHIP_F32, SJHIP_F16
 * or SJHIP_BF16), the recurrence runs in fp32 on the decoded values and only stored values are rounded (round to
 * nearest even as torch's .to(torch.float8_*): e4m3fn has no infinity and overflows to NaN, e5m2 overflows to
 * infinity); grad_x_seq [T,N] and grad_v_init [N] are fp32, or, with SJHIP_FLAG_GRAD_STORAGE, `storage_dtype` like the
 * reference's (lif.py:1115-1118 allocates them in the dtypes of x_seq and v_init; the fp32 value is rounded once).  Same params, flags and PLIF conventions as
 * sjhip_neuron_forward / sjhip_neuron_backward (PLIF: rtau_device, grad_rtau and a workspace of
 * sjhip_plif_workspace_floats(SJHIP_F32, N) floats).  N must be a multiple of 4 and every tensor 16-byte aligned
 * (a work-item owns four groups of four neurons: one 4-byte access per group of an 8-bit row); callers pad.
 * neuron: IF, LIF or PLIF.
 */
int sjhip_neuron_forward_mp(int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params *p,
                            int64_t T, int64_t N, const void *x_seq, const void *v_init, const float *rtau_device,
                            void *spike_seq, void *v_seq, void *v_last, void *h_seq, void *stream);
int sjhip_neuron_backward_mp(int neuron, int storage_dtype, int spike_dtype, const sjhip_neuron_params *p,
                             int64_t T, int64_t N, const void *grad_spike_seq, const void *grad_v_seq,
                             const void *grad_v_last, const void *h_seq, const void *v_init,
                             const float *rtau_device, void *grad_x_seq, void *grad_v_init, float *grad_rtau,
                             float *workspace, void *stream);

/*
 * Izhikevich neuron: quadratic membrane v with an adaptation current w (two states).  Stands in for
 * torch.ops.sj.cupy_multistep_izhikevich_forward / _backward,
 * spikingjelly/activation_based/cuda_kernel/neuron_kernel/multi_step/izhikevich.py, and computes the torch backend's
 * functional.izhikevich_step (functional/neuron.py:1514-1522) for every step:
 *     h = v + (x + a0 (v - v_rest)(v - v_c) - w) / tau;   u = w + (a (h - v_rest) - w) / tau_w;   s = [h >= v_th];
 *     v' = h - s v_th  or  (1 - s) h + s v_reset;         w' = u + b s
 * Forward:  x_seq [T,N], v_init / w_init [N] in ([1] with the broadcast flags); spike_seq [T,N], v_last, w_last [N]
 * out; v_seq, w_seq [T,N] out or NULL; h_seq [T,N] out or NULL (needed by the backward).
 * Backward: grad_spike_seq [T,N], h_seq [T,N] in; grad_v_seq, grad_w_seq [T,N] and grad_v_last, grad_w_last [N] in or
 * NULL; v_init in (needed for grad_v_init); grad_x_seq [T,N] out; grad_v_init, grad_w_init [N] out or NULL.
 * flags: SJHIP_FLAG_SOFT_RESET, SJHIP_FLAG_DETACH_RESET, SJHIP_FLAG_FP32_STATE, SJHIP_FLAG_V_INIT_BROADCAST,
 * SJHIP_FLAG_W_INIT_BROADCAST.
 */
#define SJHIP_FLAG_W_INIT_BROADCAST 0x800u
typedef struct sjhip_izhikevich_params {
  float tau, v_threshold, v_reset, v_rest, v_c, a0, tau_w, a, b;
  float sg_alpha;   /* backward only */
  int32_t sg_id;    /* backward only, sjhip_surrogate 0..6 */
  uint32_t flags;
} sjhip_izhikevich_params;
int sjhip_izhikevich_forward(int dtype, const sjhip_izhikevich_params *p, int64_t T, int64_t N,
                             const void *x_seq, const void *v_init, const void *w_init,
                             void *spike_seq, void *v_seq, void *w_seq, void *v_last, void *w_last, void *h_seq,
                             void *stream);
int sjhip_izhikevich_backward(int dtype, const sjhip_izhikevich_params *p, int64_t T, int64_t N,
                              const void *grad_spike_seq, const void *grad_v_seq, const void *grad_w_seq,
                              const void *grad_v_last, const void *grad_w_last, const void *h_seq, const void *v_init,
                              void *grad_x_seq, void *grad_v_init, void *grad_w_init, void *stream);
/* The same backward without a saved h_seq: the kernel replays the forward from x_seq, v_init and w_init (the forward's
 * own arithmetic, so the replayed h has its bits), keeps h of every step in LDS and then walks back.  The forward can
 * then be called with h_seq = NULL.  Limits of sjhip_recompute_supported(dtype, T, N); every tensor 16-byte aligned.
 * The reference's kernel always saves h_seq (multi_step/izhikevich.py); this variant has no counterpart there. */
int sjhip_izhikevich_backward_replay(int dtype, const sjhip_izhikevich_params *p, int64_t T, int64_t N,
                                     const void *x_seq, const void *v_init, const void *w_init,
                                     const void *grad_spike_seq, const void *grad_v_seq, const void *grad_w_seq,
                                     const void *grad_v_last, const void *grad_w_last,
                                     void *grad_x_seq, void *grad_v_init, void *grad_w_init, void *stream);

/*
 * Activation-aware IF (ANN2SNN activation-aware redistribution): an IF neuron whose threshold and membrane offset are
 * per channel or scalar; inference only.  Stands in for torch.ops.sj.multistep_activation_aware_if_forward,
 * spikingjelly/activation_based/triton_kernel/neuron_kernel/activation_aware_if.py:44-285, and computes the torch
 * backend's functional.activation_aware_if_step (functional/neuron.py:577-584) for every step:
 *     h = v + x;  s = [(h + offset_c) - threshold_c >= 0];  v = h - s threshold_c  or  s v_reset + (1 - s) h
 * with c = (n / inner_size) % channel_size the channel of neuron n of a flattened time step.
 *   x_seq [T,N] in        v_init [N] in ([1] with SJHIP_FLAG_V_INIT_BROADCAST)
 *   v_threshold, v_offset   device fp32 arrays of threshold_count / offset_count elements, each 1 (scalar) or
 *                           channel_size; rounded to `dtype` before use, like `.to(x)` in the reference
 *   spike_seq [T,N] out;  v_seq [T,N] out or NULL;  v_last [N] out or NULL (at least one of the two)
 * flags: SJHIP_FLAG_SOFT_RESET, SJHIP_FLAG_FP32_STATE, SJHIP_FLAG_V_INIT_BROADCAST.
 */
int sjhip_aaif_forward(int dtype, uint32_t flags, int64_t T, int64_t N,
                       const void *x_seq, const void *v_init,
                       const float *v_threshold, int64_t threshold_count,
                       const float *v_offset, int64_t offset_count,
                       int64_t channel_size, int64_t inner_size, float v_reset,
                       void *spike_seq, void *v_seq, void *v_last, void *stream);

/*
 * Spike bit-packing over a flattened tensor, LSB first: byte j bit i = (src[8j+i] != 0).
 *   src  n elements of `dtype` (F32/F16/BF16/U8)     dst  (n+7)/8 bytes; pad bits of the last byte are 0
 */
int sjhip_bit_pack(int dtype, int64_t n, const void *src, uint8_t *dst, void *stream);

/* Inverse: dst[8j+i] = (src[j] >> i) & 1 as 0/1 of `dtype`, n elements written. */
int sjhip_bit_unpack(int dtype, int64_t n, const uint8_t *src, void *dst, void *stream);

/*
 * Spiking self-attention contraction on the matrix cores (stands in for `_ssa_kernel_torch`,
 * spikingjelly/activation_based/layer/attention.py:346-353:  x = (v @ k^T) @ q * scale).
 *   qkv      [samples, 3, heads, channels_per_head, tokens] in: binary spikes, q / k / v stacked on dim 1
 *   out      [samples, heads, channels_per_head, tokens] out = scale * (V K^T) Q, exact (integer sums in fp32)
 *   grad_out same shape as out, in;  grad_qkv same shape as qkv, out (dq, dk, dv)
 * One block of four wavefronts (eight for heads of more than 32 channels) per (sample, head), the spikes of its three
 * tiles parked in LDS as bytes.  Forward:
 * V K^T on the int8 MFMA (exact integers), then (V K^T) Q on the bf16 MFMA with fp32 accumulation (V K^T <= 256 and
 * the spikes are exact in bf16), so out equals an integer matmul times scale bit for bit.  Backward: dS = scale dO Q^T
 * on the fp32 MFMA; dQ, dK, dV on the bf16 MFMA with the real-valued operand split into three bf16 terms that sum to
 * it exactly.  Needs sjhip_ssa_supported(): at most 64 channels per head, at most 256 tokens (V K^T must stay exact
 * in bf16) and the tiles of one head fitting in LDS.
 */
int sjhip_ssa_supported(int dtype, int channels_per_head, int64_t tokens);
int sjhip_ssa_forward(int dtype, int64_t samples, int heads, int channels_per_head, int64_t tokens, float scale,
                      const void *qkv, void *out, void *stream);
int sjhip_ssa_backward(int dtype, int64_t samples, int heads, int channels_per_head, int64_t tokens, float scale,
                       const void *qkv, const void *grad_out, void *grad_qkv, void *stream);

/*
 * The same contraction with bit-packed operands: the fused form of a kernel-backend LIF (bit-packed spike output,
 * sjhip_neuron_forward_packed) feeding the contraction, so the dense q / k / v spike tensor is never written or
 * read.  No counterpart in the reference, whose attention takes dense spike tensors (layer/attention.py:370-383).
 *   qkv_bits  [(samples*3*heads*channels_per_head*tokens)/8] bytes: the flattened qkv tensor packed LSB first
 *             (byte j bit i = element 8 j + i, the layout of sjhip_bit_pack)
 *   dtype     of out / grad_out / grad_qkv
 * channels_per_head * tokens must be a multiple of 8 so that every head's tile starts on a byte
 * (SJHIP_ERR_UNSUPPORTED otherwise); results equal the dense entry points' bit for bit.
 */
int sjhip_ssa_forward_packed(int dtype, int64_t samples, int heads, int channels_per_head, int64_t tokens, float scale,
                             const uint8_t *qkv_bits, void *out, void *stream);
int sjhip_ssa_backward_packed(int dtype, int64_t samples, int heads, int channels_per_head, int64_t tokens, float scale,
                              const uint8_t *qkv_bits, const void *grad_out, void *grad_qkv, void *stream);

/*
 * The contraction fused with the multi-step IF / LIF neuron that takes its output as input: `attn_lif` of the
 * reference's SpikingSelfAttention (layer/attention.py:321-322, 383-384), which there is a separate module call on the
 * materialised `scale (V K^T) Q`.  fp32, bit-packed q / k / v as for sjhip_ssa_forward_packed with samples = T * B
 * ordered [T][B]; tokens a multiple of 4.  A block owns one (batch element, head) and walks the T steps with the
 * membrane potential in registers; the contraction's output is never written.
 *   forward:  spike_seq [T][B][heads][cph][tokens]; h_seq (same shape: the potential before firing, kept for the
 *             backward) or NULL; v_init [B][heads][cph][tokens] or one element with SJHIP_FLAG_V_INIT_BROADCAST;
 *             v_last or NULL.  Same arithmetic as sjhip_ssa_forward_packed followed by sjhip_neuron_forward, bit for bit.
 *   backward: from h_seq, grad_spike_seq (or NULL) and grad_v_last (or NULL): grad_qkv [T * B][3][heads][cph][tokens]
 *             (the gradient with respect to the q / k / v spikes) and grad_v_init (or NULL); the recurrence of
 *             sjhip_neuron_backward and the products of sjhip_ssa_backward_packed.
 * neuron: SJHIP_NEURON_IF or SJHIP_NEURON_LIF (SJHIP_ERR_UNSUPPORTED otherwise, and for shapes the contraction does
 * not support).
 */
int sjhip_ssa_lif_forward_packed(int neuron, const sjhip_neuron_params *p, int64_t T, int64_t B, int heads, int channels_per_head,
                                 int64_t tokens, float scale, const uint8_t *qkv_bits, const float *v_init, float *spike_seq,
                                 float *h_seq, float *v_last, void *stream);
int sjhip_ssa_lif_backward_packed(int neuron, const sjhip_neuron_params *p, int64_t T, int64_t B, int heads,
                                  int channels_per_head, int64_t tokens, float scale, const uint8_t *qkv_bits,
                                  const float *h_seq, const float *grad_spike_seq, const float *grad_v_last, float *grad_qkv,
                                  float *grad_v_init, void *stream);

/*
 * Kernel-size-1 convolution over [S, C, L] activations (S samples = time steps x batch, L positions, L contiguous) as
 * GEMMs on the bf16 matrix cores.  Stands in for torch's nn.Conv1d(kernel_size=1, bias=False) inside the reference's
 * SpikingSelfAttention (spikingjelly/activation_based/layer/attention.py:310-329, applied at :370 and :382 through
 * SeqToANNContainer) and nn.Conv2d(kernel_size=1) of SpikformerConv2dBN (model/spikformer.py:85-99), forward and both
 * gradients.  fp32 operands are split into `terms` bf16 terms that sum to the value (3: exactly), and the products whose
 * combined order is below max(terms) run on v_mfma_f32_32x32x16_bf16 with fp32 accumulation: 3 terms on both sides give
 * the accuracy of an fp32 GEMM; an operand that bf16 holds exactly (spikes) needs 1 term.  Supported (a_terms, b_terms):
 * (3,3) (3,1) (2,2) (2,1) (1,1).  sjhip_pwconv_gemm needs an even L, 16-byte aligned weight planes and 8-byte
 * aligned activations; sjhip_pwconv_grad_weight needs L a multiple of 4 and 16-byte aligned tensors
 * (SJHIP_ERR_UNSUPPORTED otherwise).
 *
 *   sjhip_pwconv_split_weight   planes = bf16 terms [3][rows_pad * cols_pad] (zero padded to multiples of 128 and 32, and
 *                               stored as tiles of 128 rows x 32 columns in the order sjhip_pwconv_gemm reads them: an
 *                               opaque buffer of sjhip_pwconv_planes_elems(rows, cols) elements of 2 bytes) of the matrix A = w
 *                               ([rows][cols] fp32) or, with transpose != 0, of A = w^T ([cols][rows]): the first operand
 *                               of sjhip_pwconv_gemm.  For transpose the element count is that of (cols, rows).
 *   sjhip_pwconv_gemm           c[s][m][l] = sum_k A[m][k] b[s][k][l]: the convolution with A = weight [Cout][Cin]
 *                               (M = Cout, K = Cin), its input gradient with A = weight^T (M = Cin, K = Cout, b = dY)
 *   sjhip_pwconv_grad_weight    dw[m][n] = sum_{s,l} dy[s][m][l] x[s][n][l]; workspace of
 *                               sjhip_pwconv_grad_weight_workspace_floats(M, N, S) floats (partial sums over groups of
 *                               samples, added in a fixed order)
 */
int64_t sjhip_pwconv_planes_elems(int64_t rows, int64_t cols);
int sjhip_pwconv_split_weight(const float *w, int64_t rows, int64_t cols, int transpose, uint16_t *planes, void *stream);
int sjhip_pwconv_gemm(const uint16_t *a_planes, int a_terms, int64_t M, int64_t K, const float *b, int b_terms, int64_t S,
                      int64_t L, float *c, void *stream);
/* sjhip_pwconv_gemm that also leaves the batch-norm statistics of c: partial[r][m] = (sum, sum of squares) of row m of c
 * over a group of 64 columns (s, l), r < sjhip_pwconv_gemm_stats_rows(K, S, L); sjhip_bn_finalize_rows(partial, rows,
 * S * L, M, ...) turns them into the affine map, which saves the pass of sjhip_bn_stats over c.  The reference's
 * nn.Conv1d + nn.BatchNorm1d (layer/attention.py:314-319) read the convolution output once more for this. */
int64_t sjhip_pwconv_gemm_stats_rows(int64_t K, int64_t S, int64_t L);
int sjhip_pwconv_gemm_stats(const uint16_t *a_planes, int a_terms, int64_t M, int64_t K, const float *b, int b_terms, int64_t S,
                            int64_t L, float *c, float *partial, void *stream);
int64_t sjhip_pwconv_grad_weight_workspace_floats(int64_t M, int64_t N, int64_t S);
int sjhip_pwconv_grad_weight(const float *dy, int dy_terms, const float *x, int x_terms, int64_t S, int64_t M, int64_t N,
                             int64_t L, float *dw, float *workspace, void *stream);

/*
 * The same three GEMMs (same reference lines: layer/attention.py:310-329, model/spikformer.py:85-99) with the fp32
 * operands split into two fp16 terms and the three products hi*hi, hi*lo, lo*hi on v_mfma_f32_32x32x16_f16: half the
 * matrix-core work of the three-term bf16 split at the same accuracy class.  fp16 has 11 significant bits but a narrow
 * exponent range, so every operand is scaled by a power of two first (exact) and the scales are taken out of the result
 * (exact): weights per row of A, inside sjhip_pwconv_split_weight_f16; activations and gradients by the power of two
 * that takes a largest finite magnitude `amax` into [2^14, 2^15) (1 for a zero or subnormal amax; infinities and NaNs take
 * no part in it and propagate through the products as in fp32).  Which magnitude: in sjhip_pwconv_gemm_f16, whose output
 * columns are (sample, position) pairs, every sample s of b is scaled by its own amax (the scale leaves the sum over k
 * of a column untouched), so a sample whose values are all small beside another's keeps its significant bits; in the
 * weight gradient, which sums over samples and positions, by the amax of the whole tensor (what a small sample adds to
 * that sum is small beside the rest).  The kernels derive both from one device buffer per tensor of
 * sjhip_pwconv_amax_floats(S) = SJHIP_PW_AMAX_FLOATS + SJHIP_PW_AMAX_SAMPLE_WORDS * S non-negative floats, 16-byte
 * aligned: the first SJHIP_PW_AMAX_FLOATS words have the tensor's amax as their maximum (several words, so that the
 * blocks that fold their maxima into it do not meet on one address), and the amax of sample s is the maximum of the
 * words SJHIP_PW_AMAX_FLOATS + SJHIP_PW_AMAX_SAMPLE_WORDS * s + r, r < SJHIP_PW_AMAX_SAMPLE_WORDS.  An element above
 * 2^-16 of the amax it is scaled by is represented to 2^-23 relative or better, a smaller one to 2^-39 of that amax
 * (within one sample the spread between positions is not compensated: a token column whose values all lie below 2^-17
 * of its sample's amax loses significant bits; configure the bf16 split, which has fp32's exponent range, for such
 * data); the dropped product lo*lo is below 2^-22 of hi*hi.  Measured
 * against float64 on operands whose rows span four decades: 2^-23 of sum |a||b| (three bf16 terms: 2^-26; an fp32 dot
 * product of 384 terms: 2^-20).  An operand that fp16 holds exactly (spikes, integers up to 2048) takes one term and no
 * scale (terms = 1, amax = NULL).
 *
 *   sjhip_pwconv_split_weight_f16  planes: an opaque buffer of sjhip_pwconv_planes_elems(rows, cols) 2-byte elements,
 *                                  16-byte aligned (two fp16 planes in the tile order of sjhip_pwconv_split_weight,
 *                                  then the inverse row scales); amax_reset: NULL, or an amax buffer for
 *                                  amax_reset_samples samples that the launch also sets to zero (that of the
 *                                  activations the planes will multiply, so that no launch is spent on clearing it)
 *   sjhip_pwconv_amax              folds max |x| over the finite ones of the elements of x (S samples of per_sample
 *                                  elements each) into amax[sjhip_pwconv_amax_floats(S)]: afterwards the maximum of
 *                                  the first SJHIP_PW_AMAX_FLOATS words is the larger of what it was and max |x|, and
 *                                  the maximum of the words of sample s likewise for that sample; all zero before the
 *                                  first call for a tensor; one launch
 *   sjhip_pwconv_gemm_f16          sjhip_pwconv_gemm / sjhip_pwconv_gemm_stats (partial != NULL) on fp16 planes;
 *                                  b_terms 2 with the b_amax buffer of b (sjhip_pwconv_amax_floats(S) floats; larger
 *                                  maxima are safe, smaller ones are not), or 1 with NULL
 *   sjhip_pwconv_grad_weight_f16   sjhip_pwconv_grad_weight with two terms of dy (dy_amax) and x_terms of x
 */
#define SJHIP_PW_F16 16          /* internal term code of an fp16 operand: SJHIP_PW_F16 | terms */
#define SJHIP_PW_AMAX_FLOATS 256
#define SJHIP_PW_AMAX_SAMPLE_WORDS 16 /* words per sample (blocks that meet on one address fold one after the other) */
int64_t sjhip_pwconv_amax_floats(int64_t S);
int sjhip_pwconv_split_weight_f16(const float *w, int64_t rows, int64_t cols, int transpose, uint16_t *planes, float *amax_reset,
                                  int64_t amax_reset_samples, void *stream);
int sjhip_pwconv_amax(const float *x, int64_t S, int64_t per_sample, float *amax, void *stream);
int sjhip_pwconv_gemm_f16(const uint16_t *a_planes, int64_t M, int64_t K, const float *b, int b_terms, const float *b_amax,
                          int64_t S, int64_t L, float *c, float *partial, void *stream);
int sjhip_pwconv_grad_weight_f16(const float *dy, const float *dy_amax, const float *x, int x_terms, const float *x_amax,
                                 int64_t S, int64_t M, int64_t N, int64_t L, float *dw, float *workspace, void *stream);
/* The two of them that read a spike tensor, with the spikes bit-packed (the layout of sjhip_bit_pack over the flattened
 * [S][K][L] or [S][N][L] tensor: 1/32 of the bytes of fp32 spikes): the projection convolution of the reference's
 * SpikingSelfAttention reads the attention neuron's spikes (layer/attention.py:378-384), which that neuron can write as
 * bits (sjhip_neuron_forward_packed).  K * L (N * L) must be a multiple of 8, L even (a multiple of 4 for the weight
 * gradient); results equal those of the fp32-spike calls bit for bit. */
int sjhip_pwconv_gemm_f16_bits(const uint16_t *a_planes, int64_t M, int64_t K, const uint8_t *b_bits, int64_t S, int64_t L,
                               float *c, float *partial, void *stream);
int sjhip_pwconv_grad_weight_f16_bits(const float *dy, const float *dy_amax, const uint8_t *x_bits, int64_t S, int64_t M,
                                      int64_t N, int64_t L, float *dw, float *workspace, void *stream);

/*
 * The same GEMMs with the activations / gradients arriving as fp16 term planes that their producer wrote already scaled
 * and split (sjhip_pwconv_split_planes), instead of
 * fp32 tensors that every block of a GEMM splits again while it stages them (same reference lines:
 * layer/attention.py:310-329, model/spikformer.py:85-99).  A plane buffer of a tensor x [S][C][L] holds `terms` planes
 * [C][ld] of fp16, ld = S * L rounded up to a multiple of 8 (16-byte aligned rows): element (c, s * L + l) of plane 0 is
 * fp16(scale x[s][c][l]), of plane 1 fp16 of the remainder; scale is the power of two that the tensor's amax buffer gives
 * (the tensor's amax, the first SJHIP_PW_AMAX_FLOATS words of its buffer: planes carry one scale for all their uses), so the
 * same amax buffer must accompany the planes into every GEMM that reads them.  The
 * columns beyond S * L are never read as data.  The channel-major layout makes the columns of all samples one contiguous
 * contraction (weight gradient) or output (forward, input gradient) index; results agree with the *_f16 calls to the
 * rounding of the fp32 accumulation order.
 *
 *   sjhip_pwconv_plane_elems       2-byte elements of the plane buffer of x [S][C][L] with `terms` (1 or 2) terms
 *   sjhip_pwconv_split_planes      planes of x; terms 2 with the amax buffer of x (sjhip_pwconv_amax), or 1 (values that
 *                                  fp16 holds exactly; amax NULL); L a multiple of 4, 16-byte aligned buffers
 *   sjhip_pwconv_gemm_planes       c[s][m][l] = sum_k A[m][k] b[s][k][l] from fp16 weight planes
 *                                  (sjhip_pwconv_split_weight_f16) and the planes of b; partial as in
 *                                  sjhip_pwconv_gemm_stats with sjhip_pwconv_gemm_planes_stats_rows(S, L) rows, or NULL;
 *                                  any L
 *   sjhip_pwconv_grad_weight_planes  dw[m][n] = sum_{s,l} dy[s][m][l] x[s][n][l] from the planes of dy (two terms) and of
 *                                  x (x_terms); workspace of sjhip_pwconv_grad_weight_planes_workspace_floats floats
 */
int64_t sjhip_pwconv_plane_elems(int64_t S, int64_t C, int64_t L, int terms);
int sjhip_pwconv_split_planes(const float *x, int64_t S, int64_t C, int64_t L, int terms, const float *amax, uint16_t *planes,
                              void *stream);
int64_t sjhip_pwconv_gemm_planes_stats_rows(int64_t S, int64_t L);
int sjhip_pwconv_gemm_planes(const uint16_t *a_planes, int64_t M, int64_t K, const uint16_t *b_planes, int b_terms,
                             const float *b_amax, int64_t S, int64_t L, float *c, float *partial, void *stream);
int64_t sjhip_pwconv_grad_weight_planes_workspace_floats(int64_t M, int64_t N, int64_t S, int64_t L);
int sjhip_pwconv_grad_weight_planes(const uint16_t *dy_planes, const float *dy_amax, const uint16_t *x_planes, int x_terms,
                                    const float *x_amax, int64_t S, int64_t M, int64_t N, int64_t L, float *dw, float *workspace,
                                    void *stream);

/*
 * Batch normalisation fused with the multi-step IF / LIF neuron behind it, for fp32 activations [T][B][C][L]
 * (L contiguous, a multiple of 4).  Stands in for nn.BatchNorm1d / nn.BatchNorm2d followed by LIFNode in the reference's
 * SpikingSelfAttention (layer/attention.py:314-329, 370-384) and SpikformerConv2dBNLIF (model/spikformer.py:196-212),
 * which torch runs as separate passes; here the normalised tensor is never written.
 *
 *   sjhip_bn_stats      partial[s][c] = (sum_l y, sum_l y^2) of every row of y [S][C][L]          (training forward)
 *   sjhip_bn_finalize   per channel: mean and biased variance from the partial sums (fp64), or, with partial == NULL
 *                       (evaluation), from running_mean / running_var; writes the affine map z = y scale + shift
 *                       (scale = gamma / sqrt(var + eps), shift = beta - mean scale; gamma / beta may be NULL = 1 / 0),
 *                       mean and invstd (kept for the backward), and in training updates running_mean / running_var in
 *                       place with `momentum` (unbiased variance), when they are given, and adds 1 to *batches_tracked
 *                       (nn.BatchNorm's num_batches_tracked, an int64 on the device), when that is given
 *   sjhip_bn_lif_forward   z = y scale_c + shift_c, then charge / fire / reset over the T steps (same arithmetic and
 *                       params as sjhip_neuron_forward; neuron IF or LIF); spikes go to spike_seq [T][B][C][L] (fp32) or
 *                       bit-packed to spike_bits (the layout of sjhip_bit_pack; B*C*L must be a multiple of 8): exactly
 *                       one of the two is given; v_last [B][C][L] or NULL
 *   sjhip_bn_lif_backward  replays the neuron from y (T <= 256; beyond 16 steps in pieces of 16), runs the BPTT recurrence of sjhip_neuron_backward with
 *                       grad_spike_seq and (optionally) grad_v_last, writes grad_z = dL/dz [T][B][C][L], grad_v_init
 *                       (or NULL) and partial[b][c] = (sum g, sum g y) over the row and all steps
 *   sjhip_bn_backward_finalize   dgamma, dbeta (either may be NULL) and coef [3][C] = (p, q, r) of dy = p g + q y + r;
 *                       training != 0: batch statistics took part in the forward, else q = r = 0; amax_reset: NULL, or
 *                       the amax buffer (sjhip_pwconv_amax_floats(T * B) floats) of a following sjhip_bn_grad_input_amax,
 *                       set to zero
 *   sjhip_bn_grad_input    dy = p_c g + q_c y + r_c over [S][C][L]; dy may be g
 */
int sjhip_bn_stats(const float *y, int64_t S, int64_t C, int64_t L, float *partial, void *stream);
int sjhip_bn_finalize(const float *partial, int64_t S, int64_t C, int64_t L, const float *gamma, const float *beta, float eps,
                      float momentum, float *running_mean, float *running_var, float *scale, float *shift, float *mean,
                      float *invstd, int64_t *batches_tracked, void *stream);
/* the same from partial [rows][C][2] that sum over `count` elements per channel (training mode only: partial != NULL) */
int sjhip_bn_finalize_rows(const float *partial, int64_t rows, int64_t count, int64_t C, const float *gamma, const float *beta,
                           float eps, float momentum, float *running_mean, float *running_var, float *scale, float *shift,
                           float *mean, float *invstd, int64_t *batches_tracked, void *stream);
int sjhip_bn_lif_forward(int neuron, const sjhip_neuron_params *p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                         const float *scale, const float *shift, const float *v_init, float *spike_seq, uint8_t *spike_bits,
                         float *v_last, void *stream);
int sjhip_bn_lif_backward(int neuron, const sjhip_neuron_params *p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                          const float *scale, const float *shift, const float *v_init, const float *grad_spike_seq,
                          const float *grad_v_last, float *grad_z, float *grad_v_init, float *partial, void *stream);
/* The same two calls with a ParametricLIFNode behind the batch norm (neuron/plif.py:14-261 in the place of the LIF of
 * layer/attention.py:310-329): k = sigmoid(w) is read from device memory (k_device, one float, as sjhip_neuron_forward
 * takes it), and the backward also leaves dL/dk in grad_k[0]: every wavefront writes its share of sum G_t dh_t/dk to
 * workspace (sjhip_bn_plif_backward_workspace_floats(B, C, L) floats), and one more launch adds the shares in fp64 in a
 * fixed order, as sjhip_neuron_backward does for PLIF.  params: as for SJHIP_NEURON_PLIF (tau is ignored). */
int sjhip_bn_plif_forward(const sjhip_neuron_params *p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                          const float *scale, const float *shift, const float *v_init, const float *k_device, float *spike_seq,
                          uint8_t *spike_bits, float *v_last, void *stream);
int64_t sjhip_bn_plif_backward_workspace_floats(int64_t B, int64_t C, int64_t L);
int sjhip_bn_plif_backward(const sjhip_neuron_params *p, int64_t T, int64_t B, int64_t C, int64_t L, const float *y,
                           const float *scale, const float *shift, const float *v_init, const float *k_device,
                           const float *grad_spike_seq, const float *grad_v_last, float *grad_z, float *grad_v_init,
                           float *partial, float *grad_k, float *workspace, void *stream);
int sjhip_bn_backward_finalize(const float *partial, int64_t T, int64_t B, int64_t C, int64_t L, int training, const float *gamma,
                               const float *mean, const float *invstd, float *dgamma, float *dbeta, float *coef, float *amax_reset,
                               void *stream);
int sjhip_bn_grad_input(const float *g, const float *y, const float *coef, int64_t S, int64_t C, int64_t L, float *dy, void *stream);
/* sjhip_bn_grad_input that also folds max |dy| into amax as sjhip_pwconv_amax(dy, S, C * L) would (same contract:
 * sjhip_pwconv_amax_floats(S) floats, zero before the call): the fp16 GEMMs that consume dy (the two gradients of the convolution in front of the
 * batch norm, layer/attention.py:314-319 run backwards) then need no pass of their own over it. */
int sjhip_bn_grad_input_amax(const float *g, const float *y, const float *coef, int64_t S, int64_t C, int64_t L, float *dy,
                             float *amax, void *stream);

/*
 * Launch tuning (process-wide, read at launch).  Keys: "fwd_block" / "bwd_block" = work-items per
 * block (64, 128, 256 or 512); "fwd_blocks_per_cu" / "bwd_blocks_per_cu" = cap on resident blocks per
 * compute unit (0 = none, else 2..64; enforced through a dynamic-LDS request), and
 * "replay_blocks_per_cu" likewise for sjhip_neuron_backward_recompute.  The forward cap applies to
 * fp32 storage with v_seq or h_seq written (spikes-only and 16-bit forwards always run uncapped); it is
 * doubled for T < 16 and dropped for T < 4, where few rows are in flight per work-item.  Returns SJHIP_ERR_INVALID otherwise.
 * "column_spread" = which columns a block of the neuron kernels takes: 0 = block b takes chunk b of a row (each XCD
 * every eighth chunk), 1 = each XCD one contiguous eighth of the row, 2 (default) = order 0 except for row strides that
 * are a multiple of 4 KiB with odd parity of address bits 12 and 20, where it measured 20 to 35 % slower: there the
 * XCDs take runs of 256 consecutive blocks in turn and the block size follows the stride (256 or 128 work-items,
 * whatever the block keys say); 4 ... 65536 = runs of that many blocks at every stride.
 * Results never depend on these.
 */
int sjhip_set_tuning(const char *key, int value);
int sjhip_get_tuning(const char *key);

/*
 * Bandwidth probe: a plain streaming kernel with `reads` input and `writes` output streams of floats_per_stream fp32
 * each (0..3 of each; the instantiated mixes are r:w = 1:0 2:0 3:0 0:1 0:2 0:3 1:1 1:2 1:3 2:1 3:1), one 16-byte access
 * per work-item and stream, default or (nontemporal != 0) streaming cache policy.  in / out are host arrays of device
 * pointers (a read-only probe still takes one output pointer, which it never writes).  No counterpart in the
 * reference: it measures the ceilings the neuron kernels' bandwidth is compared with, on the device and in the run
 * that measures them (kernel class 13 of sjhip_profile_read).
 */
int sjhip_stream_probe(int reads, int writes, int nontemporal, int64_t floats_per_stream, const float *const *in,
                       float *const *out, void *stream);

/*
 * Matrix-core probe: sjhip_mfma_probe_blocks(w) blocks (compute units x w, each four wavefronts, one per SIMD) issue
 * iterations x 16 v_mfma_f32_32x32x16_f16 per wavefront on register operands and nothing else: 2 x 32 x 32 x 16 flop
 * per instruction.  operands: 0 all zero, 1 uniform random in [-1, 1) (the clock, and with it the sustained rate,
 * depends on what the matrix cores are fed).  Every block writes one float to sink (at least that many floats).
 * No counterpart in the reference: like sjhip_stream_probe it measures, on the device and in the run that quotes it,
 * the ceiling that the convolution GEMMs' rate is compared with (kernel class 14 of sjhip_profile_read).
 */
int64_t sjhip_mfma_probe_blocks(int wavefronts_per_simd);
int sjhip_mfma_probe(int operands, int wavefronts_per_simd, int iterations, float *sink, int64_t sink_floats, void *stream);

/*
 * Optional per-kernel timing.  While enabled every launch is bracketed by HIP events on its own
 * stream.  sjhip_profile_read() synchronises those events and returns, for kernel class `which`
 * (0 forward, 1 backward, 2 plif-reduce, 3 bit_pack, 4 bit_unpack, 5 ssa forward, 6 ssa backward, 7 pwconv gemm,
 * 8 pwconv grad_weight, 9 bn stats, 10 bn_lif forward, 11 bn_lif backward, 12 bn grad_input, 13 stream probe, 14 matrix-core probe), the launch count and total
 * milliseconds since the last sjhip_profile_reset().
 */
int sjhip_profile_enable(int on);
int sjhip_profile_reset(void);
int sjhip_profile_read(int which, int64_t *launches, double *total_ms);

#ifdef __cplusplus
}
#endif
#endif /* SJHIP_H_ */
