"""Process-wide switches of the hip backend (counterpart of the reference's
``spikingjelly/configure.py``, which holds ``cuda_threads`` and compiler options
for its CuPy/Triton backends).

``hip_half_precision_mode``
    How fp16/bf16 inputs are computed by ``backend='hip'``:
    ``"torch"`` rounds the result of every arithmetic op to the storage dtype and
    keeps the membrane potential in it -- bit-identical to ``backend='torch'`` on
    the same half tensors; ``"fp32_state"`` keeps state and arithmetic in fp32 and
    rounds only what is stored (the reference's mixed-precision Triton ops).

``hip_lif_reciprocal_tau``
    ``False`` (default): LIF charges with an IEEE division by ``tau``: the spikes of
    ``backend='torch'`` run on the CPU, which is what the parity tests compare with.
    ``True``: multiply by ``fl(1/tau)``: the spikes of the reference's CuPy / Triton
    kernels and of ``backend='torch'`` run on a GPU (torch divides a device tensor by
    a Python scalar as a multiplication by its reciprocal).  Identical when ``tau`` is
    a power of two; for other values (3.0, 5.0, ...) about a third of the fp32 charges
    differ in the last bit and a few spikes with them, so pick the one whose results
    you are reproducing.

``hip_plif_atomic_reduce``
    ``False``: the PLIF ``dL/dk`` sum is reduced in a fixed order (bitwise
    reproducible).  ``True``: one ``atomicAdd`` per block, order varies run to run.

``hip_backward_recompute``
    ``True``: training forwards write no ``h_seq``; the backward kernel replays the forward from
    ``x_seq`` and ``v_init`` (bit-identical ``h``, held in LDS), so autograd keeps ``x_seq`` alive
    instead of a same-sized ``h_seq`` and the forward's largest write disappears.  Used whenever the
    library prefers it for the shape (``sjhip_recompute_preferred``: ``N`` a multiple of the 128-bit
    vector width and the sequence short enough for the replayed ``h`` to stay in LDS with enough
    resident wavefronts); other shapes and ``False`` fall back to saving ``h_seq``.
"""

hip_half_precision_mode = "torch"
# How the fp32 operands of the fused kernel-size-1 convolutions reach the 16-bit matrix cores (hip_kernel/conv_bn_lif.py).
# "f16": two fp16 terms of operands scaled by powers of two (weights per row, activations and gradients per tensor, from
# a pass that finds the largest magnitude), three products per pair of real operands, two when one operand is spikes;
# accuracy of an fp32 GEMM (2^-23 of sum |a||b| measured).  "bf16": hip_conv_terms bf16 terms, no scaling, no extra pass.
hip_conv_split = "f16"
# True: where a hip LIF feeds a fused kernel-size-1 convolution + batch norm + LIF (the attention neuron and the projection
# of the spiking self-attention), the first neuron writes its spikes bit-packed and the convolution GEMMs read the bits:
# the spikes never exist as a float tensor (needs hip_conv_split = "f16").  False: dense fp32 spikes between the two.
hip_conv_bit_spikes = True
# True: the weight gradient of a fused convolution runs on a second stream beside its input gradient (they only share
# their inputs), so that the blocks of one kernel fill the compute units that the last, partly filled round of the
# other leaves idle.  False (default): one after the other on the caller's stream.  It paid while the GEMM kernel kept
# two blocks per compute unit (config 5: 1.51 -> 1.49 ms per step); with three it measures 1.47 ms either way (1.473,
# 1.477, 1.467 against 1.466, 1.462, 1.463), so the simpler schedule is the default.
hip_conv_overlap_gradients = False
# Number of bf16 terms with hip_conv_split = "bf16": 3 keeps the accuracy of an fp32 GEMM (six matrix-core products per
# pair of real operands, three when one operand is spikes), 2 gives about 2^-17 relative per product at half the
# products, 1 is a plain bf16 GEMM.
hip_conv_terms = 3
# False: modules keep torch's convolution and batch norm around the hip neurons even where the fused
# convolution / batch norm / LIF kernels could serve the chain (layer/fused.py).
hip_fuse_conv_bn_lif = True
# True: the spiking self-attention feeds the contraction's output of every step straight into its `attn_lif` inside one
# kernel (`sjhip_ssa_lif_forward_packed` / `_backward_packed`) where that kernel can serve, instead of writing the output
# and running the neuron as a launch of its own.  Same results; off by default because it measured no faster (what
# bounds the kernels on both sides is not the bytes the fusion saves).
hip_fuse_ssa_lif = False
hip_backward_recompute = True
# Sequences longer than the replaying backward prefers in one piece (its LDS buffer for h grows with T) run, outside a
# tracing compiler, as pieces of this many steps: the forward leaves the state after every piece ([T / chunk, N], in
# place of a [T, N] h_seq), the backward replays piece by piece from those checkpoints.  0 switches it off (such
# sequences then save h_seq).
hip_replay_chunk = 16
hip_lif_reciprocal_tau = False
hip_plif_atomic_reduce = False

# ``save_bool_spike_level`` (same name and meaning as the reference's ``configure.py:59-67``): how the spike operators
# of ``hip_kernel/spike_op.py`` keep their binary input for the backward.  0: as ``torch.bool`` (one byte per spike);
# 1: bit-packed, eight spikes per byte (``hip_kernel/tensor_cache.float_spike_to_bool``).
save_bool_spike_level = 0

# ``save_spike_as_bool_in_neuron_kernel`` (the reference's ``configure.py:54``: its QIF / EIF / Izhikevich CuPy kernels
# may keep the forward's spikes as bools for the backward, ``qif.py:437,471``).  Kept for callers that set it; the hip
# backward keeps no spikes at all (it recomputes them from ``h``), so the value changes nothing here.
save_spike_as_bool_in_neuron_kernel = False
