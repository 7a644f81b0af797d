"""Headline benchmark: multi-step LIF forward+backward, T=16, N=33.5M neurons, fp32, one MI355X.

One "step" is one forward plus one backward of ``LIFNode(step_mode='m', backend='hip',
store_v_seq=True)`` over x [16,256,128,32,32] (tau=2, hard reset to 0, ATan(2)), with upstream
gradients for both the spikes and v_seq, inputs resident in HBM.  Prints ONE JSON line:
``value`` = T*N / seconds per step (neuron-steps/s); ``roofline`` = algorithmic bytes of the slower of
the two kernels / its mean duration measured with HIP events on the launch stream, against the 8 TB/s
HBM3E peak; ``cpu_baseline`` = the torch-ops port of the reference's CPU backend timed on this host on
a bounded sample of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
T_STEPS = 16
SHAPE = (T_STEPS, 256, 128, 32, 32)


def cpu_baseline(torch, sample_neurons: int, repeats: int, threads: int = 0):
    """torch-ops port of the reference torch backend (oracle/neuron_oracle.py), forward + autograd
    backward, on ``sample_neurons`` neurons x T=16 of the same input distribution; ``threads``: intra-op threads for
    this measurement (0: as torch is configured)."""
    from oracle import neuron_oracle as no

    before = torch.get_num_threads()
    if threads > 0:
        torch.set_num_threads(threads)
    try:
        return _cpu_baseline(torch, no, sample_neurons, repeats)
    finally:
        torch.set_num_threads(before)


def _cpu_baseline(torch, no, sample_neurons: int, repeats: int):
    cores = torch.get_num_threads()
    g = torch.Generator().manual_seed(1002)
    x = torch.randn((T_STEPS, sample_neurons), generator=g) * 0.8 + 0.3
    gs = torch.randn((T_STEPS, sample_neurons), generator=g)
    gv = torch.randn((T_STEPS, sample_neurons), generator=g) * 0.1
    v0 = torch.zeros(sample_neurons)
    times = []
    for i in range(repeats + 1):
        t0 = time.perf_counter()
        no.forward_backward("lif", x, v0, gs, gv, None, 2.0, True, 1.0, 0.0, "atan", 2.0, False)
        dt = time.perf_counter() - t0
        if i > 0:  # first run is the warm-up
            times.append(dt)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": T_STEPS * sample_neurons / med,
        "unit": "neuron-steps/s",
        "cores": cores,
        "kind": "port",
        "sample": f"N={sample_neurons} neurons x T={T_STEPS}, fwd+autograd bwd, median of {repeats} after 1 warm-up, "
                  f"{med * 1e3:.0f} ms each",
    }


# source files whose kernels the counter-measured traffic in profiles/traffic_*.json belongs to
TRAFFIC_SOURCES = ("neuron_fwd.h", "neuron_bwd.h", "neuron_bwd_recompute.h", "neuron_bwd_recompute_launch.h", "sjhip_common.h")


def kernel_source_digest() -> str:
    """sha256 over the sources of the forward / backward kernels: the recorded HBM traffic is reported only while it
    still describes the kernels that run (an edit to any of these files makes it stale)."""
    import hashlib

    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        with open(os.path.join(ROOT, "spikingjelly_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def recorded_traffic():
    """The rocprofv3 FETCH_SIZE / WRITE_SIZE record of the headline kernels, or None when it is missing or stale."""
    path = os.path.join(ROOT, "profiles", "traffic_lif_fp32_T16_N33554432.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        rec = json.load(f)
    return rec if rec.get("kernel_source_sha256") == kernel_source_digest() else None


def measure_mfma_ceiling(torch, L, random_operands: bool = True, iterations: int = 20000, repeats: int = 3):
    """TFLOP/s that the matrix cores sustain on v_mfma_f32_32x32x16_f16 alone (sjhip_mfma_probe: one wavefront per SIMD
    issuing nothing else, register operands), here and now: the chip lowers its clock under their power draw, by how much
    depends on the operands, so the published 2.5 PFLOP/s is not what a kernel on real data can be held against."""
    sink = torch.empty(4096, dtype=torch.float32, device="cuda:0")
    L.mfma_probe(random_operands, 1, 2000, sink)
    torch.cuda.synchronize()
    L.profile_reset()
    L.profile_enable(True)
    flop = 0
    for _ in range(repeats):
        flop = L.mfma_probe(random_operands, 1, iterations, sink)
    torch.cuda.synchronize()
    L.profile_enable(False)
    n, ms = L.profile_read(L.KC_MFMA_PROBE)
    return flop / (ms / max(n, 1) * 1e-3) / 1e12


def measure_ceilings(torch, L, floats_per_stream: int, repeats: int = 5):
    """GB/s of the library's plain streaming kernel (sjhip_stream_probe) for the access mixes of the neuron kernels,
    over streams of the size of one [T, N] tensor of the workload; best cache policy of the two for each mix."""
    dev = torch.device("cuda:0")
    bufs = [torch.empty(floats_per_stream, dtype=torch.float32, device=dev) for _ in range(4)]
    for b in bufs[:3]:
        b.fill_(0.5)
    mixes = {"read_1r0w": (1, 0), "write_0r1w": (0, 1), "copy_1r1w": (1, 1), "forward_1r2w": (1, 2),
             "forward_saving_h_1r3w": (1, 3), "backward_3r1w": (3, 1)}
    out = {}
    for name, (r, w) in mixes.items():
        best = 0.0
        for nt in (False, True):
            ins, outs = bufs[:r], bufs[r:r + max(w, 1)]  # a read-only probe still takes one (unwritten) output
            for _ in range(2):
                L.stream_probe(r, w, nt, ins, outs)
            torch.cuda.synchronize()
            L.profile_reset()
            L.profile_enable(True)
            for _ in range(repeats):
                L.stream_probe(r, w, nt, ins, outs)
            torch.cuda.synchronize()
            L.profile_enable(False)
            n, ms = L.profile_read(L.KC_STREAM_PROBE)
            gbs = (r + w) * floats_per_stream * 4 / (ms / max(n, 1) * 1e-3) / 1e9
            best = max(best, gbs)
        out[name] = best
    del bufs
    torch.cuda.empty_cache()
    return out


class _quiet_collector:
    """Python's cyclic garbage collector off for a timed region (as ``timeit`` does): with torch imported a full
    collection takes 70-80 ms of host time, and whether one falls among twenty timed steps depends on how many objects
    the process happened to allocate before (measured: 0.29 against 4.4 ms per step for the same 20 steps of configs[2])."""

    def __enter__(self):
        import gc

        gc.collect()
        self.was_enabled = gc.isenabled()
        gc.disable()

    def __exit__(self, *exc):
        import gc

        if self.was_enabled:
            gc.enable()


def _time_steps(torch, L, step, steps, warmup):
    """warm-up, then `steps` timed steps bracketed by synchronisation, then the same steps once more under the library's
    event profiler for the per-kernel durations: its two events per launch would otherwise sit in the timed region of
    workloads with dozens of short launches per step (the attention block: 1.88 against 1.77 ms per step)."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    with _quiet_collector():
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    L.profile_reset()
    L.profile_enable(True)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    L.profile_enable(False)
    return elapsed


def _kernel_ms(L, which):
    n, ms = L.profile_read(which)
    return ms / max(n, 1)


def _emit(args, metric, unit, value, elapsed, dtype, config, roofline):
    line = {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic", "config": config, "roofline": roofline}
    collect = getattr(args, "collect", None)
    if collect is not None:  # a secondary measurement inside the default run: kept for the headline's JSON line
        collect.append(line)
    else:
        print(json.dumps(line))


def secondary_measurements(args):
    """BASELINE configs[2], [3] and [4] timed after the headline (a few hundred ms in all), condensed for the
    ``secondary`` object of the default JSON line: ms per step, the metric value, and the dominant kernel with its
    duration and its fraction of the roofline that bounds it."""
    import copy

    out = {}
    for name in ("config3", "config4", "config5"):
        sub = copy.copy(args)
        sub.workload, sub.steps, sub.warmup, sub.collect = name, 20, 5, []
        other_workload(sub)
        line = sub.collect[0]
        r = line["roofline"]
        out[name] = {"metric": line["metric"], "value": line["value"], "unit": line["unit"], "ms_per_step": line["ms_per_step"],
                     "kernel": r["kernel"], "kernel_ms": r["kernel_ms"], "bound": r["bound"], "achieved": r["achieved"],
                     "peak": r["peak"], "roofline_unit": r["unit"], "frac": r["frac"]}
        for extra in ("forward_ms", "backward_ms", "graph_replay_ms_per_step", "fused_forward_packed_ms", "fused_forward_packed_GBs", "gemm_ms_per_step",
                      "ssa_backward_ms", "ssa_backward_GBs", "mfma_sustained_random_operands_TFLOPs", "frac_of_sustained"):
            if extra in r:
                out[name][extra] = r[extra]
    return out


def other_workload(args) -> int:
    """Secondary workloads (BASELINE configs 3-5), same JSON shape; parity for them lives in tests/."""
    import torch

    from spikingjelly_amd import configure
    from spikingjelly_amd.activation_based import functional, layer, neuron, surrogate
    from spikingjelly_amd.activation_based.hip_kernel import library as L
    from spikingjelly_amd.activation_based.hip_kernel.compress import bit_spike_compress, bit_spike_decompress

    L.load()
    dev = torch.device("cuda:0")

    def randn(shape, seed, mean, std, dtype):
        g = torch.Generator().manual_seed(seed)
        return (torch.randn(shape, generator=g) * std + mean).to(dtype).to(dev)

    if args.workload == "config3":
        shape = (8, 128, 256, 16, 16)
        T, N = shape[0], 128 * 256 * 16 * 16
        configure.hip_half_precision_mode = "fp32_state"
        x = randn(shape, 1003, 0.2, 1.0, torch.bfloat16).requires_grad_()
        gs = randn(shape, 1103, 0.0, 1.0, torch.bfloat16)
        gv = randn(shape, 1203, 0.0, 0.1, torch.bfloat16)
        node = neuron.ParametricLIFNode(init_tau=2.0, v_reset=None, surrogate_function=surrogate.Sigmoid(4.0),
                                        step_mode="m", backend="hip", store_v_seq=True).to(dev)

        def step():
            s = node(x)
            torch.autograd.backward([s, node.v_seq], [gs, gv])
            x.grad = None
            node.w.grad = None
            functional.reset_net(node)

        elapsed = _time_steps(torch, L, step, args.steps, args.warmup)
        f_ms, b_ms = _kernel_ms(L, L.KC_FORWARD), _kernel_ms(L, L.KC_BACKWARD)
        plif_reduce_ms = _kernel_ms(L, L.KC_PLIF_REDUCE)
        # The same step recorded into a HIP graph and replayed: at this size the Python around the launches (0.2-0.3 ms
        # per step) is longer than the kernels (0.17 ms), and a replay issues them without it.  (Replays of the recorded
        # step on its static input; a caller with new data per step adds the copy into that buffer.)
        from spikingjelly_amd.activation_based.hip_kernel.graph import GraphedStep

        eager_spikes = node(x).detach().clone()
        functional.reset_net(node)

        def recorded(xs):
            s = node(xs)
            torch.autograd.backward([s, node.v_seq], [gs, gv])
            functional.reset_net(node)
            return s

        graphed = GraphedStep(recorded, [x], parameters=[node.w])
        for _ in range(args.warmup):
            graphed.graph.replay()
        torch.cuda.synchronize()
        with _quiet_collector():
            t0 = time.perf_counter()
            for _ in range(args.steps):
                graphed.graph.replay()
            torch.cuda.synchronize()
            graph_elapsed = time.perf_counter() - t0
        assert torch.equal(graphed.static_outputs.detach(), eager_spikes)
        bytes_each = 8 * T * N + 2 * N  # 4 tensors x 2 B per step + one [N] state
        dom = "forward" if f_ms >= b_ms else "backward"
        d_ms = max(f_ms, b_ms)
        _emit(args, "neuron-steps/sec PLIF fwd+bwd bf16 storage / fp32 state, T=8 N=8.4M, 1 MI355X", "neuron-steps/s",
              T * N / (elapsed / args.steps), elapsed, "f32",
              {"workload": "configs[2]: ParametricLIFNode init_tau=2, soft reset, Sigmoid(4), x [8,128,256,16,16] bf16, "
                           "store_v_seq=True, incl. dL/dw reduction", "T": T, "N": N},
              {"bound": "hbm", "achieved": bytes_each / (d_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
               "frac": bytes_each / (d_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel": dom,
               "kernel_ms": d_ms, "algorithmic_bytes": bytes_each, "forward_ms": f_ms, "backward_ms": b_ms,
               "plif_reduce_ms": plif_reduce_ms, "graph_replay_ms_per_step": graph_elapsed / args.steps * 1e3,
               "graph_replay_neuron_steps_per_s": T * N / (graph_elapsed / args.steps)})
        return 0

    if args.workload in ("qif", "ilif", "eif", "izhikevich"):
        # the config-2 shape with another neuron of the same kernels: the quadratic integrate-and-fire neuron
        # (state-dependent dh/dv in the backward) or the integer-valued LIF (multi-level counts, windowed gradient)
        shape = (16, 256, 128, 32, 32)
        T, N = shape[0], 256 * 128 * 32 * 32
        g = torch.Generator(device=dev).manual_seed(1002)
        if args.workload == "qif":
            x = (torch.randn(shape, generator=g, device=dev) * 0.4 + 0.3).requires_grad_()
            node = neuron.QIFNode(tau=2.0, surrogate_function=surrogate.ATan(2.0), step_mode="m", backend="hip",
                                  store_v_seq=True).to(dev)
            label, what = "QIF", "QIFNode tau=2, v_c=0.8, a0=1, hard reset -0.1, ATan(2), x [16,256,128,32,32] fp32 ~N(0.3,0.4)"
        elif args.workload == "eif":
            x = (torch.randn(shape, generator=g, device=dev) * 0.6 + 0.3).requires_grad_()
            node = neuron.EIFNode(tau=2.0, surrogate_function=surrogate.ATan(2.0), step_mode="m", backend="hip",
                                  store_v_seq=True).to(dev)
            label, what = "EIF", "EIFNode tau=2, delta_T=1, theta_rh=0.8, hard reset -0.1, ATan(2), x [16,256,128,32,32] fp32 ~N(0.3,0.6)"
        elif args.workload == "izhikevich":
            x = (torch.randn(shape, generator=g, device=dev) * 0.6 + 0.4).requires_grad_()
            node = neuron.IzhikevichNode(tau=2.0, a=0.3, b=0.2, tau_w=3.0, surrogate_function=surrogate.ATan(2.0),
                                         step_mode="m", backend="hip", store_v_seq=True).to(dev)
            label, what = "Izhikevich", ("IzhikevichNode tau=2, v_c=0.8, a0=1, tau_w=3, a=0.3, b=0.2, hard reset 0, ATan(2), "
                                         "x [16,256,128,32,32] fp32 ~N(0.4,0.6)")
        else:
            x = (torch.randn(shape, generator=g, device=dev) * 1.5 + 1.0).requires_grad_()
            node = neuron.ILIFNode(tau=4.0 / 3.0, surrogate_function=surrogate.MultiLevelSpikeCount(4), step_mode="m",
                                   backend="hip", store_v_seq=True).to(dev)
            label, what = "ILIF", "ILIFNode tau=4/3, v_th=1, counts 0..4, x [16,256,128,32,32] fp32 ~N(1.0,1.5)"
        gs = torch.randn(shape, generator=g, device=dev)
        gv = torch.randn(shape, generator=g, device=dev) * 0.1

        def step():
            s = node(x)
            torch.autograd.backward([s, node.v_seq], [gs, gv])
            x.grad = None
            functional.reset_net(node)

        elapsed = _time_steps(torch, L, step, args.steps, args.warmup)
        f_ms, b_ms = _kernel_ms(L, L.KC_FORWARD), _kernel_ms(L, L.KC_BACKWARD)
        bytes_each = 16 * T * N + 4 * N
        if args.workload == "izhikevich":
            bytes_each = 16 * T * N + 16 * N  # backward: grad_s, grad_v, x (replayed into h) in, grad_x out; two states in and out
        dom = "forward" if f_ms >= b_ms else "backward"
        d_ms = max(f_ms, b_ms)
        _emit(args, f"neuron-steps/sec {label} fwd+bwd fp32 T=16 N=33.5M, 1 MI355X", "neuron-steps/s",
              T * N / (elapsed / args.steps), elapsed, "f32",
              {"workload": what + ", store_v_seq=True, grad_spike ~N(0,1), grad_v ~N(0,0.1)", "T": T, "N": N},
              {"bound": "hbm", "achieved": bytes_each / (d_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
               "frac": bytes_each / (d_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel": dom,
               "kernel_ms": d_ms, "algorithmic_bytes": bytes_each, "forward_ms": f_ms, "backward_ms": b_ms})
        return 0

    if args.workload == "aaif":
        # activation-aware IF (inference), per-channel threshold and offset over the channel axis of [B, C, H, W]
        shape = (16, 256, 128, 32, 32)
        T, N = shape[0], 256 * 128 * 32 * 32
        g = torch.Generator(device=dev).manual_seed(1002)
        x = torch.randn(shape, generator=g, device=dev) * 0.5 + 0.2
        node = neuron.ActivationAwareIFNode(v_threshold=torch.linspace(0.5, 2.0, 128), v_offset=torch.linspace(-0.2, 0.2, 128),
                                            channel_dim=1, step_mode="m", backend="hip").to(dev).eval()

        def step():
            with torch.no_grad():
                out = node(x)
            functional.reset_net(node)
            return out

        elapsed = _time_steps(torch, L, step, args.steps, args.warmup)
        f_ms = _kernel_ms(L, L.KC_FORWARD)
        rate = float(step().mean())
        bytes_each = 8 * T * N + 4 * N  # x in, spike_seq out, v_last out
        _emit(args, "neuron-steps/sec activation-aware IF inference fp32 T=16 N=33.5M, 1 MI355X", "neuron-steps/s",
              T * N / (elapsed / args.steps), elapsed, "f32",
              {"workload": "ActivationAwareIFNode, 128 per-channel thresholds and offsets (channel_dim=1), soft reset, "
                           "x [16,256,128,32,32] fp32 ~N(0.2,0.5), eval", "T": T, "N": N, "firing_rate": rate},
              {"bound": "hbm", "achieved": bytes_each / (f_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
               "frac": bytes_each / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel": "aaif_forward",
               "kernel_ms": f_ms, "algorithmic_bytes": bytes_each})
        return 0

    if args.workload == "fp8":
        # the config-2 shape with 8-bit floating-point storage (mixed precision): x, v_seq, h_seq, grad_v in float8_e4m3fn,
        # spikes and their gradient in bf16, fp32 recurrence; the two operators are called directly so that the casts
        # a caller's dtypes may add stay outside the timed region
        from spikingjelly_amd.activation_based.hip_kernel import neuron_mp_kernel as M

        T, N = 16, 256 * 128 * 32 * 32
        g = torch.Generator(device=dev).manual_seed(1002)
        f8, sp = torch.float8_e4m3fn, torch.bfloat16
        x = (torch.randn((T, N), generator=g, device=dev) * 0.8 + 0.3).to(f8)
        v0 = torch.zeros((N,), device=dev).to(f8)
        gs = torch.randn((T, N), generator=g, device=dev).to(sp)
        gv = (torch.randn((T, N), generator=g, device=dev) * 0.1).to(f8)
        scalars = (L.NEURON_LIF, 2.0, True, 1.0, 0.0, False, False, 1, 2.0)
        rate = []

        def step():
            s, v_seq, h_seq = M.hip_multistep_mp_forward(x, v0, None, *scalars, f8, sp, True)
            M.hip_multistep_mp_backward(gs, gv, h_seq, v0, None, *scalars, sp, True)
            if not rate:
                rate.append(float(s.float().mean()))

        elapsed = _time_steps(torch, L, step, args.steps, args.warmup)
        f_ms, b_ms = _kernel_ms(L, L.KC_FORWARD), _kernel_ms(L, L.KC_BACKWARD)
        fwd_bytes = 5 * T * N + N          # x 1, spikes 2, v_seq 1, h_seq 1; v_init
        bwd_bytes = 5 * T * N + N          # grad_spike 2, grad_v 1, h_seq 1, grad_x 1 (storage dtype, as x is); grad_v_init
        dom, d_ms, d_bytes = ("forward", f_ms, fwd_bytes) if f_ms >= b_ms else ("backward", b_ms, bwd_bytes)
        _emit(args, "neuron-steps/sec LIF fwd+bwd float8_e4m3fn storage T=16 N=33.5M, 1 MI355X", "neuron-steps/s",
              T * N / (elapsed / args.steps), elapsed, "f32",
              {"workload": "sj::hip_multistep_mp_forward + _backward, LIF tau=2, hard reset 0, ATan(2), x [16, 33554432] "
                           "float8_e4m3fn ~N(0.3,0.8), spikes and grad_spike bf16, v_seq / h_seq / grad_v / grad_x float8_e4m3fn", "T": T, "N": N, "firing_rate": rate[0]},
              {"bound": "hbm", "achieved": d_bytes / (d_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
               "frac": d_bytes / (d_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel": dom, "kernel_ms": d_ms,
               "algorithmic_bytes": d_bytes, "forward_ms": f_ms, "backward_ms": b_ms,
               "forward_GBs": fwd_bytes / (f_ms * 1e-3) / 1e9, "backward_GBs": bwd_bytes / (b_ms * 1e-3) / 1e9})
        return 0

    if args.workload == "stbif":
        # SpikeZIP's signed ternary neuron (inference): the config-2 shape, the activation fed at the first step
        shape = (16, 256, 128, 32, 32)
        T, N = shape[0], 256 * 128 * 32 * 32
        g = torch.Generator(device=dev).manual_seed(1002)
        x = torch.zeros(shape, device=dev)
        x[0] = torch.randn(shape[1:], generator=g, device=dev) * 0.6
        node = neuron.STBIFNeuron(0.25, level=8, sym=True, step_mode="m").to(dev)
        node.backend = "hip"

        def step():
            with torch.no_grad():
                out = node(x)
            functional.reset_net(node)
            return out

        elapsed = _time_steps(torch, L, step, args.steps, args.warmup)
        f_ms = _kernel_ms(L, L.KC_FORWARD)
        out = step()
        want = torch.clamp(torch.floor(x[0].double() / 0.25 + 0.5), -4, 3) * 0.25
        assert float((out.sum(0).double() - want).abs().max()) <= 0.25  # the quantiser, up to fp32 boundary cases
        bytes_each = 8 * T * N + 12 * N  # x in, out_seq out; q, acc_q, cur_output out
        _emit(args, "neuron-steps/sec ST-BIF inference fp32 T=16 N=33.5M, 1 MI355X", "neuron-steps/s",
              T * N / (elapsed / args.steps), elapsed, "f32",
              {"workload": "STBIFNeuron(0.25, level=8, sym=True), x [16,256,128,32,32] fp32, x[0] ~N(0,0.6), zeros after, "
                           "fresh states; includes the is_work read-back", "T": T, "N": N},
              {"bound": "hbm", "achieved": bytes_each / (f_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
               "frac": bytes_each / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel": "stbif_forward",
               "kernel_ms": f_ms, "algorithmic_bytes": bytes_each})
        return 0

    if args.workload == "config4":
        shape = (32, 64, 512, 14, 14)
        T, N = shape[0], 64 * 512 * 14 * 14
        g = torch.Generator().manual_seed(1004)
        x = (torch.rand(shape, generator=g) * 0.25).half().to(dev)
        node = neuron.IFNode(v_threshold=1.0, v_reset=None, step_mode="m", backend="hip").to(dev).eval()

        def step():
            with torch.no_grad():
                s = node(x)
                packed = bit_spike_compress(s)
                back = bit_spike_decompress(packed, s.shape, dtype=torch.float16)
            functional.reset_net(node)
            return s, back

        elapsed = _time_steps(torch, L, step, args.steps, args.warmup)
        s, back = step()
        assert torch.equal(s, back)
        f_ms, p_ms, u_ms = _kernel_ms(L, L.KC_FORWARD), _kernel_ms(L, L.KC_BIT_PACK), _kernel_ms(L, L.KC_BIT_UNPACK)
        n = T * N
        fwd_bytes, pack_bytes, unpack_bytes = 4 * n + 4 * N, 2 * n + n // 8, n // 8 + 2 * n

        # the same work with the spikes bit-packed by the neuron kernel itself (no dense spike tensor, no pack pass)
        v0 = torch.zeros(shape[1:], dtype=torch.float16, device=dev)

        def fused_step():
            bits, _, _ = functional.if_multi_step_hip_packed(x, v0, 1.0, None)
            return bits, bit_spike_decompress(bits, x.shape, dtype=torch.float16)

        fused_elapsed = _time_steps(torch, L, fused_step, args.steps, args.warmup)
        fused_ms = _kernel_ms(L, L.KC_FORWARD)
        assert torch.equal(fused_step()[1], s)
        fused_bytes = 2 * n + n // 8 + 4 * N
        _emit(args, "neuron-steps/sec IF inference fp16 + spike bit-pack/unpack, T=32 N=6.4M, 1 MI355X", "neuron-steps/s",
              n / (elapsed / args.steps), elapsed, "f16",
              {"workload": "configs[3]: IFNode soft reset eval, x [32,64,512,14,14] fp16 uniform[0,0.25), then "
                           "bit_spike_compress + bit_spike_decompress(fp16)", "T": T, "N": N,
               "firing_rate": float(s.float().mean())},
              {"bound": "hbm", "achieved": fwd_bytes / (f_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
               "frac": fwd_bytes / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel": "forward(inference)",
               "kernel_ms": f_ms, "algorithmic_bytes": fwd_bytes,
               "pack_ms": p_ms, "pack_GBs": pack_bytes / (p_ms * 1e-3) / 1e9,
               "unpack_ms": u_ms, "unpack_GBs": unpack_bytes / (u_ms * 1e-3) / 1e9,
               "fused_forward_packed_ms": fused_ms, "fused_forward_packed_GBs": fused_bytes / (fused_ms * 1e-3) / 1e9,
               "fused_ms_per_step": fused_elapsed / args.steps * 1e3})
        return 0

    if args.workload == "ceilings":
        # what the memory system gives to plain streams of the config-2 tensor size (2.1 GB each)
        floats = 16 * 256 * 128 * 32 * 32
        t0 = time.perf_counter()
        c = measure_ceilings(torch, L, floats, repeats=args.steps)
        c["mfma_f16_zero_operands_TFLOPs"] = measure_mfma_ceiling(torch, L, False)
        c["mfma_f16_random_operands_TFLOPs"] = measure_mfma_ceiling(torch, L, True)
        elapsed = time.perf_counter() - t0
        top = max(v for k, v in c.items() if not k.startswith("mfma"))
        _emit(args, "GB/s of plain fp32 streams (sjhip_stream_probe), 2.1 GB per stream, 1 MI355X", "GB/s", top, elapsed, "f32",
              {"workload": "one 16-byte access per work-item and stream; read-only, write-only, copy and the read:write "
                           "mixes of the neuron kernels (1:2 forward, 1:3 forward saving h_seq, 3:1 backward); best of "
                           "default and streaming cache policy; mfma_*: what the matrix cores sustain on "
                           "v_mfma_f32_32x32x16_f16 alone (sjhip_mfma_probe)", **{k: round(v, 1) for k, v in c.items()}},
              {"bound": "hbm", "achieved": top, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": top / HBM_PEAK_GBS,
               "traffic": None, "kernel": "stream_probe"})
        return 0

    if args.workload == "pwconv":
        # the three GEMMs of the qkv convolution of configs[4] alone: Y = W X, dX = W^T dY, dW = sum dY X^T
        from spikingjelly_amd.activation_based.hip_kernel import conv_bn_lif as CB

        S, Cin, Cout, tokens = 256, 384, 1152, 196
        terms = args.terms if args.conv_split == "bf16" else CB.F16 | 2
        x = randn((S, Cin, tokens), 1, 0.0, 1.0, torch.float32)
        dy = randn((S, Cout, tokens), 2, 0.0, 1.0, torch.float32)
        w = randn((Cout, Cin), 3, 0.0, 0.05, torch.float32)

        def step():  # as the fused block calls them: with fp16 terms one pass per tensor finds its scale
            x_amax = CB.amax(x) if terms & CB.F16 else None
            CB.pw_gemm(CB.split_weight(w, False, terms), terms, Cout, Cin, x, terms, False, x_amax)
            dy_amax = CB.amax(dy) if terms & CB.F16 else None
            CB.pw_gemm(CB.split_weight(w, True, terms), terms, Cin, Cout, dy, terms, False, dy_amax)
            CB.pw_grad_weight(dy, terms, x, terms, dy_amax, x_amax)

        elapsed = _time_steps(torch, L, step, args.steps, args.warmup)
        g_ms, d_ms = _kernel_ms(L, L.KC_PW_GEMM), _kernel_ms(L, L.KC_PW_GRAD_WEIGHT)
        sustained = measure_mfma_ceiling(torch, L, True)
        flop = 2.0 * S * Cin * Cout * tokens                      # of one GEMM, counted once per fp32 product
        products = {3: 6, 2: 3, 1: 1, CB.F16 | 2: 3}[terms]      # 16-bit matrix-core products per fp32 product
        split = "2 fp16 terms per scaled operand" if terms & CB.F16 else f"{terms} bf16 terms per operand"
        _emit(args, "fp32-equivalent TFLOP/s of the kernel-size-1 convolution GEMMs, qkv of configs[4], 1 MI355X", "TFLOP/s",
              3 * flop / (elapsed / args.steps) / 1e12, elapsed, "f16" if terms & CB.F16 else "bf16",
              {"workload": f"Y = W X, dX = W^T dY, dW = dY X^T for W [1152, 384], X [256, 384, 196] fp32, {split}"},
              {"bound": "mfma", "achieved": products * flop / (g_ms * 1e-3) / 1e12, "peak": 2500.0, "unit": "TFLOP/s",
               "frac": products * flop / (g_ms * 1e-3) / 1e12 / 2500.0, "traffic": None, "kernel": "pw_gemm",
               "kernel_ms": g_ms, "grad_weight_ms": d_ms,
               "grad_weight_TFLOPs": products * flop / (d_ms * 1e-3) / 1e12,
               "fp32_equivalent_TFLOPs": flop / (g_ms * 1e-3) / 1e12,
               "mfma_sustained_random_operands_TFLOPs": sustained,
               "frac_of_sustained": products * flop / (g_ms * 1e-3) / 1e12 / sustained})
        return 0

    if args.workload == "config5":
        T, B, D, H, tokens = 4, 64, args.dim, 12, 196
        configure.hip_fuse_ssa_lif = bool(args.fuse_ssa_lif)
        configure.hip_conv_split, configure.hip_conv_terms = args.conv_split, args.terms
        configure.hip_conv_overlap_gradients = bool(args.overlap)
        torch.manual_seed(1005)
        block = layer.SpikingSelfAttention(D, H, backend="hip").to(dev)
        x = randn((T, B, D, tokens), 1105, 0.0, 1.0, torch.float32).requires_grad_()
        g = randn((T, B, D, tokens), 1205, 0.0, 1.0, torch.float32)

        def step():
            y = block(x)
            y.backward(g)
            x.grad = None
            block.zero_grad(set_to_none=True)
            functional.reset_net(block)

        elapsed = _time_steps(torch, L, step, args.steps, args.warmup)
        sf, sb = _kernel_ms(L, L.KC_SSA_FORWARD), _kernel_ms(L, L.KC_SSA_BACKWARD)
        # The convolution GEMMs are the largest share of the step and the part that the matrix cores bound: 16-bit
        # products per step (three per pair of real operands, two when one operand is spikes; bf16 terms: six and
        # three) over the time of all their launches.  qkv: Y = W X (real), dX (real), dW (real x real);
        # projection: Y (spikes), dX (real), dW (real x spikes).
        S_ = T * B
        flop_qkv, flop_proj = 2.0 * S_ * D * 3 * D * tokens, 2.0 * S_ * D * D * tokens
        real, spk = (3, 2) if args.conv_split == "f16" else ({3: 6, 2: 3, 1: 1}[args.terms], {3: 3, 2: 2, 1: 1}[args.terms])
        gemm_products = flop_qkv * 3 * real + flop_proj * (2 * spk + real)
        n_g, ms_g = L.profile_read(L.KC_PW_GEMM)
        n_d, ms_d = L.profile_read(L.KC_PW_GRAD_WEIGHT)
        gemm_ms_per_step = (ms_g + ms_d) / args.steps
        gemm_tflops = gemm_products / (gemm_ms_per_step * 1e-3) / 1e12 if gemm_ms_per_step else 0.0
        sustained = measure_mfma_ceiling(torch, L, True)
        cph = D // H
        probs = T * B * H
        n = T * B * D * tokens
        product = probs * 2 * cph * cph * tokens  # flops of one [cph, L] x [L, cph] (or [cph, cph] x [cph, L]) product
        # the qkv spikes travel bit-packed between the LIF and the contraction: 3 n / 8 bytes; fp32 elsewhere
        bytes_f = 3 * n // 8 + 4 * n              # bits read, out written
        bytes_b = 3 * n // 8 + 4 * n + 12 * n     # bits and grad_out read, dq / dk / dv written
        _emit(args, f"tokens/sec spiking self-attention block fwd+bwd, T=4 B=64 N=196 D={D} 12 heads, 1 MI355X",
              "tokens/s", T * B * tokens / (elapsed / args.steps), elapsed, args.conv_split,
              {"workload": f"configs[4]: SpikingSelfAttention({D}, 12, backend='hip'), x [4,64,{D},196] fp32 ~N(0,1), "
                           f"channels per head = {cph} (dim // heads, as the reference computes it); convolution GEMMs on "
                           f"{'two fp16' if args.conv_split == 'f16' else str(args.terms) + ' bf16'} terms per fp32 operand"},
              {"bound": "mfma", "achieved": gemm_tflops, "peak": 2500.0, "unit": "TFLOP/s", "frac": gemm_tflops / 2500.0,
               "traffic": None, "kernel": "pw_gemm + pw_dw (the six convolution GEMM launches of a step)",
               "kernel_ms": gemm_ms_per_step / max((n_g + n_d) / args.steps, 1), "gemm_ms_per_step": gemm_ms_per_step,
               "gemm_launches_per_step": (n_g + n_d) / args.steps, "gemm_16bit_product_flops_per_step": gemm_products,
               "mfma_sustained_random_operands_TFLOPs": sustained, "frac_of_sustained": gemm_tflops / sustained,
               "ssa_backward_ms": sb, "ssa_backward_GBs": bytes_b / (sb * 1e-3) / 1e9,
               "ssa_backward_frac_of_hbm": bytes_b / (sb * 1e-3) / 1e9 / HBM_PEAK_GBS, "ssa_backward_bytes": bytes_b,
               "ssa_backward_TFLOPs": 4 * product / (sb * 1e-3) / 1e12,
               "ssa_forward_ms": sf, "ssa_forward_GBs": bytes_f / (sf * 1e-3) / 1e9,
               "ssa_forward_TFLOPs": 2 * product / (sf * 1e-3) / 1e12,
               "lif_forward_ms": _kernel_ms(L, L.KC_FORWARD), "lif_backward_ms": _kernel_ms(L, L.KC_BACKWARD)})
        return 0
    raise SystemExit(f"unknown workload {args.workload}")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-sample-neurons", type=int, default=1 << 23)
    ap.add_argument("--cpu-repeats", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="default workload: skip the condensed measurements of BASELINE configs 3-5 after the headline")
    ap.add_argument("--terms", type=int, default=3, choices=[1, 2, 3],
                    help="pwconv and config5 workloads with --conv-split bf16: bf16 terms per fp32 operand")
    ap.add_argument("--overlap", action="store_true",
                    help="config5 workload: run the weight gradient of a convolution on a second stream beside its input gradient "
                         "(configure.hip_conv_overlap_gradients)")
    ap.add_argument("--conv-split", default="f16", choices=["f16", "bf16"],
                    help="pwconv and config5 workloads: how fp32 operands of the convolution GEMMs are split for the matrix cores")
    ap.add_argument("--dim", type=int, default=384, choices=[384, 768],
                    help="config5 workload: embedding width (12 heads of dim // 12 channels: 32, or 64 with 768)")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="launch tuning of the library for this run (sjhip_set_tuning), e.g. --tune column_spread=1 "
                         "--tune fwd_block=256; may be given several times")
    ap.add_argument("--fuse-ssa-lif", action="store_true",
                    help="config5 workload: run the contraction and the attention's LIF as one kernel (configure.hip_fuse_ssa_lif)")
    ap.add_argument("--seq-len", type=int, default=SHAPE[0],
                    help="config2 variant: T steps over 2^29 / T neurons (the headline is T=16); a secondary measurement")
    ap.add_argument("--n-offset", type=int, default=0,
                    help="config2 variant: K more neurons than the power of two, i.e. another row stride (multiple of 4)")
    ap.add_argument("--workload", default="config2", choices=["config2", "config3", "config4", "config5", "pwconv", "ceilings", "qif", "eif", "izhikevich", "ilif", "stbif", "aaif", "fp8"],
                    help="config2 (default) is the headline metric; the others are secondary measurements")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path shards over neurons with no exchange, and this build runs "
              "on single-GPU boxes only; run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    from spikingjelly_amd.activation_based import functional, neuron, surrogate
    from spikingjelly_amd.activation_based.hip_kernel import library as L

    L.load()
    for item in args.tune:
        key, _, value = item.partition("=")
        L.set_tuning(key.strip(), int(value))
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm device", file=sys.stderr)
        return 2
    if args.workload != "config2":
        return other_workload(args)
    dev = torch.device("cuda:0")
    N = 1
    for d in SHAPE[1:]:
        N *= d
    T, shape = args.seq_len, SHAPE
    variant = args.seq_len != SHAPE[0] or args.n_offset != 0
    if variant:
        if args.seq_len < 1 or (SHAPE[0] * N) % args.seq_len or args.n_offset % 4 or args.n_offset < 0:
            raise SystemExit("--seq-len must divide 2^29 and --n-offset must be a non-negative multiple of 4")
        N = SHAPE[0] * N // args.seq_len + args.n_offset
        shape = (T, N)

    # inputs: CPU generator with the configured seeds, then resident on the device
    def make(seed, mean, std):
        g = torch.Generator().manual_seed(seed)
        return (torch.randn(shape, generator=g) * std + mean).to(dev)

    x = make(1002, 0.3, 0.8).requires_grad_()
    grad_spike = make(1102, 0.0, 1.0)
    grad_v = make(1202, 0.0, 0.1)

    node = neuron.LIFNode(tau=2.0, v_threshold=1.0, v_reset=0.0, surrogate_function=surrogate.ATan(2.0),
                          step_mode="m", backend="hip", store_v_seq=True).to(dev)

    def step():
        spikes = node(x)
        torch.autograd.backward([spikes, node.v_seq], [grad_spike, grad_v])
        x.grad = None
        functional.reset_net(node)
        return spikes

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    L.profile_reset()
    L.profile_enable(True)
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    with _quiet_collector():
        t0 = time.perf_counter()
        for i in range(args.steps):
            marks[i].record()  # on the stream the kernels are launched on
            spikes = step()
        marks[-1].record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    L.profile_enable(False)
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))
    quantile = lambda q: per_step[min(len(per_step) - 1, int(q * len(per_step)))]
    rate = float(spikes.detach().mean())
    n_fwd, ms_fwd = L.profile_read(L.KC_FORWARD)
    n_bwd, ms_bwd = L.profile_read(L.KC_BACKWARD)

    # measured ceilings on the same box: the library's plain streaming kernel over streams of the size of x (2.1 GB)
    del spikes
    node.v_seq = None
    torch.cuda.empty_cache()
    ceilings = measure_ceilings(torch, L, x.numel())

    ms_per_step = elapsed / args.steps * 1e3
    value = T * N / (elapsed / args.steps)

    # algorithmic bytes per launch: each tensor of the operator contract touched once
    fwd_bytes = 16 * T * N + 4 * N  # x, spike, v_seq, h_seq per step + v_init
    bwd_bytes = 16 * T * N + 4 * N  # grad_spike, grad_v, h_seq, grad_x per step + grad_v_init
    fwd_ms = ms_fwd / max(n_fwd, 1)
    bwd_ms = ms_bwd / max(n_bwd, 1)
    dominant = "forward" if fwd_ms >= bwd_ms else "backward"
    dom_ms, dom_bytes = (fwd_ms, fwd_bytes) if dominant == "forward" else (bwd_ms, bwd_bytes)
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    # HBM bytes the kernels actually move, each tensor touched once: the forward writes no h_seq (the backward replays
    # it) and the module's initial state is one broadcast element, so forward = x in, spikes + v_seq + v_last out;
    # backward = x, grad_spike, grad_v in, grad_x out.  The counter-measured figures (rocprofv3 FETCH_SIZE / WRITE_SIZE,
    # profiles/) are reported while they still describe the kernels that ran.
    fwd_moved = 12 * T * N + 4 * N
    bwd_moved = 16 * T * N
    rec = None if variant else recorded_traffic()
    traffic = rec.get(dominant) if rec else None
    if rec:
        fwd_moved, bwd_moved = rec["forward"], rec["backward"]

    out = {
        "metric": "neuron-steps/sec LIF fwd+bwd T=16 N=33.5M, 1 MI355X; % of HBM roofline" if not variant else
                  f"neuron-steps/sec LIF fwd+bwd T={T} N={N}, 1 MI355X; % of HBM roofline",
        "value": value,
        "unit": "neuron-steps/s",
        "n_gpus": 1,
        "step_ms_quantiles": {"p25": quantile(0.25), "median": quantile(0.5), "p75": quantile(0.75)},
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": ("configs[1]: LIFNode multi-step fwd+bwd, x [16,256,128,32,32]" if not variant else
                                f"variant of configs[1] with another shape: LIFNode multi-step fwd+bwd, x [{T},{N}]") +
                               " fp32 ~N(0.3,0.8), tau=2, hard reset 0, ATan(2), store_v_seq=True, grad_spike ~N(0,1), "
                               "grad_v ~N(0,0.1)",
                   "T": T, "N": N, "backend": "hip", "firing_rate": rate},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "kernel": dominant,
                     "kernel_ms": dom_ms, "algorithmic_bytes": dom_bytes,
                     "forward_ms": fwd_ms, "backward_ms": bwd_ms,
                     "forward_traffic_GBs": fwd_moved / (fwd_ms * 1e-3) / 1e9 if fwd_ms else None,
                     "backward_traffic_GBs": bwd_moved / (bwd_ms * 1e-3) / 1e9 if bwd_ms else None,
                     "step_traffic_frac": (fwd_moved + bwd_moved) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic_source": "rocprofv3 counters (profiles/)" if rec else "tensor sizes",
                     "ceilings_GBs": {k: round(v, 1) for k, v in ceilings.items()}},
    }
    del x, grad_spike, grad_v
    torch.cuda.empty_cache()
    if not variant and not args.no_secondary:
        out["secondary"] = secondary_measurements(args)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, args.cpu_sample_neurons, args.cpu_repeats)
        # the same port on one thread (a quarter of the sample: about as long as the run above)
        out["cpu_baseline_1thread"] = cpu_baseline(torch, max(args.cpu_sample_neurons // 4, 1 << 16), 2, threads=1)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
