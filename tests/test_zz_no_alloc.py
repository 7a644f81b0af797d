"""``sjhip_neuron_backward_static``: the PLIF backward whose partial sums live in the library's own device array.

Called through ctypes on the C ABI and compared with ``sjhip_neuron_backward`` (same kernels, caller's workspace):
``grad_x_seq``, ``grad_v_init`` and ``dL/dk`` bit for bit (the reduction order is fixed), and ``dL/dk`` against the
oracle's autograd (fp32 gradients rtol 1e-5; the sum of millions of terms against float64, rel 1e-4).  Two calls in a row on one stream, the second
with a smaller input, so partial sums left behind by the first call would show up in the second.
"""

import ctypes

import pytest
import torch

from oracle import neuron_oracle as no

from helpers import bits_equal, seeded_randn

pytestmark = pytest.mark.gpu

GRAD_RTOL = 1e-5


@pytest.fixture(scope="module")
def L():
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    from spikingjelly_amd.activation_based.hip_kernel import library

    library.load()
    return library


def _plif_case(L, T, N, seed, dtype=torch.float32):
    """Forward through the C ABI (h_seq saved); returns the device tensors the two backwards share."""
    lib = L.load()
    dev = torch.device("cuda:0")
    k = 0.375
    x = seeded_randn((T, N), seed, 0.2, 1.0).to(dtype).to(dev)
    v0 = (seeded_randn((N,), seed + 1) * 0.1).to(dtype).to(dev)
    gs = seeded_randn((T, N), seed + 2).to(dtype).to(dev)
    gv = (seeded_randn((T, N), seed + 3) * 0.1).to(dtype).to(dev)
    kd = torch.tensor([k], dtype=torch.float32, device=dev)
    p = L.NeuronParams(k, 1.0, 0.0, 4.0, 0, L.FLAG_DECAY_INPUT | L.FLAG_SOFT_RESET)
    s, v, h = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    stream = L.current_stream_ptr(dev)
    L.check(lib.sjhip_neuron_forward(L.NEURON_PLIF, L.dtype_id(dtype), ctypes.byref(p), T, N, x.data_ptr(), v0.data_ptr(),
                                     kd.data_ptr(), s.data_ptr(), v.data_ptr(), None, h.data_ptr(), stream), "forward")
    return dict(p=p, T=T, N=N, x=x, v0=v0, gs=gs, gv=gv, kd=kd, h=h, k=k, dtype=dtype, stream=stream)


def _backward(L, c, static):
    lib = L.load()
    gx = torch.full_like(c["x"], float("nan"))
    gv0 = torch.full_like(c["v0"], float("nan"))
    gk = torch.full((1,), float("nan"), dtype=torch.float32, device=c["x"].device)
    head = (L.NEURON_PLIF, L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), c["T"], c["N"], c["gs"].data_ptr(),
            c["gv"].data_ptr(), None, c["h"].data_ptr(), c["v0"].data_ptr(), c["kd"].data_ptr(), gx.data_ptr(),
            gv0.data_ptr(), gk.data_ptr())
    if static:
        L.check(lib.sjhip_neuron_backward_static(*head, c["stream"]), "backward_static")
    else:
        ws = torch.empty(lib.sjhip_plif_workspace_floats(L.dtype_id(c["dtype"]), c["N"]), dtype=torch.float32,
                         device=c["x"].device)
        L.check(lib.sjhip_neuron_backward(*head, ws.data_ptr(), c["stream"]), "backward")
    torch.cuda.synchronize()
    return gx.cpu(), gv0.cpu(), gk.cpu()


def _check(L, c):
    ref = _backward(L, c, static=False)
    got = _backward(L, c, static=True)
    for name, a, b in zip(("grad_x_seq", "grad_v_init", "grad_rtau"), got, ref):
        assert bits_equal(a, b), name
    if c["dtype"] == torch.float32:
        x, v0, gs, gv = (c[n].cpu() for n in ("x", "v0", "gs", "gv"))
        kt = torch.tensor(c["k"], dtype=torch.float32)
        want = no.forward_backward("plif_k", x, v0, gs, gv, None, kt, True, 1.0, None, "sigmoid", 4.0, False)
        assert torch.equal(want["h_seq"], c["h"].cpu())
        torch.testing.assert_close(got[0], want["grad_x"], rtol=GRAD_RTOL, atol=1e-6)
        torch.testing.assert_close(got[1], want["grad_v_init"], rtol=GRAD_RTOL, atol=1e-6)
        want64 = no.forward_backward("plif_k", x.double(), v0.double(), gs.double(), gv.double(), None, kt.double(), True,
                                     1.0, None, "sigmoid", 4.0, False)
        if torch.equal(want64["spike_seq"].float(), want["spike_seq"]):
            assert float(got[2]) == pytest.approx(float(want64["grad_p"]), rel=1e-4, abs=1e-3)


def test_static_workspace_backward_equals_the_callers_workspace_backward_twice_in_a_row(L):
    big = _plif_case(L, 8, 1 << 20, 4101)       # 2048 partial sums at 128 lanes x 4 neurons
    small = _plif_case(L, 5, 12 * 1024 + 4, 4201)  # fewer blocks, the last one partly filled
    _check(L, big)
    _check(L, small)
    _check(L, big)


def test_static_workspace_backward_odd_size_and_bf16(L):
    _check(L, _plif_case(L, 4, 1037, 4301))                      # element-wise kernel (N not a multiple of 4)
    _check(L, _plif_case(L, 8, 1 << 16, 4401, torch.bfloat16))


def test_static_workspace_backward_refuses_what_does_not_fit(L):
    lib = L.load()
    p = L.NeuronParams(0.5, 1.0, 0.0, 4.0, 0, L.FLAG_DECAY_INPUT)
    n = L.STATIC_WORKSPACE_MAX_NEURONS + 64
    rc = lib.sjhip_neuron_backward_static(L.NEURON_PLIF, L.DTYPE_F32, ctypes.byref(p), 2, n, 16, None, None, 16, 16, 16, 16,
                                          None, 16, None)
    assert rc == -4 and b"built-in workspace" in lib.sjhip_last_error()


def test_static_workspace_backward_passes_other_neurons_through(L):
    lib = L.load()
    dev = torch.device("cuda:0")
    T, N = 6, 4096
    h = seeded_randn((T, N), 4501, 0.5, 1.0).to(dev)
    gs = seeded_randn((T, N), 4502).to(dev)
    p = L.NeuronParams(2.0, 1.0, 0.0, 2.0, 1, L.FLAG_DECAY_INPUT)
    out = []
    for static in (False, True):
        gx, gv0 = torch.empty_like(h), torch.empty(N, device=dev)
        head = (L.NEURON_LIF, L.DTYPE_F32, ctypes.byref(p), T, N, gs.data_ptr(), None, None, h.data_ptr(), None, None,
                gx.data_ptr(), gv0.data_ptr(), None)
        if static:
            L.check(lib.sjhip_neuron_backward_static(*head, L.current_stream_ptr(dev)), "backward_static")
        else:
            L.check(lib.sjhip_neuron_backward(*head, None, L.current_stream_ptr(dev)), "backward")
        torch.cuda.synchronize()
        out.append((gx.cpu(), gv0.cpu()))
    assert bits_equal(out[0][0], out[1][0]) and bits_equal(out[0][1], out[1][1])


def test_a_call_on_another_stream_is_refused_while_the_array_is_in_use(L):
    """Calls on one GPU share its array.  A call on a second stream while the first call's kernels still run would mix
    two sets of partial sums: the library refuses it (SJHIP_ERR_INVALID) instead; after the first stream has finished,
    or on the first stream itself, the call goes through."""
    lib = L.load()
    c = _plif_case(L, 16, 1 << 24, 31)   # a backward of about a millisecond
    small = _plif_case(L, 4, 4 * 1024, 32)
    torch.cuda.synchronize()
    other = torch.cuda.Stream()

    def buffers(case):
        return (torch.empty_like(case["x"]), torch.empty_like(case["v0"]),
                torch.empty((1,), dtype=torch.float32, device=case["x"].device))

    def call(case, out, stream_ptr):
        gx, gv0, gk = out
        return lib.sjhip_neuron_backward_static(L.NEURON_PLIF, L.dtype_id(case["dtype"]), ctypes.byref(case["p"]), case["T"],
                                                case["N"], case["gs"].data_ptr(), case["gv"].data_ptr(), None, case["h"].data_ptr(),
                                                case["v0"].data_ptr(), case["kd"].data_ptr(), gx.data_ptr(), gv0.data_ptr(),
                                                gk.data_ptr(), stream_ptr)

    # every buffer exists before the first launch: nothing between the launches below waits for the device
    big_out, same_out, other_out, out = buffers(c), buffers(small), buffers(small), buffers(small)
    import gc

    main = torch.cuda.current_stream()
    for calls in (20, 80, 320):   # some fifteen milliseconds of work on the first stream, more if the host was held up
        torch.cuda.synchronize()
        gc.collect()
        gc.disable()   # (a full collection takes longer than the queued work)
        try:
            for _ in range(calls):
                assert call(c, big_out, c["stream"]) == 0
            rc_same = call(small, same_out, c["stream"])          # same stream: ordered behind the calls before
            rc_other = call(small, other_out, other.cuda_stream)  # another stream while the first one still works
            message = lib.sjhip_last_error()
            still_busy = not main.query()
        finally:
            gc.enable()
        torch.cuda.synchronize()
        assert rc_same == 0
        if still_busy:   # the premise held: the first stream was still working after the call on the other one returned
            break
    else:
        pytest.fail("the first stream finished 320 backward calls before the host could issue the next call")
    assert rc_other == -1 and b"another stream" in message
    assert call(small, out, other.cuda_stream) == 0       # everything has finished: the other stream may use the array
    torch.cuda.synchronize()
    ref = _backward(L, small, False)
    assert bits_equal(out[0].cpu(), ref[0]) and bits_equal(out[1].cpu(), ref[1]) and bits_equal(out[2].cpu(), ref[2])
