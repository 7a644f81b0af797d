"""``sjhip_neuron_forward_pieces`` / ``sjhip_neuron_backward_recompute_pieces`` through the C ABI.

The forward over pieces must equal ``sjhip_neuron_forward`` over the whole sequence bit for bit (spikes, states) and
its checkpoints must be the states ``v_seq`` holds at the piece boundaries.  The backward over pieces keeps the gradient
of a piece's initial state in fp32 registers for the piece before it.  In fp32 storage it must equal, bit for bit,
``sjhip_neuron_backward_recompute`` called once per piece from the last to the first with ``grad_v_init`` handed on as
``grad_v_last`` (piece lengths above the short-sequence variant's, so both run the same device code); in 16-bit storage
that hand-over through memory rounds, so there the reference is ``sjhip_neuron_backward`` over the whole sequence on a
saved ``h_seq`` (the same fp32 carry throughout), within one rounding of the storage dtype.  PLIF's dL/dk is a sum in
another order.  fp32 is also checked against the oracle.
"""

import ctypes

import numpy as np

import pytest
import torch

from oracle import neuron_oracle as no

from helpers import bits_equal, seeded_randn

pytestmark = pytest.mark.gpu

ERR_INVALID, ERR_UNSUPPORTED = -1, -2  # SJHIP_ERR_INVALID, SJHIP_ERR_UNSUPPORTED


@pytest.fixture(scope="module")
def L():
    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    from spikingjelly_amd.activation_based.hip_kernel import library

    library.load()
    return library


def _case(L, neuron, dtype, T, N, flags, seed):
    dev = torch.device("cuda:0")
    c = dict(neuron=neuron, dtype=dtype, T=T, N=N)
    c["x"] = seeded_randn((T, N), seed, 0.3, 1.0).to(dtype).to(dev)
    c["v0"] = (seeded_randn((N,), seed + 1) * 0.2).to(dtype).to(dev)
    c["gs"] = seeded_randn((T, N), seed + 2).to(dtype).to(dev)
    c["gv"] = (seeded_randn((T, N), seed + 3) * 0.1).to(dtype).to(dev)
    c["gl"] = (seeded_randn((N,), seed + 4) * 0.1).to(dtype).to(dev)
    c["k"] = 0.375 if neuron == L.NEURON_PLIF else 0.5
    c["kd"] = torch.tensor([c["k"]], dtype=torch.float32, device=dev)
    c["p"] = L.NeuronParams(c["k"] if neuron == L.NEURON_PLIF else 2.0, 1.0, 0.0, 2.0, 1, flags)
    c["stream"] = L.current_stream_ptr(dev)
    return c


def _kd(L, c):
    return c["kd"].data_ptr() if c["neuron"] == L.NEURON_PLIF else None


def _forward_whole(L, c):
    s, v, vl = torch.empty_like(c["x"]), torch.empty_like(c["x"]), torch.empty_like(c["v0"])
    L.check(L.load().sjhip_neuron_forward(c["neuron"], L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), c["T"], c["N"],
                                          c["x"].data_ptr(), c["v0"].data_ptr(), _kd(L, c), s.data_ptr(), v.data_ptr(),
                                          vl.data_ptr(), None, c["stream"]), "forward")
    return s, v, vl


def _forward_pieces(L, c, chunk, with_v_seq=True):
    lib = L.load()
    pieces = lib.sjhip_replay_pieces(c["T"], chunk)
    s, vl = torch.empty_like(c["x"]), torch.full_like(c["v0"], float("nan"))
    v = torch.empty_like(c["x"]) if with_v_seq else None
    # a state kept in fp32 beside 16-bit storage is checkpointed in fp32
    ck_dtype = torch.float32 if c["p"].flags & L.FLAG_FP32_STATE else c["dtype"]
    ck = torch.full((max(pieces - 1, 1), c["N"]), float("nan"), dtype=ck_dtype, device=c["x"].device)
    L.check(lib.sjhip_neuron_forward_pieces(c["neuron"], L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), c["T"], c["N"], chunk,
                                            c["x"].data_ptr(), c["v0"].data_ptr(), _kd(L, c), s.data_ptr(),
                                            v.data_ptr() if with_v_seq else None, vl.data_ptr(), ck.data_ptr(),
                                            c["stream"]), "forward_pieces")
    return s, v, vl, ck[: pieces - 1]


def _plif_buffers(L, c):
    if c["neuron"] != L.NEURON_PLIF:
        return None, None
    ws = torch.empty(L.load().sjhip_plif_workspace_floats(L.dtype_id(c["dtype"]), c["N"]), dtype=torch.float32, device="cuda:0")
    return torch.full((1,), float("nan"), dtype=torch.float32, device="cuda:0"), ws


def _backward_pieces(L, c, chunk, ck, with_gv):
    gx, gv0 = torch.full_like(c["x"], float("nan")), torch.full_like(c["v0"], float("nan"))
    gk, ws = _plif_buffers(L, c)
    L.check(L.load().sjhip_neuron_backward_recompute_pieces(
        c["neuron"], L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), c["T"], c["N"], chunk, c["x"].data_ptr(), c["v0"].data_ptr(),
        _kd(L, c), ck.data_ptr() if ck.numel() else None, c["gs"].data_ptr(), c["gv"].data_ptr() if with_gv else None,
        c["gl"].data_ptr(), gx.data_ptr(), gv0.data_ptr(), L.ptr(gk), L.ptr(ws), c["stream"]),
        "backward_recompute_pieces")
    return gx, gv0, gk


def _backward_whole_saved_h(L, c, with_gv):
    """sjhip_neuron_forward saving h_seq, then sjhip_neuron_backward over the whole sequence."""
    lib = L.load()
    s, v, h = torch.empty_like(c["x"]), torch.empty_like(c["x"]), torch.empty_like(c["x"])
    L.check(lib.sjhip_neuron_forward(c["neuron"], L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), c["T"], c["N"], c["x"].data_ptr(),
                                     c["v0"].data_ptr(), _kd(L, c), s.data_ptr(), v.data_ptr(), None, h.data_ptr(), c["stream"]),
            "forward")
    gx, gv0 = torch.full_like(c["x"], float("nan")), torch.full_like(c["v0"], float("nan"))
    gk, ws = _plif_buffers(L, c)
    L.check(lib.sjhip_neuron_backward(c["neuron"], L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), c["T"], c["N"], c["gs"].data_ptr(),
                                      c["gv"].data_ptr() if with_gv else None, c["gl"].data_ptr(), h.data_ptr(), c["v0"].data_ptr(),
                                      _kd(L, c), gx.data_ptr(), gv0.data_ptr(), L.ptr(gk), L.ptr(ws), c["stream"]), "backward")
    return gx, gv0, (float(gk.item()) if gk is not None else 0.0)


def _backward_piece_by_piece(L, c, chunk, ck, with_gv):
    """One sjhip_neuron_backward_recompute call per piece, last to first."""
    lib = L.load()
    T, N = c["T"], c["N"]
    row = N * c["x"].element_size()
    gx, gv0 = torch.full_like(c["x"], float("nan")), torch.full_like(c["v0"], float("nan"))
    carries = [torch.empty_like(c["v0"]), torch.empty_like(c["v0"])]
    starts = list(range(0, T, chunk))
    gk_total = 0.0
    for j in range(len(starts) - 1, -1, -1):
        t0 = starts[j]
        length = min(chunk, T - t0)
        gk, ws = _plif_buffers(L, c)
        state = c["v0"] if j == 0 else ck[j - 1]
        g_last = c["gl"] if j == len(starts) - 1 else carries[(j + 1) & 1]
        g_init = gv0 if j == 0 else carries[j & 1]
        L.check(lib.sjhip_neuron_backward_recompute(
            c["neuron"], L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), length, N, c["x"].data_ptr() + t0 * row, state.data_ptr(),
            _kd(L, c), c["gs"].data_ptr() + t0 * row, c["gv"].data_ptr() + t0 * row if with_gv else None, g_last.data_ptr(),
            gx.data_ptr() + t0 * row, g_init.data_ptr(), L.ptr(gk), L.ptr(ws), c["stream"]), "backward_recompute")
        if gk is not None:
            gk_total += float(gk.item())
    return gx, gv0, gk_total


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=lambda v: str(v).replace("torch.", ""))
@pytest.mark.parametrize("neuron_name", ["IF", "LIF", "PLIF", "QIF"])
# (pieces of 18 and 40 steps need more than 64 KiB of dynamic LDS per block at 256 and 128 work-items)
@pytest.mark.parametrize("T,chunk", [(44, 16), (64, 16), (30, 10), (12, 16), (40, 18), (90, 40)])
def test_pieces_equal_whole_forward_and_piecewise_backward(L, dtype, neuron_name, T, chunk):
    neuron = getattr(L, "NEURON_" + neuron_name)
    flags = L.FLAG_DECAY_INPUT
    N = 8 * 300
    c = _case(L, neuron, dtype, T, N, flags, 100 + T)
    if neuron == L.NEURON_QIF:
        c["p"] = L.NeuronParams(2.0, 1.0, 0.0, 2.0, 1, flags, 0.0, 0.8, 1.0)  # v_rest, v_c, a0 as the Python wrapper lays them out
    s, v, vl = _forward_whole(L, c)
    sp, vp, vlp, ck = _forward_pieces(L, c, chunk)
    torch.cuda.synchronize()
    assert bits_equal(sp, s) and bits_equal(vp, v) and bits_equal(vlp, vl)
    for j in range(ck.shape[0]):
        assert bits_equal(ck[j], v[(j + 1) * chunk - 1]), f"checkpoint {j}"
    s2, _, vl2, ck2 = _forward_pieces(L, c, chunk, with_v_seq=False)
    torch.cuda.synchronize()
    assert bits_equal(s2, s) and bits_equal(vl2, vl) and bits_equal(ck2, ck)
    for with_gv in (True, False):
        got = _backward_pieces(L, c, chunk, ck, with_gv)
        if dtype == torch.float32:
            ref = _backward_piece_by_piece(L, c, chunk, ck, with_gv)
            torch.cuda.synchronize()
            assert bits_equal(got[0], ref[0]), "grad_x_seq"
            assert bits_equal(got[1], ref[1]), "grad_v_init"
        else:
            ref = _backward_whole_saved_h(L, c, with_gv)
            torch.cuda.synchronize()
            ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7  # one rounding of the storage dtype
            torch.testing.assert_close(got[0].float(), ref[0].float(), rtol=ulp, atol=1e-4)
            torch.testing.assert_close(got[1].float(), ref[1].float(), rtol=ulp, atol=1e-4)
        if neuron == L.NEURON_PLIF:
            assert float(got[2].item()) == pytest.approx(ref[2], rel=1e-3 if dtype != torch.float32 else 1e-5, abs=1e-3)


def _backward_whole_replay(L, c, with_gv):
    """sjhip_neuron_backward_recompute over the whole sequence (it holds every step's h on chip, so T is bounded)."""
    gx, gv0 = torch.full_like(c["x"], float("nan")), torch.full_like(c["v0"], float("nan"))
    gk, ws = _plif_buffers(L, c)
    L.check(L.load().sjhip_neuron_backward_recompute(
        c["neuron"], L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), c["T"], c["N"], c["x"].data_ptr(), c["v0"].data_ptr(), _kd(L, c),
        c["gs"].data_ptr(), c["gv"].data_ptr() if with_gv else None, c["gl"].data_ptr(), gx.data_ptr(), gv0.data_ptr(),
        L.ptr(gk), L.ptr(ws), c["stream"]), "backward_recompute")
    return gx, gv0, (float(gk.item()) if gk is not None else 0.0)


def _fp32_state_oracle(c, kind, with_gv):
    """float64 backward over the unrounded fp32 h of the mixed-precision forward (what a replay sees)."""
    from oracle import bptt_oracle

    k = {"if": 0.0, "lif": 0.5, "plif": c["k"]}[kind]
    x, v0 = c["x"].cpu(), c["v0"].cpu()
    _, _, _, raw_h = no.multi_step_mixed_precision(kind, x.float(), v0.float(), c["dtype"], k, True, 1.0, 0.0, return_raw_h=True)
    h64 = raw_h.double().numpy()
    s64 = (h64 >= 1.0).astype(np.float64)
    v64 = (1 - s64) * h64
    v_prev = np.concatenate([v0.double().numpy()[None], v64[:-1]])
    x_implied = (h64 - v_prev) / k + v_prev if k else None
    sgp = lambda z: no.surrogate_grad("atan", torch.from_numpy(np.ascontiguousarray(z)), 2.0).numpy()
    return bptt_oracle.bptt(kind, h64, s64, sgp, c["gs"].cpu().double().numpy(),
                            c["gv"].cpu().double().numpy() if with_gv else None, c["gl"].cpu().double().numpy(), k, True, 1.0,
                            0.0, False, v_prev, x_implied)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=lambda v: str(v).replace("torch.", ""))
@pytest.mark.parametrize("neuron_name", ["IF", "LIF", "PLIF"])
@pytest.mark.parametrize("T,chunk,other", [(44, 16, 22), (64, 16, 32), (30, 10, 0)])
def test_pieces_with_16_bit_storage_and_fp32_state(L, dtype, neuron_name, T, chunk, other):
    """16-bit storage with the state kept in fp32 (``SJHIP_FLAG_FP32_STATE``): the checkpoints are fp32 rows, so the
    pieces reproduce the whole forward bit for bit (a checkpoint in the storage dtype would round the state).  The
    backward replays the unrounded h, as the whole-sequence replay does (the route over a saved ``h_seq`` sees h
    rounded, and decides a few spikes differently): it equals that replay bit for bit where the sequence fits one,
    equals itself at another piece length, and agrees with the float64 recurrence over the unrounded h."""
    neuron = getattr(L, "NEURON_" + neuron_name)
    flags = L.FLAG_DECAY_INPUT | L.FLAG_FP32_STATE
    c = _case(L, neuron, dtype, T, 8 * 300, flags, 300 + T)
    s, v, vl = _forward_whole(L, c)
    sp, vp, vlp, ck = _forward_pieces(L, c, chunk)
    torch.cuda.synchronize()
    assert ck.dtype == torch.float32 and not torch.isnan(ck).any()
    assert bits_equal(sp, s) and bits_equal(vp, v) and bits_equal(vlp, vl)
    for j in range(ck.shape[0]):  # the stored v_seq row is the checkpoint rounded once
        assert bits_equal(ck[j].to(dtype), v[(j + 1) * chunk - 1]), f"checkpoint {j}"
    assert float((ck != ck.to(dtype).float()).float().mean()) > 0.2  # and the checkpoint really holds more bits
    for with_gv in (True, False):
        got = _backward_pieces(L, c, chunk, ck, with_gv)
        if other:
            ck2 = _forward_pieces(L, c, other)[3]
            ref = _backward_pieces(L, c, other, ck2, with_gv)
            ref = (ref[0], ref[1], float(ref[2].item()) if ref[2] is not None else 0.0)
        else:
            ref = _backward_whole_replay(L, c, with_gv)
        torch.cuda.synchronize()
        assert not torch.isnan(got[0].float()).any() and not torch.isnan(got[1].float()).any()
        assert bits_equal(got[0], ref[0]), "grad_x_seq"
        assert bits_equal(got[1], ref[1]), "grad_v_init"
        egx, egv0, egk = _fp32_state_oracle(c, neuron_name.lower(), with_gv)
        torch.testing.assert_close(got[0].cpu().double(), torch.from_numpy(egx), rtol=1e-2, atol=1e-3)
        torch.testing.assert_close(got[1].cpu().double(), torch.from_numpy(egv0), rtol=1e-2, atol=1e-3)
        if neuron == L.NEURON_PLIF:
            assert float(got[2].item()) == pytest.approx(ref[2], rel=1e-4, abs=1e-3)
            assert float(got[2].item()) == pytest.approx(egk, rel=1e-3, abs=1e-2)


@pytest.mark.parametrize("neuron_name,kind", [("IF", "if"), ("LIF", "lif")])
def test_pieces_against_the_oracle(L, neuron_name, kind):
    T, N, chunk = 50, 4 * 257, 16
    c = _case(L, getattr(L, "NEURON_" + neuron_name), torch.float32, T, N, L.FLAG_DECAY_INPUT, 7)
    s, v, vl, ck = _forward_pieces(L, c, chunk)
    gx, gv0, _ = _backward_pieces(L, c, chunk, ck, True)
    torch.cuda.synchronize()
    x, v0, gs, gv, gl = (c[n].cpu() for n in ("x", "v0", "gs", "gv", "gl"))
    want = no.forward_backward(kind, x, v0, gs, gv, gl, 2.0, True, 1.0, 0.0, "atan", 2.0, False)
    assert torch.equal(want["spike_seq"], s.cpu()) and torch.equal(want["v_seq"], v.cpu())
    torch.testing.assert_close(gx.cpu(), want["grad_x"], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(gv0.cpu(), want["grad_v_init"], rtol=1e-5, atol=1e-6)


def test_pieces_argument_checks(L):
    lib = L.load()
    c = _case(L, L.NEURON_LIF, torch.float32, 40, 64, L.FLAG_DECAY_INPUT, 3)
    s, vl = torch.empty_like(c["x"]), torch.empty_like(c["v0"])
    head = (L.NEURON_LIF, L.dtype_id(torch.float32), ctypes.byref(c["p"]), 40, 64)
    # several pieces without a checkpoint buffer
    assert lib.sjhip_neuron_forward_pieces(*head, 16, c["x"].data_ptr(), c["v0"].data_ptr(), None, s.data_ptr(), None,
                                           vl.data_ptr(), None, c["stream"]) == ERR_INVALID
    assert lib.sjhip_neuron_forward_pieces(*head, 0, c["x"].data_ptr(), c["v0"].data_ptr(), None, s.data_ptr(), None,
                                           vl.data_ptr(), None, c["stream"]) == ERR_INVALID
    # a piece too long for LDS
    ck = torch.empty((1, 64), device="cuda:0")
    gx = torch.empty_like(c["x"])
    assert lib.sjhip_neuron_backward_recompute_pieces(*head[:3], 400, 64, 200, c["x"].data_ptr(), c["v0"].data_ptr(), None,
                                                      ck.data_ptr(), c["gs"].data_ptr(), None, None, gx.data_ptr(), None, None,
                                                      None, c["stream"]) == ERR_UNSUPPORTED
    assert lib.sjhip_replay_pieces(40, 16) == 3 and lib.sjhip_replay_pieces(16, 16) == 1 and lib.sjhip_replay_pieces(0, 16) == 0


@pytest.mark.parametrize("N", [8 * 300, 128 * 4 * 8 * 37 + 4, 1 << 20, 1024 * 2049, 262144 * 9])
def test_block_to_column_order_does_not_change_results(L, N):
    """``column_spread`` only permutes which block works on which columns: forward, saved-h backward, replaying backward
    and the pieces kernels must give the same bits whichever order runs (grids of fewer than eight blocks, a grid that
    is not a multiple of eight, a large one; the last two row lengths are strides at which the automatic mode deals
    runs of 256 blocks to the XCDs, with 256 and with 128 work-items per block, over more than 2048 blocks and a
    remainder)."""
    lib = L.load()
    c = _case(L, L.NEURON_PLIF, torch.float32, 24, N, L.FLAG_DECAY_INPUT, 11)
    results = []
    try:
        for mode in (0, 1, 2, 4, 64):
            assert lib.sjhip_set_tuning(b"column_spread", mode) == 0
            s, v, vl = _forward_whole(L, c)
            sp, vp, vlp, ck = _forward_pieces(L, c, 16)
            gx, gv0, gk = _backward_pieces(L, c, 16, ck, True)
            gx1, gv1 = torch.full_like(c["x"], float("nan")), torch.full_like(c["v0"], float("nan"))
            gk1, ws = _plif_buffers(L, c)
            L.check(lib.sjhip_neuron_backward_recompute(
                c["neuron"], L.dtype_id(c["dtype"]), ctypes.byref(c["p"]), c["T"], N, c["x"].data_ptr(), c["v0"].data_ptr(),
                c["kd"].data_ptr(), c["gs"].data_ptr(), c["gv"].data_ptr(), c["gl"].data_ptr(), gx1.data_ptr(), gv1.data_ptr(),
                gk1.data_ptr(), ws.data_ptr(), c["stream"]), "backward_recompute")
            torch.cuda.synchronize()
            assert bits_equal(sp, s) and bits_equal(vp, v)
            results.append((s, v, vl, gx, gv0, gx1, gv1, gk1))
    finally:
        lib.sjhip_set_tuning(b"column_spread", 2)
    for other in results[1:]:
        for a, b in zip(results[0][:7], other[:7]):
            assert bits_equal(a, b)
        assert float(results[0][7].item()) == pytest.approx(float(other[7].item()), rel=1e-5)
