"""Vectors written by the reference's own torch backend (tests/golden/make_reference_golden.py ran its
``LIFNode`` / ``ParametricLIFNode`` / ``IFNode`` on the CPU once and stored inputs and outputs) against

* the oracle and this package's ``backend='torch'`` nodes (CPU tests): spikes and ``v_seq`` bit for bit, gradients
  bit for bit as well (the same torch ops in the same order on the same torch build; a tolerance of 1e-6 relative
  is written down in case another torch build associates a reduction differently);
* the HIP kernels (``-m gpu``): spikes and ``v_seq`` bit for bit, gradients within 1e-5 relative (fp32), 1e-2 (fp16).

These are the vectors that pin the op order of the charge on inputs that are not dyadic (``v + (x - (v - v_reset)) / tau``
and ``v - (v - v_reset) / tau + x`` with a non-zero ``v_reset``), which exact rational arithmetic cannot.
"""

import os

import numpy as np
import pytest
import torch

from oracle import neuron_oracle as no
from spikingjelly_amd.activation_based import neuron, surrogate

from helpers import GOLDEN_DIR, bits_equal

CASES = {
    # name: (class, constructor arguments, oracle kind, oracle tau / w source, surrogate name, alpha)
    "config1": (neuron.LIFNode, dict(tau=2.0), "lif", "atan", 2.0),
    "lif_a": (neuron.LIFNode, dict(tau=3.0, decay_input=False, v_reset=-0.2), "lif", "sigmoid", 4.0),
    "plif_a": (neuron.ParametricLIFNode, dict(init_tau=2.0, v_reset=None), "plif", "sigmoid", 4.0),
    "plif_b": (neuron.ParametricLIFNode, dict(init_tau=3.5, decay_input=False, v_reset=-0.2), "plif", "atan", 2.0),
    "if_a": (neuron.IFNode, dict(v_reset=None), "if", "sigmoid", 4.0),
    "lif_b": (neuron.LIFNode, dict(tau=5.0, v_threshold=0.8, v_reset=0.3, detach_reset=True), "lif", "atan", 2.0),
}
SG = {"atan": surrogate.ATan, "sigmoid": surrogate.Sigmoid}


def load(name):
    z = np.load(os.path.join(GOLDEN_DIR, f"reference_{name}.npz"))
    d = {k: z[k] for k in z.files}
    shape = tuple(int(i) for i in d["shape"])
    n = int(np.prod(shape))
    dtype = torch.from_numpy(d["x"]).dtype
    d["spike"] = torch.from_numpy(np.unpackbits(d["spike_bits"], bitorder="little")[:n].reshape(shape).astype(np.float32)).to(dtype)
    for k in ("x", "grad_spike", "v_seq", "grad_x", "grad_v_seq", "v_init", "w", "grad_w", "k"):
        if k in d:
            d[k] = torch.from_numpy(d[k])
    return d


def grad_tolerance(dtype):
    # fp16: the reference's autograd rounds every backward op to fp16 (its gradients of O(1) carry a few 1e-3 of
    # rounding noise of their own and flush to zero below 6e-8); the kernel computes in fp32 and rounds once
    return dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=5e-3)


def run_node(name, backend, device):
    cls, kw, _, sg, alpha = CASES[name]
    g = load(name)
    node = cls(surrogate_function=SG[sg](alpha), step_mode="m", backend=backend, store_v_seq=True, **kw).to(device)
    x = g["x"].to(device).requires_grad_(True)
    if "v_init" in g:
        node.v = g["v_init"].to(device)
    s = node(x)
    outs, grads = [s], [g["grad_spike"].to(device)]
    if "grad_v_seq" in g:
        outs.append(node.v_seq)
        grads.append(g["grad_v_seq"].to(device))
    torch.autograd.backward(outs, grads)
    return g, node, s.detach().cpu(), node.v_seq.detach().cpu(), x.grad.cpu()


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_the_reference_vectors(name):
    _, kw, kind, sg, alpha = CASES[name]
    g = load(name)
    x = g["x"].flatten(1)
    v0 = g["v_init"].flatten() if "v_init" in g else torch.full_like(x[0], kw.get("v_reset", 0.0) or 0.0)
    p = g["w"].reshape(()) if kind == "plif" else kw.get("tau")
    gv = g["grad_v_seq"].flatten(1) if "grad_v_seq" in g else None
    ref = no.forward_backward(kind, x, v0, g["grad_spike"].flatten(1), gv, None, p, kw.get("decay_input", True),
                              kw.get("v_threshold", 1.0), kw.get("v_reset", 0.0), sg, alpha, kw.get("detach_reset", False))
    assert bits_equal(ref["spike_seq"], g["spike"].flatten(1))
    assert bits_equal(ref["v_seq"], g["v_seq"].flatten(1))
    torch.testing.assert_close(ref["grad_x"], g["grad_x"].flatten(1), rtol=1e-6, atol=0.0)
    if kind == "plif":
        torch.testing.assert_close(ref["grad_p"].reshape(1), g["grad_w"], rtol=1e-6, atol=0.0)


@pytest.mark.parametrize("name", sorted(CASES))
def test_torch_backend_nodes_reproduce_the_reference_vectors(name):
    g, node, s, v_seq, grad_x = run_node(name, "torch", "cpu")
    assert bits_equal(s, g["spike"]) and bits_equal(v_seq, g["v_seq"])
    torch.testing.assert_close(grad_x, g["grad_x"], rtol=1e-6, atol=0.0)
    if "grad_w" in g:
        torch.testing.assert_close(node.w.grad.reshape(1), g["grad_w"], rtol=1e-6, atol=0.0)


def test_charge_order_matters_on_these_vectors():
    """The vectors would catch a re-associated charge: ``v + (x - v + v_reset) / tau`` and a reciprocal multiply give
    other bits on them."""
    g = load("lif_a")
    x, v_seq = g["x"], g["v_seq"]
    v_prev = torch.cat([torch.full_like(x[:1], -0.2), v_seq[:-1]])
    spike = g["spike"]
    h_ref = v_prev - (v_prev - (-0.2)) / 3.0 + x
    v_ref = spike * -0.2 + (1.0 - spike) * h_ref
    assert bits_equal(v_ref, v_seq)
    h_alt = v_prev - (v_prev + 0.2) * torch.tensor(1.0 / 3.0) + x
    assert not bits_equal(spike * -0.2 + (1.0 - spike) * h_alt, v_seq)
    h_alt2 = (v_prev + x) - (v_prev - (-0.2)) / 3.0
    assert not bits_equal(spike * -0.2 + (1.0 - spike) * h_alt2, v_seq)


@pytest.mark.gpu
@pytest.mark.parametrize("name", [n for n in sorted(CASES) if n != "plif_b"])
def test_hip_nodes_reproduce_the_reference_vectors(name):
    g, node, s, v_seq, grad_x = run_node(name, "hip", "cuda")
    assert bits_equal(s, g["spike"]) and bits_equal(v_seq, g["v_seq"])
    torch.testing.assert_close(grad_x, g["grad_x"], **grad_tolerance(g["x"].dtype))
    if "grad_w" in g:
        torch.testing.assert_close(node.w.grad.cpu().reshape(1), g["grad_w"], rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
def test_hip_plif_operator_reproduces_the_reference_vectors_with_the_stored_k():
    """``init_tau = 3.5``: ``k = sigmoid(w)`` is not a power of two and a device sigmoid may round it differently from
    the CPU, so the operator is fed the fp32 ``k`` the reference computed."""
    from spikingjelly_amd.activation_based.hip_kernel import neuron_kernel as K

    g = load("plif_b")
    x = g["x"].cuda().requires_grad_(True)
    k = g["k"].cuda().reshape(()).requires_grad_(True)
    v0 = torch.full_like(x[0], -0.2)
    out = K.hip_multistep_plif_forward(x, v0, k, 1.0, -0.2, False, False, False, no.SG_IDS["atan"], 2.0, True, 0, False)
    out[0].backward(g["grad_spike"].cuda())
    assert bits_equal(out[0].detach().cpu(), g["spike"]) and bits_equal(out[1].detach().cpu(), g["v_seq"])
    torch.testing.assert_close(x.grad.cpu(), g["grad_x"], rtol=1e-5, atol=1e-6)
    kf = float(g["k"])
    torch.testing.assert_close(k.grad.cpu().reshape(1) * kf * (1.0 - kf), g["grad_w"], rtol=1e-4, atol=1e-5)
