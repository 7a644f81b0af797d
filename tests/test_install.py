"""``spikingjelly_amd.install``: the ``'hip'`` backend added to another package's IFNode / LIFNode / ParametricLIFNode.

The reference itself is not importable where these tests run, so they install into a stand-in package written here with
the interface ``install`` relies on (``activation_based.base.check_backend_library``; classes with a
``supported_backends`` property, a checking ``backend`` setter, ``materialize_states``, ``_memories`` and the three
forward methods that dispatch on the backend string; ``neuron/lif.py:231-398`` and ``base.py:398-430`` of the reference
have this shape).  CPU: the names appear, the setter accepts them, nothing falls back (CPU tensors and unknown surrogates
raise), other backends are untouched, a second install changes nothing.  GPU: the stand-in classes on ``'hip'`` give
what this package's own nodes give, bit for bit.
"""

import importlib
import sys
import textwrap

import pytest
import torch

import spikingjelly_amd
from spikingjelly_amd.activation_based import neuron, surrogate

from helpers import bits_equal, seeded_randn

BASE = '''
def check_backend_library(backend):
    if backend == "cupy":
        raise ImportError("CuPy is not installed!")
'''

NEURON = '''
import math
import torch
from . import base


class ATan(torch.nn.Module):
    def __init__(self, alpha=2.0, spiking=True):
        super().__init__()
        self.alpha, self.spiking = alpha, spiking

    def forward(self, x):
        return (x >= 0).to(x)


class Triangle(ATan):
    pass


class _Node(torch.nn.Module):
    def __init__(self, v_threshold=1.0, v_reset=0.0, surrogate_function=None, detach_reset=False, step_mode="s",
                 backend="torch", store_v_seq=False):
        super().__init__()
        self.v_threshold, self.v_reset, self.detach_reset = v_threshold, v_reset, detach_reset
        self.surrogate_function = surrogate_function if surrogate_function is not None else ATan()
        self.step_mode, self.store_v_seq = step_mode, store_v_seq
        self._memories = {"v": 0.0 if v_reset is None else v_reset}
        self._backend = "torch"
        self.backend = backend

    v = property(lambda self: self._memories["v"], lambda self, value: self._memories.__setitem__("v", value))

    @property
    def supported_backends(self):
        return ("torch", "cupy")

    @property
    def backend(self):
        return self._backend

    @backend.setter
    def backend(self, value):
        if value not in self.supported_backends:
            raise NotImplementedError(f"{value} is not a supported backend of {type(self).__name__}!")
        base.check_backend_library(value)
        self._backend = value

    def materialize_states(self, inputs, states, step_mode):
        ref = inputs[0][0] if step_mode == "m" else inputs[0]
        return tuple(s if isinstance(s, torch.Tensor) else torch.full_like(ref, s) for s in states)

    def charge(self, x, v):
        return v + x

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend != "torch":
            raise ValueError(self.backend)
        h = self.charge(inputs[0], states[0])
        s = self.surrogate_function(h - self.v_threshold)
        v = h - s * self.v_threshold if self.v_reset is None else s * self.v_reset + (1.0 - s) * h
        return (s,), (v, *states[1:])

    def multi_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend != "torch":
            raise ValueError(self.backend)
        out = []
        for x in inputs[0]:
            (s,), states = self.single_step_functional_forward((x,), states)
            out.append(s)
        return (torch.stack(out),), states

    def multi_step_forward(self, x_seq, *args, **kwargs):
        states = self.materialize_states((x_seq, *args), tuple(self._memories.values()), "m")
        (s,), states = self.multi_step_functional_forward((x_seq,), states)
        self.v = states[0]
        return s

    def single_step_forward(self, x):
        states = self.materialize_states((x,), tuple(self._memories.values()), "s")
        (s,), states = self.single_step_functional_forward((x,), states)
        self.v = states[0]
        return s

    def forward(self, x):
        return self.multi_step_forward(x) if self.step_mode == "m" else self.single_step_forward(x)


class IFNode(_Node):
    pass


class LIFNode(_Node):
    def __init__(self, tau=2.0, decay_input=True, **kwargs):
        super().__init__(**kwargs)
        self.tau, self.decay_input = tau, decay_input

    def charge(self, x, v):
        vr = 0.0 if self.v_reset is None else self.v_reset
        return v + (x - (v - vr)) / self.tau if self.decay_input else v - (v - vr) / self.tau + x


class ParametricLIFNode(_Node):
    def __init__(self, init_tau=2.0, decay_input=True, **kwargs):
        super().__init__(**kwargs)
        self.decay_input = decay_input
        self.w = torch.nn.Parameter(torch.as_tensor(-math.log(init_tau - 1.0)))

    def charge(self, x, v):
        vr = 0.0 if self.v_reset is None else self.v_reset
        k = self.w.sigmoid()
        return v + (x - (v - vr)) * k if self.decay_input else v - (v - vr) * k + x
'''


@pytest.fixture()
def stand_in(tmp_path, monkeypatch):
    """A freshly written, freshly imported package ``sj_stand_in`` with the reference's dispatch interface."""
    root = tmp_path / "sj_stand_in" / "activation_based"
    root.mkdir(parents=True)
    (tmp_path / "sj_stand_in" / "__init__.py").write_text("")
    (root / "__init__.py").write_text("")
    (root / "base.py").write_text(textwrap.dedent(BASE))
    (root / "neuron.py").write_text(textwrap.dedent(NEURON))
    monkeypatch.syspath_prepend(str(tmp_path))
    for name in [n for n in sys.modules if n.startswith("sj_stand_in")]:
        del sys.modules[name]
    importlib.invalidate_caches()
    package = importlib.import_module("sj_stand_in")
    yield package
    for name in [n for n in sys.modules if n.startswith("sj_stand_in")]:
        del sys.modules[name]


def test_install_without_a_package_says_what_is_missing(monkeypatch):
    monkeypatch.setitem(sys.modules, "spikingjelly", None)  # whatever is installed, the import fails
    with pytest.raises(ImportError, match="importable `spikingjelly`"):
        spikingjelly_amd.install()
    empty = type(sys)("sj_empty_stand_in")
    with pytest.raises(ImportError, match="activation_based"):
        spikingjelly_amd.install(empty)


def test_install_adds_the_backend_and_nothing_else(stand_in):
    sn = importlib.import_module("sj_stand_in.activation_based.neuron")
    x = seeded_randn((5, 3, 16), 1, 0.4, 1.0)
    before = sn.LIFNode(tau=3.0, step_mode="m")(x)
    assert "hip" not in sn.LIFNode().supported_backends
    with pytest.raises(NotImplementedError):
        sn.LIFNode(backend="hip")
    assert spikingjelly_amd.install(stand_in) is stand_in
    spikingjelly_amd.install(stand_in)  # a second call changes nothing
    for cls in (sn.IFNode, sn.LIFNode, sn.ParametricLIFNode):
        for mode in ("s", "m"):
            names = cls(step_mode=mode).supported_backends
            assert names == ("torch", "cupy", "hip")
        node = cls(step_mode="m", backend="hip")
        assert node.backend == "hip"
    # the other backends: same results, same errors
    assert torch.equal(sn.LIFNode(tau=3.0, step_mode="m")(x), before)
    with pytest.raises(ImportError, match="CuPy"):
        sn.LIFNode(backend="cupy")
    with pytest.raises(NotImplementedError, match="triton is not a supported backend"):
        sn.LIFNode(backend="triton")


@pytest.mark.parametrize("store_v_seq", [False, True])
def test_installed_backend_does_not_fall_back(stand_in, store_v_seq):
    spikingjelly_amd.install(stand_in)
    sn = importlib.import_module("sj_stand_in.activation_based.neuron")
    x = seeded_randn((4, 2, 8), 2)
    node = sn.LIFNode(step_mode="m", backend="hip", store_v_seq=store_v_seq)
    with pytest.raises(RuntimeError, match="device"):  # a CPU tensor is refused, not served by another backend
        node(x)
    with pytest.raises(RuntimeError, match="device"):
        sn.IFNode(step_mode="s", backend="hip")(x[0])
    odd = sn.LIFNode(step_mode="m", backend="hip", store_v_seq=store_v_seq, surrogate_function=torch.nn.Identity())
    with pytest.raises(NotImplementedError, match="Identity"):
        odd(x.requires_grad_())
    quiet = sn.LIFNode(step_mode="m", backend="hip", store_v_seq=store_v_seq, surrogate_function=sn.ATan(spiking=False)).eval()
    with pytest.raises(NotImplementedError, match="spiking"):
        quiet(x)


def test_a_subclass_of_a_known_surrogate_is_translated_by_its_base(stand_in):
    from spikingjelly_amd.install import _translate_surrogate

    sn = importlib.import_module("sj_stand_in.activation_based.neuron")
    sg = _translate_surrogate(sn.Triangle(alpha=3.0))
    assert isinstance(sg, surrogate.ATan) and sg.alpha == 3.0 and sg.spiking
    own = surrogate.Sigmoid(alpha=5.0)
    assert _translate_surrogate(own) is own


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["IFNode", "LIFNode", "ParametricLIFNode"])
@pytest.mark.parametrize("store_v_seq", [False, True])
def test_installed_classes_run_the_hip_kernels(stand_in, kind, store_v_seq):
    spikingjelly_amd.install(stand_in)
    sn = importlib.import_module("sj_stand_in.activation_based.neuron")
    kw = {"IFNode": {}, "LIFNode": dict(tau=3.0, decay_input=False), "ParametricLIFNode": dict(init_tau=2.0)}[kind]
    theirs = getattr(sn, kind)(v_reset=-0.1, step_mode="m", backend="hip", store_v_seq=store_v_seq,
                               surrogate_function=sn.ATan(alpha=3.0), **kw).cuda()
    ours = getattr(neuron, kind)(v_reset=-0.1, step_mode="m", backend="hip", store_v_seq=store_v_seq,
                                 surrogate_function=surrogate.ATan(alpha=3.0), **kw).cuda()
    x = seeded_randn((6, 4, 64), 3, 0.4, 1.0).cuda()
    g = seeded_randn((6, 4, 64), 4).cuda()
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    sa, sb = theirs(xa), ours(xb)
    assert bits_equal(sa, sb) and float(sa.sum()) > 0
    assert bits_equal(theirs.v, ours.v)
    if store_v_seq:
        assert bits_equal(theirs.v_seq, ours.v_seq)
    (sa * g).sum().backward()
    (sb * g).sum().backward()
    assert bits_equal(xa.grad, xb.grad)
    if kind == "ParametricLIFNode":
        torch.testing.assert_close(theirs.w.grad, ours.w.grad)
    # a second call continues from the stored state; single-step mode runs the same kernels on one row
    assert bits_equal(theirs(x), ours(x))
    single_a = getattr(sn, kind)(step_mode="s", backend="hip", surrogate_function=sn.ATan(), **kw).cuda()
    single_b = getattr(neuron, kind)(step_mode="s", backend="hip", surrogate_function=surrogate.ATan(), **kw).cuda()
    for t in range(3):
        assert bits_equal(single_a(x[t]), single_b(x[t]))


def test_stand_in_and_install_agree_with_the_reference_interface(stand_in):
    """``tests/golden/reference_install_facts.json`` (written by ``tests/golden/make_install_facts.py`` from the
    reference's source text: ``neuron/lif.py:231-398``, ``neuron/integrate_and_fire.py``, ``neuron/plif.py``,
    ``base.py:35-90, 398-440``) lists what ``install`` relies on.  The stand-in package of these tests must have that
    interface, and what ``install`` replaces must exist in the reference under the same names and parameter lists."""
    import inspect
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_install_facts.json")) as f:
        facts = json.load(f)
    sn = importlib.import_module("sj_stand_in.activation_based.neuron")
    sb = importlib.import_module("sj_stand_in.activation_based.base")

    def parameters(fn):
        out = []
        for p in inspect.signature(fn).parameters.values():
            out.append({p.VAR_POSITIONAL: "*", p.VAR_KEYWORD: "**"}.get(p.kind, "") + p.name)
        return out

    assert parameters(sb.check_backend_library) == facts["check_backend_library"]["parameters"]
    assert facts["MemoryModule"]["backend_setter_calls_check_backend_library"]
    assert facts["MemoryModule"]["backend_setter_not_implemented_message"] == ["f'{value} is not a supported backend of {self._get_name()}!'"]
    for name, ref in facts["classes"].items():
        cls = getattr(sn, name)
        assert ref["supported_backends_is_property"] and isinstance(inspect.getattr_static(cls, "supported_backends"), property)
        for forward, params in ref["forwards"].items():
            assert parameters(getattr(cls, forward)) == params, (name, forward)
        assert parameters(cls.materialize_states) == facts["MemoryModule"]["materialize_states"]
        # the stand-in offers a subset of the reference's backends in either step mode, 'torch' among them
        for mode in ("s", "m"):
            assert set(cls(step_mode=mode).supported_backends) - {"hip"} <= set(ref["supported_backends"][mode]) | {"cupy"}
            assert "torch" in ref["supported_backends"][mode]
        with pytest.raises(NotImplementedError, match="is not a supported backend of"):
            cls(step_mode="m").backend = "no-such-backend"
    spikingjelly_amd.install(stand_in)
    for name, ref in facts["classes"].items():
        cls = getattr(sn, name)
        assert isinstance(inspect.getattr_static(cls, "supported_backends"), property)
        for forward, params in ref["forwards"].items():   # the replaced methods keep the reference's parameter lists
            assert parameters(getattr(cls, forward)) == params, (name, forward)
        for mode in ("s", "m"):
            node = cls(step_mode=mode)
            assert node.supported_backends[-1] == "hip" and "hip" not in ref["supported_backends"][mode]
    assert parameters(sb.check_backend_library) == facts["check_backend_library"]["parameters"]
