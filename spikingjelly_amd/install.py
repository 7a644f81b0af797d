"""``install()``: teach an importable ``spikingjelly`` package the ``'hip'`` backend.

The reference's neuron classes choose their kernels by a backend string: ``supported_backends`` lists what a class
accepts (``neuron/lif.py:231-238``), the ``backend`` setter checks the name against it and asks
``base.check_backend_library`` whether the library is there (``base.py:398-430``), and ``multi_step_forward`` /
``multi_step_functional_forward`` / ``single_step_functional_forward`` dispatch on it (``neuron/lif.py:243-398``,
``integrate_and_fire.py:230-369``, ``plif.py:164-261``).  ``install`` adds one more name to each of those places for
``IFNode``, ``LIFNode`` and ``ParametricLIFNode`` of the package it is given, so that

    import spikingjelly, spikingjelly_amd
    spikingjelly_amd.install(spikingjelly)
    node = spikingjelly.activation_based.neuron.LIFNode(step_mode="m", backend="hip")

runs this library's kernels behind the reference's own classes, with the reference's own surrogate objects.  Nothing is
redirected silently: a CPU tensor, an unsupported dtype or an unsupported surrogate raises exactly as with this
package's own nodes, and every other backend of the patched classes behaves as before.
"""

from __future__ import annotations

import importlib
from types import ModuleType
from typing import Optional

BACKEND = "hip"
_MARK = "_sjhip_installed"


def _translate_surrogate(surrogate_function):
    """The same surrogate as an object of this package's classes (the kernels select by class and ``alpha``); a
    surrogate the kernels do not implement raises ``NotImplementedError`` naming its class, as the reference's kernel
    backends do (``triton_kernel/surrogate_kernel.py:128-134``)."""
    from .activation_based import surrogate as ours
    from .activation_based.hip_kernel.surrogate_registry import SG_HIP_IDS

    if isinstance(surrogate_function, ours.SurrogateFunctionBase):
        return surrogate_function
    by_name = {t.__name__: t for t in SG_HIP_IDS}
    for cls in type(surrogate_function).__mro__:
        mine = by_name.get(cls.__name__)
        if mine is not None:
            if not hasattr(surrogate_function, "alpha"):
                raise TypeError("hip backend requires surrogate_function.alpha, but got "
                                f"{type(surrogate_function).__name__} without 'alpha'.")
            return mine(alpha=surrogate_function.alpha, spiking=getattr(surrogate_function, "spiking", True))
    raise NotImplementedError(
        f"hip backend only supports surrogate functions {tuple(by_name)}, but got "
        f"{type(surrogate_function).__name__}. Use backend='torch' for other surrogate functions."
    )


def _check_spiking(node) -> None:
    if not node.training and not getattr(node.surrogate_function, "spiking", True):
        raise NotImplementedError("hip backend only supports spiking surrogate functions. "
                                  "Use backend='torch' for non-spiking surrogate functions.")


def _call(node, kind: str, x, v, store_v_seq: bool, single: bool):
    """One call of this package's functional for a reference node of ``kind`` ('if', 'lif', 'plif')."""
    from .activation_based.functional import neuron as F

    _check_spiking(node)
    sg = _translate_surrogate(node.surrogate_function)
    if kind == "if":
        head = ()
    elif kind == "lif":
        head = (node.tau, node.decay_input)
    else:
        head = (node.w, node.decay_input)
    if single:
        fn = {"if": F.if_step_hip, "lif": F.lif_step_hip, "plif": F.plif_step_hip}[kind]
        return fn(x, v, *head, node.v_threshold, node.v_reset, sg, node.detach_reset)
    fn = {"if": F.if_multi_step_hip, "lif": F.lif_multi_step_hip, "plif": F.plif_multi_step_hip}[kind]
    return fn(x, v, *head, node.v_threshold, node.v_reset, sg, node.detach_reset, store_v_seq)


def _patch_class(cls, kind: str) -> None:
    if cls.__dict__.get(_MARK):
        return
    supported = cls.supported_backends
    multi_functional = cls.multi_step_functional_forward
    single_functional = cls.single_step_functional_forward
    multi = cls.multi_step_forward

    def supported_backends(self):
        names = tuple(supported.fget(self))
        return names if BACKEND in names else names + (BACKEND,)

    def multi_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend != BACKEND:
            return multi_functional(self, inputs, states, **kwargs)
        spike_seq, v, _ = _call(self, kind, inputs[0], states[0], False, False)
        return (spike_seq,), (v, *states[1:])

    def single_step_functional_forward(self, inputs, states, **kwargs):
        if self.backend != BACKEND:
            return single_functional(self, inputs, states, **kwargs)
        spike, v = _call(self, kind, inputs[0], states[0], False, True)
        return (spike,), (v, *states[1:])

    def multi_step_forward(self, x_seq, *args, **kwargs):
        if self.backend != BACKEND or not self.store_v_seq:
            # without v_seq the base class walks through multi_step_functional_forward, patched above
            return multi(self, x_seq, *args, **kwargs)
        states = self.materialize_states((x_seq, *args), tuple(self._memories.values()), "m")
        spike_seq, v, v_seq = _call(self, kind, x_seq, states[0], True, False)
        self.v = v
        self.v_seq = v_seq
        return spike_seq

    cls.supported_backends = property(supported_backends)
    cls.multi_step_functional_forward = multi_step_functional_forward
    cls.single_step_functional_forward = single_step_functional_forward
    cls.multi_step_forward = multi_step_forward
    setattr(cls, _MARK, True)


def _patch_library_check(base: ModuleType) -> None:
    original = base.check_backend_library
    if getattr(original, _MARK, False):
        return

    def check_backend_library(backend: str):
        if backend == BACKEND:
            try:
                from .activation_based.hip_kernel import library

                library.load()
            except OSError as e:
                raise ImportError("The hip backend needs libsjhip.so (make -C spikingjelly_amd/csrc)") from e
            return
        return original(backend)

    setattr(check_backend_library, _MARK, True)
    base.check_backend_library = check_backend_library


def install(package: Optional[ModuleType] = None) -> ModuleType:
    """Adds ``'hip'`` to ``IFNode``, ``LIFNode`` and ``ParametricLIFNode`` of ``package`` (default: the importable
    ``spikingjelly``) and returns the package.  Calling it again changes nothing."""
    if package is None:
        try:
            package = importlib.import_module("spikingjelly")
        except ImportError as e:
            raise ImportError("install() needs an importable `spikingjelly` package, or the package object as its "
                              "argument") from e
    name = package.__name__
    try:
        base = importlib.import_module(name + ".activation_based.base")
        neuron = importlib.import_module(name + ".activation_based.neuron")
    except ImportError as e:
        raise ImportError(f"`{name}` has no activation_based.base / activation_based.neuron to install into") from e
    classes = {"if": "IFNode", "lif": "LIFNode", "plif": "ParametricLIFNode"}
    missing = [c for c in classes.values() if not hasattr(neuron, c)]
    if missing:
        raise AttributeError(f"`{name}.activation_based.neuron` lacks {', '.join(missing)}")
    _patch_library_check(base)
    for kind, cls_name in classes.items():
        _patch_class(getattr(neuron, cls_name), kind)
    return package
