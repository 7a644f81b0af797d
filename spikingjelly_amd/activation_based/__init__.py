from . import base, surrogate, functional, neuron  # noqa: F401
