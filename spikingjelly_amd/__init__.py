"""MI355X-native multi-step spiking-neuron engine.

Mirrors the module layout of SpikingJelly for the one path it implements
(``activation_based.neuron.{IFNode, LIFNode, ParametricLIFNode}`` in multi-step
mode, their surrogate functions, ``functional.reset_net``/``set_backend`` and the
``memopt`` spike bit-packing) and adds ``backend='hip'``: hand-written HIP kernels
for gfx950 behind the C ABI of ``libsjhip.so``.
"""

__version__ = "0.1.0"

from .install import install  # noqa: E402,F401
