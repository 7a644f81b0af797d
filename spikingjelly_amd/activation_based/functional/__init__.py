from .neuron import *  # noqa: F401,F403
from .net_config import *  # noqa: F401,F403
from . import neuron, net_config  # noqa: F401
