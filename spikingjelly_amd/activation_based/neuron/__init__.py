from .activation_aware_if import ActivationAwareIFNode
from .adapt import AdaptBaseNode, IzhikevichNode
from .base_node import BaseNode
from .ilif import ILIFNode
from .integrate_and_fire import IFNode
from .lif import LIFNode
from .nonlinear_if import EIFNode, QIFNode
from .plif import ParametricLIFNode
from .spikezip import STBIFNeuron

__all__ = ["BaseNode", "IFNode", "LIFNode", "ParametricLIFNode", "QIFNode", "EIFNode", "ILIFNode", "STBIFNeuron", "ActivationAwareIFNode", "AdaptBaseNode", "IzhikevichNode"]
