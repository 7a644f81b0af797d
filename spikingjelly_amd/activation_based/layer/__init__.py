from .attention import SpikingSelfAttention
from .container import SeqToANNContainer

__all__ = ["SeqToANNContainer", "SpikingSelfAttention"]
