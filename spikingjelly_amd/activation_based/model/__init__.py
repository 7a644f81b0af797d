from . import spikformer

__all__ = ["spikformer"]
