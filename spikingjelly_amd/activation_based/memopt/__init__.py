from .compress import (  # noqa: F401
    BaseSpikeCompressor,
    BitSpikeCompressor,
    BooleanSpikeCompressor,
    NullSpikeCompressor,
    Uint8SpikeCompressor,
)
