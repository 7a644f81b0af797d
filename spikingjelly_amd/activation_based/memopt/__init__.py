from .checkpointing import (  # noqa: F401
    GCContainer,
    InputCompressedGC,
    TCGCContainer,
    in_gc_1st_forward,
    input_compressed_gc,
    query_autocast,
    to_gc_function,
)
from .compress import (  # noqa: F401
    BaseSpikeCompressor,
    BitSpikeCompressor,
    BooleanSpikeCompressor,
    NullSpikeCompressor,
    Uint8SpikeCompressor,
)
