"""numpy restatement of the reference's spike bit-packing.  Test infrastructure only.

Follows the torch path of ``spikingjelly/activation_based/triton_kernel/compress.py:19-44``
(identical to ``memopt/compress.py:32-54``): cast to bool, flatten, OR bit ``i`` of byte ``j`` from
element ``8j+i``; decompress reads ``(byte >> i) & 1``.
"""

from __future__ import annotations

import numpy as np


def bit_spike_compress(s_seq: np.ndarray) -> np.ndarray:
    bits = (np.asarray(s_seq) != 0).reshape(-1)  # .to(dtype=torch.bool).reshape(-1), compress.py:20
    n_bytes = (bits.size + 7) // 8  # compress.py:21
    out = np.zeros(n_bytes, dtype=np.uint8)
    for i in range(8):  # compress.py:25-29
        sliced = bits[i::8].astype(np.uint8)
        if sliced.size > 0:
            out[: sliced.size] |= (sliced << i).astype(np.uint8)
    return out


def bit_spike_decompress(packed: np.ndarray, shape) -> np.ndarray:
    n = int(np.prod(shape, dtype=np.int64))  # compress.py:36
    out = np.zeros(n, dtype=np.uint8)
    for i in range(8):  # compress.py:40-43
        sliced_len = (n - i + 7) // 8
        out[i::8] = ((packed >> i) & 1)[:sliced_len]
    return out.reshape(shape)
