"""BF16 bit planes and the split-k chooser (oracle; test infrastructure only).

Restates, in numpy on raw uint16 bit patterns:

* ``split_bf16``      -- reference ``bf16_huffman_infer/utils.py:7-12``
* ``rebuild_bf16``    -- reference ``src/kernel.cu:156`` and ``:300``
* ``get_block_size_n``-- reference ``bf16_huffman_infer/utils.py:15-31``

Pins: ``rebuild(split(b)) == b`` by brute force over all 65536 bit patterns and the
field positions against IEEE bfloat16 (sign 15, exponent 14..7, mantissa 6..0);
``get_block_size_n`` against a table worked by hand from the loop bounds
(4096->1, 3584->1, 12288->3, 18944->4, 11008->2, 128/256 -> error).
"""
import numpy as np


def split_bf16(bits: np.ndarray):
    """bits: uint16 BF16 patterns -> (rem, exp) uint8 planes of the same shape.

    exp = bits 14..7; rem = sign in bit 7, mantissa in bits 6..0.
    """
    b = bits.astype(np.uint32)
    exp = ((b >> 7) & 0xFF).astype(np.uint8)
    rem = (((b >> 8) & 0x80) | (b & 0x7F)).astype(np.uint8)
    return rem, exp


def rebuild_bf16(rem: np.ndarray, exp: np.ndarray) -> np.ndarray:
    r = rem.astype(np.uint32)
    e = exp.astype(np.uint32)
    return (((r << 8) & 0x8000) | (r & 0x7F) | (e << 7)).astype(np.uint16)


def get_block_size_n(n: int) -> int:
    """Number of contiguous column blocks (split_k) for in_features ``n``."""
    if n % 128 == 0:
        q = n // 128
        for i in range(32, 2, -1):
            if q % i == 0 and q // i <= 8:
                return q // i
        for i in range(32, 129):
            if q % i == 0 and q // i <= 32:
                return q // i
        for i in range(32, 2, -1):
            if q % i == 0 and q // i <= 32:
                return q // i
    raise RuntimeError(f"Could not find suitable block size for in_features {n}")
