"""GGUF dense type ids and block geometry of the quantized-op layer.

Mirrors the reference's id map (src/loader/gguf/quant_types.py:3-13, src/csrc/cuda_kernel.cpp:401-412).
Q8_0 has no type id: it is served by its own operator.
"""
from __future__ import annotations

GGUF_DENSE_TYPE_IDS = {
    "iq2_xxs": 0,
    "q2_k": 1,
    "iq1_m": 2,
    "q4_k": 3,
    "q5_k": 4,
    "iq2_xs": 5,
    "iq3_xxs": 6,
    "iq4_xs": 7,
    "q6_k": 8,
}
GGUF_DENSE_TYPE_NAMES = {v: k for k, v in GGUF_DENSE_TYPE_IDS.items()}

# bytes per 256-weight super-block, by type id (src/csrc/cuda_kernel.cpp:401-412)
GGUF_BLOCK_BYTES = {0: 66, 1: 84, 2: 56, 3: 144, 4: 176, 5: 74, 6: 98, 7: 136, 8: 210}

# type ids this library has kernels for; the others are known to the id map but raise
IMPLEMENTED_TYPE_IDS = (0, 1, 2, 3, 4, 5, 6, 7, 8)

Q8_0_BLOCK_BYTES = 34
Q8_0_BLOCK_ELEMS = 32
SUPER_BLOCK_ELEMS = 256


def block_bytes_for_type(type_id: int) -> int:
    try:
        return GGUF_BLOCK_BYTES[int(type_id)]
    except KeyError:
        raise RuntimeError(f"unsupported GGUF quant type_id: {type_id}") from None
