"""ctypes loader for oracle/_build/librawblock_cpu.so, the plain-C restatement of the raw-block matvec (rawblock_cpu.c).

TEST INFRASTRUCTURE ONLY: built by `make -C oracle cpu`; the benchmark's CPU-baseline leg times it, tests compare it with
the numpy oracle.
"""
from __future__ import annotations

import ctypes
from pathlib import Path

import numpy as np

_SO = Path(__file__).resolve().parent / "_build" / "librawblock_cpu.so"
_LIB = None
FORMATS = {"q8_0": 0, "q4_k": 3, "q5_k": 4}


def available() -> bool:
    return _SO.exists()


def _lib():
    global _LIB
    if _LIB is None:
        lib = ctypes.CDLL(str(_SO))
        lib.rawblock_matvec_f32.restype = ctypes.c_int
        lib.rawblock_matvec_f32.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.rawblock_q8_0_dequantize.restype = None
        lib.rawblock_q8_0_dequantize.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        _LIB = lib
    return _LIB


def matvec(blocks: np.ndarray, type_name: str, x: np.ndarray) -> np.ndarray:
    """y[t, r] = dot(x[t], row r of the decoded matrix), float32.  blocks uint8 [N, blocks per row, block bytes], x [T, K]."""
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32)
    t, k = x.shape
    n, bpr, _ = blocks.shape
    y = np.empty((t, n), dtype=np.float32)
    st = _lib().rawblock_matvec_f32(blocks.ctypes.data, FORMATS[type_name], x.ctypes.data, y.ctypes.data, t, n, k, bpr)
    if st != 0:
        raise ValueError(f"rawblock_matvec_f32: format {type_name} not served")
    return y


def q8_0_dequantize(blocks: np.ndarray) -> np.ndarray:
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    n, bpr, _ = blocks.shape
    out = np.empty((n, bpr * 32), dtype=np.float32)
    _lib().rawblock_q8_0_dequantize(blocks.ctypes.data, out.ctypes.data, n, bpr)
    return out
