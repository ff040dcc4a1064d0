"""Loader for oracle/_ref: the reference's own C++ CPU kernels, compiled by oracle/Makefile.

TEST INFRASTRUCTURE ONLY.  Wraps the three GGUF entry points of the reference's CPU extension
(src/csrc/deepseek_cpu_moe_ext.cpp:2759-3007); they serve IQ2_XXS (type 0) and Q2_K (type 1).
"""
from __future__ import annotations

import importlib.machinery
import importlib.util
from pathlib import Path

import numpy as np

_SO = Path(__file__).resolve().parent / "_ref" / "deepseek_cpu_moe_ext.so"
_MOD = None


def available() -> bool:
    return _SO.exists()


def _mod():
    global _MOD
    if _MOD is None:
        loader = importlib.machinery.ExtensionFileLoader("deepseek_cpu_moe_ext", str(_SO))
        spec = importlib.util.spec_from_loader("deepseek_cpu_moe_ext", loader)
        mod = importlib.util.module_from_spec(spec)
        loader.exec_module(mod)
        _MOD = mod
    return _MOD


def quantized_matmul(x: np.ndarray, blocks: np.ndarray, type_id: int, signed_grid: np.ndarray) -> np.ndarray:
    """out[t, r] = dot(x[t], row r) with the reference's AVX2 block dots (float32 accumulate).

    x float32 [T, K]; blocks uint8 [N, K/256, bb]; signed_grid int8 [256, 128, 8] (used by type 0).
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    grid = np.ascontiguousarray(signed_grid, dtype=np.int8)
    t, k = x.shape
    n, bpr, bb = blocks.shape
    out = np.zeros((t, n), dtype=np.float32)
    _mod().gguf_quantized_matmul(x.ctypes.data, blocks.ctypes.data, out.ctypes.data,
                                 t, k, n, bpr, bb, int(type_id), grid.ctypes.data)
    return out


def expert_forward(x, route_w, w1, w3, w2, t1, t3, t2, swiglu_limit, signed_grid) -> np.ndarray:
    """One expert applied to T tokens: W2 (silu(W1 x) * (W3 x) * w).  x float32 [T, D]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w1 = np.ascontiguousarray(w1); w3 = np.ascontiguousarray(w3); w2 = np.ascontiguousarray(w2)
    grid = np.ascontiguousarray(signed_grid, dtype=np.int8)
    t, d = x.shape
    inter = w1.shape[0]
    out = np.zeros((t, d), dtype=np.float32)
    rw = None if route_w is None else np.ascontiguousarray(route_w, dtype=np.float32)
    _mod().gguf_expert_forward(
        x.ctypes.data, 0 if rw is None else rw.ctypes.data, out.ctypes.data,
        w1.ctypes.data, w3.ctypes.data, w2.ctypes.data,
        t, d, inter,
        w1.shape[1], w1.shape[2], int(t1), w3.shape[1], w3.shape[2], int(t3), w2.shape[1], w2.shape[2], int(t2),
        float(swiglu_limit), grid.ctypes.data)
    return out
