"""Finds the native kernel module.

Same contract as the reference's src/kernels/cuda_loader.py:54-58: `load_cuda_kernel()` returns an
object exposing the quantized operators by their reference names, or None when the native library
is not built.  Callers decide what a missing library means; the operator wrappers of this package
raise.
"""
from __future__ import annotations

from typing import Optional

_NATIVE_MOD = None


def load_cuda_kernel() -> Optional[object]:
    global _NATIVE_MOD
    if _NATIVE_MOD is None:
        from pocketllm_amd import _ffi

        if _ffi.load_library() is None:
            return None
        from pocketllm_amd import hip_kernel

        _NATIVE_MOD = hip_kernel
    return _NATIVE_MOD
