"""IQ2_XXS / IQ1_M / IQ2_XS / IQ3_XXS codebooks as host arrays and tensors.

The kernels carry their own copy of these constants (compiled from csrc/ggml_codebooks.inc and
staged in LDS), so nothing here is needed to run them.  The tensor getters exist because callers of
the reference operator surface pass a grid tensor on every call
(src/loader/gguf/tensor_reader.py:177-250): the shapes and values match what those callers
build, and the operators validate them the way the reference extension does.
"""
from __future__ import annotations

import re
from functools import lru_cache
from pathlib import Path

import numpy as np
import torch

_INC = Path(__file__).resolve().parent / "csrc" / "ggml_codebooks.inc"


def _table(name: str) -> list[int]:
    text = _INC.read_text(encoding="utf-8")
    m = re.search(r"PLLM_TABLE_U\d+\(%s,\s*\d+\)(.*?)PLLM_TABLE_END" % re.escape(name), text, flags=re.S)
    if m is None:
        raise RuntimeError(f"codebook table {name} missing from {_INC}")
    return [int(v, 16) for v in re.findall(r"0x[0-9a-fA-F]+", m.group(1))]


@lru_cache(maxsize=1)
def iq2xxs_grid() -> np.ndarray:
    """(256, 8) uint8 magnitudes (8, 25 or 43)."""
    return np.asarray(_table("PLLM_IQ2XXS_GRID"), dtype="<u8").view(np.uint8).reshape(256, 8).copy()


@lru_cache(maxsize=1)
def ksigns() -> np.ndarray:
    """(128,) uint8: 7-bit sign index with its parity in bit 7."""
    return np.asarray([i | ((bin(i).count("1") & 1) << 7) for i in range(128)], dtype=np.uint8)


@lru_cache(maxsize=1)
def iq2xxs_signed_grid() -> np.ndarray:
    """(256, 128, 8) int8: grid entry x sign pattern, the layout reference callers upload."""
    bits = (ksigns()[:, None] >> np.arange(8)[None, :]) & 1
    signs = np.where(bits != 0, -1, 1).astype(np.int16)
    return (iq2xxs_grid().astype(np.int16)[:, None, :] * signs[None, :, :]).astype(np.int8)


@lru_cache(maxsize=1)
def iq1_grid() -> np.ndarray:
    """(2048, 8) int8 in {-1, 0, 1}."""
    packed = np.asarray(_table("PLLM_IQ1_GRID_PACKED"), dtype=np.uint16)
    vals = (packed[:, None] >> (2 * np.arange(8, dtype=np.uint16))[None, :]) & 3
    return (vals.astype(np.int8) - 1).astype(np.int8)


def _sign_factors() -> np.ndarray:
    """(128, 8) int16 of +1 / -1: bit j of ksigns()[i] set means lane j is negated."""
    bits = (ksigns()[:, None] >> np.arange(8)[None, :]) & 1
    return np.where(bits != 0, -1, 1).astype(np.int16)


@lru_cache(maxsize=1)
def iq2xs_grid() -> np.ndarray:
    """(512, 8) uint8 magnitudes (8, 25 or 43)."""
    return np.asarray(_table("PLLM_IQ2XS_GRID"), dtype="<u8").view(np.uint8).reshape(512, 8).copy()


@lru_cache(maxsize=1)
def iq3xxs_grid() -> np.ndarray:
    """(256, 4) uint8 magnitudes (4 ... 62)."""
    return np.asarray(_table("PLLM_IQ3XXS_GRID"), dtype="<u4").view(np.uint8).reshape(256, 4).copy()


@lru_cache(maxsize=1)
def iq2xs_signed_grid() -> np.ndarray:
    """(512, 128, 8) int8: grid entry x sign pattern (src/loader/gguf/tensor_reader.py:177-187)."""
    return (iq2xs_grid().astype(np.int16)[:, None, :] * _sign_factors()[None, :, :]).astype(np.int8)


@lru_cache(maxsize=1)
def iq3xxs_signed_grid() -> np.ndarray:
    """(256, 128, 8) int8: the 4-weight entry under the low and under the high half of each sign
    pattern, side by side (src/loader/gguf/tensor_reader.py:190-203)."""
    entry = np.tile(iq3xxs_grid().astype(np.int16), (1, 2))
    return (entry[:, None, :] * _sign_factors()[None, :, :]).astype(np.int8)


def get_iq2xxs_signed_grid_tensor() -> torch.Tensor:
    return torch.from_numpy(iq2xxs_signed_grid().copy()).contiguous()


def get_iq1_grid_tensor() -> torch.Tensor:
    return torch.from_numpy(iq1_grid().copy()).contiguous()


def get_iq2xs_signed_grid_tensor() -> torch.Tensor:
    return torch.from_numpy(iq2xs_signed_grid().copy()).contiguous()


def get_iq3xxs_signed_grid_tensor() -> torch.Tensor:
    return torch.from_numpy(iq3xxs_signed_grid().copy()).contiguous()


def get_iq2xs_iq3xxs_signed_grid_tensor() -> torch.Tensor:
    """Both tables flattened back to back: the one tensor callers pass for type ids 5 and 6
    (src/loader/gguf/tensor_reader.py:234-243)."""
    return torch.cat([get_iq2xs_signed_grid_tensor().reshape(-1), get_iq3xxs_signed_grid_tensor().reshape(-1)]).contiguous()


def grid_tensor_for_type(type_id: int) -> torch.Tensor:
    """The grid tensor the operators expect beside blocks of this type id (empty where the type has
    no codebook), on the CPU: callers move it to their device once and keep it."""
    type_id = int(type_id)
    if type_id == 0:
        return get_iq2xxs_signed_grid_tensor()
    if type_id == 2:
        return get_iq1_grid_tensor()
    if type_id in (5, 6):
        return get_iq2xs_iq3xxs_signed_grid_tensor()
    return torch.empty(0, dtype=torch.int8)
