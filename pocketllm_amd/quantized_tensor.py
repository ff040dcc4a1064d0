"""Carrier for device-resident raw GGUF blocks (reference: src/loader/gguf/quantized_tensor.py:8-26)."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from pocketllm_amd.quant_types import GGUF_DENSE_TYPE_IDS


@dataclass(frozen=True)
class QuantizedGGUFTensor:
    """Raw blocks `[out_dim, blocks_per_row, block_bytes]` plus what a kernel needs to read them.

    `row_start` is non-zero only for row-sliced tensors (a shard of a vocabulary or lm_head matrix).
    """

    source_name: str
    blocks: torch.Tensor
    type_name: str
    type_id: int
    row_elems: int
    out_dim: int
    row_start: int = 0

    @property
    def nbytes(self) -> int:
        return int(self.blocks.numel() * self.blocks.element_size())

    @classmethod
    def from_blocks(cls, blocks: torch.Tensor, type_name: str, row_elems: int, *, source_name: str = "", row_start: int = 0):
        return cls(source_name, blocks, type_name, GGUF_DENSE_TYPE_IDS[type_name], int(row_elems), int(blocks.size(0)), int(row_start))
