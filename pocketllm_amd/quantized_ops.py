"""Linear / embedding modules over raw GGUF blocks.

Host-side mirror of the reference's src/components/gguf/quantized_ops.py: same class names,
constructor arguments, properties, dispatch by row count (one activation row takes the decode
operator, more rows the prefill operator), output cast and exception types.  The native library is
mandatory: construction raises RuntimeError when it is not built; nothing falls back to a CPU path.
"""
from __future__ import annotations

import torch

from pocketllm_amd.cuda_loader import load_cuda_kernel
from pocketllm_amd.quantized_tensor import QuantizedGGUFTensor


def _require_kernel(what: str, attr: str | None = None):
    mod = load_cuda_kernel()
    if mod is None or (attr is not None and not hasattr(mod, attr)):
        raise RuntimeError(f"{what}: the native HIP library is required")
    return mod


_GRID_CACHE: dict[tuple[int, str], torch.Tensor] = {}


class _BlockModule:
    """Shared state of the block-backed modules: the tensor, the output dtype and the grid argument."""

    def __init__(self, tensor: QuantizedGGUFTensor, out_dtype: torch.dtype, what: str):
        self.tensor = tensor
        self.out_dtype = out_dtype
        self._cuda = _require_kernel(what)
        # callers of the reference pass an empty grid for the non-codebook types; codebook types get
        # the grid they would upload (the kernels carry the codebooks themselves)
        self._grid = self._grid_for(tensor)

    @staticmethod
    def _grid_for(tensor: QuantizedGGUFTensor) -> torch.Tensor:
        """The codebook tensor of the tensor's type on the tensor's device (empty for the table-free types), one upload per
        (type, device) shared by every module."""
        dev = tensor.blocks.device
        key = (int(tensor.type_id) if int(tensor.type_id) in (0, 2, 5, 6) else -1, str(dev))
        grid = _GRID_CACHE.get(key)
        if grid is None:
            from pocketllm_amd.codebooks import grid_tensor_for_type
            grid = grid_tensor_for_type(key[0]).to(dev)
            _GRID_CACHE[key] = grid
        return grid


class QuantizedGGUFLinear(_BlockModule):
    """y = x W^T over raw GGUF super-blocks (reference: quantized_ops.py:9-75)."""

    def __init__(self, tensor: QuantizedGGUFTensor, *, out_dtype: torch.dtype = torch.float16):
        super().__init__(tensor, out_dtype, "QuantizedGGUFLinear")

    @property
    def in_dim(self) -> int:
        return int(self.tensor.row_elems)

    @property
    def out_dim(self) -> int:
        return int(self.tensor.out_dim)

    @property
    def row_start(self) -> int:
        return int(self.tensor.row_start)

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        if x.size(-1) != self.in_dim:
            raise ValueError(f"{self.tensor.source_name}: expected input dim {self.in_dim}, got {x.size(-1)}")
        t = self.tensor
        op = self._cuda.gguf_quant_gemm_prefill_forward if x.numel() // self.in_dim > 1 else self._cuda.gguf_quant_gemm_forward
        return op(x.contiguous(), t.blocks, int(t.row_elems), int(t.type_id), self._grid).to(self.out_dtype)

    @staticmethod
    def pair(first: "QuantizedGGUFLinear", second: "QuantizedGGUFLinear", x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        for name, a, b in (("input dims", first.in_dim, second.in_dim), ("output dims", first.out_dim, second.out_dim),
                           ("type ids", first.tensor.type_id, second.tensor.type_id)):
            if a != b:
                raise ValueError(f"paired GGUF GEMM requires matching {name}, got {a} and {b}")
        if x.size(-1) != first.in_dim:
            raise ValueError(f"paired GGUF GEMM expected input dim {first.in_dim}, got {x.size(-1)}")
        a, b = first.tensor, second.tensor
        y = first._cuda.gguf_quant_gemm_pair_forward(x.contiguous(), a.blocks, int(a.row_elems), int(a.type_id),
                                                     b.blocks, int(b.row_elems), int(b.type_id), first._grid)
        return y[0].to(first.out_dtype), y[1].to(second.out_dtype)


class Q8_0GGUFLinear:
    """y = x W^T over raw Q8_0 blocks `[out_dim, blocks_per_row, 34]` (reference: quantized_ops.py:78-123)."""

    def __init__(self, blocks: torch.Tensor, row_elems: int, *, source_name: str = "",
                 out_dtype: torch.dtype = torch.float16, row_start: int = 0):
        if blocks.dim() != 3 or blocks.size(-1) != 34:
            raise ValueError(f"q8_0 blocks must be [N, K_blocks, 34], got {tuple(blocks.shape)}")
        self.blocks = blocks.contiguous()
        self.row_elems = int(row_elems)
        self.source_name = source_name
        self.out_dtype = out_dtype
        self._row_start = int(row_start)
        self._cuda = _require_kernel("Q8_0GGUFLinear", "q8_0_gemm_forward")

    @property
    def in_dim(self) -> int:
        return self.row_elems

    @property
    def out_dim(self) -> int:
        return int(self.blocks.size(0))

    @property
    def row_start(self) -> int:
        return self._row_start

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        if x.size(-1) != self.in_dim:
            raise ValueError(f"{self.source_name}: expected input dim {self.in_dim}, got {x.size(-1)}")
        return self._cuda.q8_0_gemm_forward(x.contiguous(), self.blocks, self.row_elems).to(self.out_dtype)


class QuantizedGGUFEmbedding(_BlockModule):
    """Selected-row dequantization of raw GGUF blocks (reference: quantized_ops.py:126-151)."""

    def __init__(self, tensor: QuantizedGGUFTensor, *, out_dtype: torch.dtype = torch.float16):
        super().__init__(tensor, out_dtype, "QuantizedGGUFEmbedding")

    @property
    def dim(self) -> int:
        return int(self.tensor.row_elems)

    def __call__(self, token_ids: torch.Tensor) -> torch.Tensor:
        ids = token_ids if token_ids.dtype == torch.long else token_ids.to(torch.long)
        t = self.tensor
        return self._cuda.gguf_quant_embedding_forward(ids.contiguous(), t.blocks, int(t.row_elems), int(t.type_id), self._grid).to(self.out_dtype)
