"""GGUF file -> raw-block tensors for the quantized operators.

The kernels consume exactly the bytes a GGUF file stores: a 2-D quantized tensor is `out_dim` rows of
`ceil(in_dim / 256)` super-blocks (Q8_0: `ceil(in_dim / 32)` blocks of 34 bytes), a routed expert tensor the
same per expert, experts outermost.  This reader maps the file, walks the header (version 2 or 3), and hands
out those bytes as `uint8 [N, blocks_per_row, block_bytes]` / `[E, N, blocks_per_row, block_bytes]` views or
device tensors without touching them; nothing is dequantized or repacked.

Mirrors the raw-block side of the reference's reader (src/loader/gguf/reader.py:25-230 for the header,
src/loader/gguf/tensor_reader.py:387-413, 461-510 for `read_routed_layer_blocks`, `read_q8_0_blocks`,
`read_quantized_matrix_blocks` / `_block_rows`): same method names, argument meaning and error types.
Host to device copies go through two pinned staging buffers so that the next chunk is read from the file
mapping while the previous one is on its way.
"""
from __future__ import annotations

import mmap
import struct
import warnings
from dataclasses import dataclass
from typing import Any

import torch

from .quant_types import GGUF_DENSE_TYPE_IDS
from .quantized_tensor import QuantizedGGUFTensor

# ggml type id -> (name, elements per block, bytes per block); only what a GGUF checkpoint of this path can hold
GGML_TYPES = {
    0: ("f32", 1, 4), 1: ("f16", 1, 2), 8: ("q8_0", 32, 34), 10: ("q2_k", 256, 84), 11: ("q3_k", 256, 110),
    12: ("q4_k", 256, 144), 13: ("q5_k", 256, 176), 14: ("q6_k", 256, 210), 16: ("iq2_xxs", 256, 66), 17: ("iq2_xs", 256, 74),
    18: ("iq3_xxs", 256, 98), 23: ("iq4_xs", 256, 136), 24: ("i8", 1, 1), 25: ("i16", 1, 2), 26: ("i32", 1, 4), 27: ("i64", 1, 8),
    28: ("f64", 1, 8), 29: ("iq1_m", 256, 56), 30: ("bf16", 1, 2),
}
# types the raw-block readers serve (super-block formats with a kernel type id, and Q8_0)
RAW_BLOCK_TYPES = {name: (elems, nbytes) for name, elems, nbytes in GGML_TYPES.values() if name in GGUF_DENSE_TYPE_IDS}

_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_STRING, _ARRAY = 8, 9
_STAGE_BYTES = 64 << 20


@dataclass(frozen=True)
class GGUFTensorInfo:
    name: str
    dimensions: tuple[int, ...]        # GGUF order: dimensions[0] is the innermost (row) length
    type_id: int
    offset: int                        # relative to the data section
    absolute_offset: int

    @property
    def type_name(self) -> str:
        return GGML_TYPES.get(self.type_id, (f"unknown_{self.type_id}", 0, 0))[0]

    @property
    def nbytes(self) -> int | None:
        if self.type_id not in GGML_TYPES:
            return None
        _, elems, nbytes = GGML_TYPES[self.type_id]
        rows = 1
        for d in self.dimensions[1:]:
            rows *= int(d)
        return rows * ((int(self.dimensions[0]) + elems - 1) // elems) * nbytes


class _Cursor:
    def __init__(self, buf, pos: int = 0):
        self.buf, self.pos = buf, pos

    def unpack(self, fmt: str):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise ValueError("GGUF header is truncated")
        (value,) = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += size
        return value

    def string(self) -> str:
        n = self.unpack("<Q")
        if self.pos + n > len(self.buf):
            raise ValueError("GGUF header is truncated")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8", errors="replace")
        self.pos += n
        return s

    def value(self, vtype: int, keep_arrays_up_to: int = 64) -> Any:
        if vtype in _SCALARS:
            return self.unpack(_SCALARS[vtype])
        if vtype == _STRING:
            return self.string()
        if vtype == _ARRAY:
            item, count = self.unpack("<I"), self.unpack("<Q")
            if item in _SCALARS and count > keep_arrays_up_to:     # token tables and the like: skipped, not materialised
                self.pos += struct.calcsize(_SCALARS[item]) * count
                return None
            values = [self.value(item, keep_arrays_up_to) for _ in range(count)]
            return values if count <= keep_arrays_up_to else None
        raise ValueError(f"unknown GGUF metadata value type {vtype}")


class GGUFBlockReader:
    """Memory-maps a GGUF file and serves its quantized tensors as raw blocks."""

    def __init__(self, path: str):
        self.path = str(path)
        self._file = open(self.path, "rb")
        try:
            self._mmap = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ)
        except Exception:
            self._file.close()
            raise
        self._stage: list[torch.Tensor] = []
        try:
            self._parse()
        except Exception:
            self.close()
            raise

    # ---- header ------------------------------------------------------------------------------------
    def _parse(self) -> None:
        cur = _Cursor(self._mmap)
        if bytes(self._mmap[:4]) != b"GGUF":
            raise ValueError(f"{self.path} is not a GGUF file")
        cur.pos = 4
        self.version = cur.unpack("<I")
        if self.version not in (2, 3):
            raise ValueError(f"unsupported GGUF version {self.version}")
        n_tensors, n_kv = cur.unpack("<Q"), cur.unpack("<Q")
        self.metadata: dict[str, Any] = {}
        for _ in range(n_kv):
            key = cur.string()
            self.metadata[key] = cur.value(cur.unpack("<I"))
        records = []
        for _ in range(n_tensors):
            name = cur.string()
            n_dims = cur.unpack("<I")
            dims = tuple(cur.unpack("<Q") for _ in range(n_dims))
            records.append((name, dims, cur.unpack("<I"), cur.unpack("<Q")))
        self.alignment = int(self.metadata.get("general.alignment") or 32)
        self.data_offset = (cur.pos + self.alignment - 1) // self.alignment * self.alignment
        self.tensors: dict[str, GGUFTensorInfo] = {}
        for name, dims, type_id, offset in records:
            info = GGUFTensorInfo(name, dims, type_id, offset, self.data_offset + offset)
            if info.nbytes is not None and info.absolute_offset + info.nbytes > len(self._mmap):
                raise ValueError(f"tensor {name} runs past the end of {self.path}")
            self.tensors[name] = info

    def close(self) -> None:
        self._stage = []
        if getattr(self, "_mmap", None) is not None:
            try:
                self._mmap.close()
            except BufferError:          # views handed out are still alive: the mapping goes with them
                pass
            self._mmap = None
        if getattr(self, "_file", None) is not None:
            self._file.close()
            self._file = None

    def __enter__(self) -> "GGUFBlockReader":
        return self

    def __exit__(self, *exc) -> None:
        self.close()

    def _tensor(self, name: str | GGUFTensorInfo) -> GGUFTensorInfo:
        if isinstance(name, GGUFTensorInfo):
            return name
        try:
            return self.tensors[name]
        except KeyError:
            raise KeyError(f"tensor {name} not found in {self.path}") from None

    # ---- bytes -> tensors ----------------------------------------------------------------------------
    def _bytes(self, offset: int, nbytes: int, shape: tuple[int, ...], device) -> torch.Tensor:
        view = memoryview(self._mmap)[offset:offset + nbytes]
        with warnings.catch_warnings():          # the mapping is read-only on purpose; nothing here writes through the tensor
            warnings.simplefilter("ignore", UserWarning)
            host = torch.frombuffer(view, dtype=torch.uint8, count=nbytes) if nbytes else torch.empty(0, dtype=torch.uint8)
        if device is None or torch.device(device).type == "cpu":
            return host.view(shape)
        device = torch.device(device)
        out = torch.empty(nbytes, dtype=torch.uint8, device=device)
        if not self._stage:
            self._stage = [torch.empty(_STAGE_BYTES, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
        events = [None, None]
        with torch.cuda.device(device):
            for i, start in enumerate(range(0, nbytes, _STAGE_BYTES)):
                n = min(_STAGE_BYTES, nbytes - start)
                slot = i & 1
                if events[slot] is not None:
                    events[slot].synchronize()               # the copy that last used this staging buffer has left it
                self._stage[slot][:n].copy_(host[start:start + n])
                out[start:start + n].copy_(self._stage[slot][:n], non_blocking=True)
                events[slot] = torch.cuda.Event()
                events[slot].record()
            for ev in events:
                if ev is not None:
                    ev.synchronize()
        return out.view(shape)

    def _raw_geometry(self, tensor: GGUFTensorInfo, what: str) -> tuple[int, int, int]:
        if tensor.type_name not in RAW_BLOCK_TYPES:
            raise NotImplementedError(f"{what} for {tensor.name} ({tensor.type_name}) are not supported")
        elems, block_bytes = RAW_BLOCK_TYPES[tensor.type_name]
        in_dim = int(tensor.dimensions[0])
        return in_dim, (in_dim + elems - 1) // elems, block_bytes

    def read_quantized_matrix_block_rows(self, name, row_start: int, row_count: int, device=None) -> tuple[torch.Tensor, str, int]:
        """Rows [row_start, row_start + row_count) of a 2-D quantized tensor: (blocks [rows, blocks_per_row, block_bytes], type name, in_dim)."""
        tensor = self._tensor(name)
        if len(tensor.dimensions) != 2:
            raise ValueError(f"{tensor.name} is not a 2D quantized matrix tensor")
        in_dim, bpr, bb = self._raw_geometry(tensor, "raw quantized matrix blocks")
        rows = int(tensor.dimensions[1])
        row_start, row_count = int(row_start), int(row_count)
        if row_start < 0 or row_count < 0 or row_start + row_count > rows:
            raise ValueError(f"row range [{row_start}, {row_start + row_count}) is outside {tensor.name} rows={rows}")
        offset = tensor.absolute_offset + row_start * bpr * bb
        return self._bytes(offset, row_count * bpr * bb, (row_count, bpr, bb), device), tensor.type_name, in_dim

    def read_quantized_matrix_blocks(self, name, device=None) -> tuple[torch.Tensor, str, int]:
        tensor = self._tensor(name)
        if len(tensor.dimensions) != 2:
            raise ValueError(f"{tensor.name} is not a 2D quantized matrix tensor")
        return self.read_quantized_matrix_block_rows(tensor, 0, int(tensor.dimensions[1]), device)

    def read_routed_layer_blocks(self, name, expert_start: int = 0, expert_count: int | None = None, device=None) -> tuple[torch.Tensor, str, int]:
        """A routed expert tensor (GGUF dims [in_dim, out_dim, n_experts]): (blocks [experts, out_dim, blocks_per_row, block_bytes], type name, in_dim)."""
        tensor = self._tensor(name)
        if len(tensor.dimensions) != 3:
            raise ValueError(f"{tensor.name} is not a routed expert tensor")
        in_dim, bpr, bb = self._raw_geometry(tensor, "routed expert raw blocks")
        if tensor.type_name != "q8_0" and in_dim % 256 != 0:
            raise ValueError(f"{tensor.name} in_dim={in_dim} is not divisible by 256")
        out_dim, n_experts = int(tensor.dimensions[1]), int(tensor.dimensions[2])
        expert_start = int(expert_start)
        expert_count = n_experts - expert_start if expert_count is None else int(expert_count)
        if expert_start < 0 or expert_count < 0 or expert_start + expert_count > n_experts:
            raise ValueError(f"expert range [{expert_start}, {expert_start + expert_count}) is outside {tensor.name} experts={n_experts}")
        expert_bytes = out_dim * bpr * bb
        offset = tensor.absolute_offset + expert_start * expert_bytes
        return self._bytes(offset, expert_count * expert_bytes, (expert_count, out_dim, bpr, bb), device), tensor.type_name, in_dim

    def read_q8_0_blocks(self, name, device=None) -> torch.Tensor:
        tensor = self._tensor(name)
        if tensor.type_name != "q8_0":
            raise NotImplementedError(f"raw q8_0 blocks for {tensor.name} ({tensor.type_name}) are not supported")
        rows = 1
        for d in tensor.dimensions[1:]:
            rows *= int(d)
        return self.read_q8_0_block_rows(tensor, 0, rows, device)

    def read_q8_0_block_rows(self, name, row_start: int, row_count: int, device=None) -> torch.Tensor:
        tensor = self._tensor(name)
        if tensor.type_name != "q8_0":
            raise NotImplementedError(f"raw q8_0 block rows for {tensor.name} ({tensor.type_name}) are not supported")
        rows = 1
        for d in tensor.dimensions[1:]:
            rows *= int(d)
        row_start, row_count = int(row_start), int(row_count)
        if row_start < 0 or row_count < 0 or row_start + row_count > rows:
            raise ValueError(f"row range [{row_start}, {row_start + row_count}) is outside {tensor.name} rows={rows}")
        bpr = (int(tensor.dimensions[0]) + 31) // 32
        return self._bytes(tensor.absolute_offset + row_start * bpr * 34, row_count * bpr * 34, (row_count, bpr, 34), device)

    def quantized_tensor(self, name, device=None, row_start: int = 0, row_count: int | None = None) -> QuantizedGGUFTensor:
        """A 2-D super-block tensor (or a range of its rows) as the carrier the linear / embedding modules take."""
        tensor = self._tensor(name)
        if tensor.type_name == "q8_0":
            raise NotImplementedError(f"{tensor.name} is q8_0: use read_q8_0_blocks and Q8_0GGUFLinear")
        rows = int(tensor.dimensions[1]) if len(tensor.dimensions) == 2 else 0
        count = rows - int(row_start) if row_count is None else int(row_count)
        blocks, type_name, in_dim = self.read_quantized_matrix_block_rows(tensor, row_start, count, device)
        return QuantizedGGUFTensor.from_blocks(blocks, type_name, in_dim, source_name=tensor.name, row_start=int(row_start))
