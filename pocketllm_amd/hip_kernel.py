"""The native operator module: reference operator names over the libpllm_hip C ABI.

Each function keeps the positional signature, argument meaning, output shape/dtype and error
behaviour (RuntimeError with the reference's message) of the operator it replaces in the
reference's `cuda_kernel` extension (src/csrc/cuda_kernel.cpp:1987-2038).  Outputs are fresh torch
tensors; kernels are enqueued on torch's current stream of x's device and return asynchronously.

One extension over the reference: a keyword-only `out_dtype` (default the reference's dtype) so that
parity checks can read the float32 accumulators before the bf16 rounding.
"""
from __future__ import annotations

import torch

from pocketllm_amd import _ffi
from pocketllm_amd.quant_types import GGUF_BLOCK_BYTES, IMPLEMENTED_TYPE_IDS

_DTYPE_CODE = {torch.float32: _ffi.DTYPE_F32, torch.float16: _ffi.DTYPE_F16, torch.bfloat16: _ffi.DTYPE_BF16}


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _lib():
    lib = _ffi.load_library()
    if lib is None:
        raise RuntimeError("libpllm_hip.so is not built (run `python -m pocketllm_amd.build`)")
    return lib


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    # scratch for the pre-quantized activations: a fresh tensor from torch's caching allocator, so
    # stream ordering and lifetime follow torch's rules exactly as the reference's temporaries do
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _check_x(x: torch.Tensor) -> None:
    _check(x.dtype in _DTYPE_CODE, "x must be float16, bfloat16, or float32")


def _check_grid(grid: torch.Tensor, type_id: int, name: str) -> None:
    # src/csrc/cuda_kernel.cpp:420-437; the kernels use their built-in codebooks, the tensor is
    # validated so that callers written against the reference fail the same way
    if type_id == 0:
        _check(grid.is_cuda, f"{name} must be CUDA for iq2_xxs")
        _check(grid.dtype == torch.int8, f"{name} must be int8")
        _check(grid.is_contiguous(), f"{name} must be contiguous")
        _check(grid.numel() == 256 * 128 * 8, f"{name} must contain 256*128*8 entries for iq2_xxs")
    elif type_id == 2:
        _check(grid.is_cuda, f"{name} must be CUDA for iq1_m")
        _check(grid.dtype == torch.int8, f"{name} must be int8")
        _check(grid.is_contiguous(), f"{name} must be contiguous")
        _check(grid.numel() == 2048 * 8, f"{name} must contain 2048*8 entries for iq1_m")


def _check_type(type_id: int, what: str = "type_id") -> None:
    _check(type_id in GGUF_BLOCK_BYTES, f"unsupported GGUF quant {what}: {type_id}")
    _check(type_id in IMPLEMENTED_TYPE_IDS, f"GGUF quant {what} {type_id} has no MI355X kernel in this build")


def q8_0_gemm_forward(x: torch.Tensor, blocks: torch.Tensor, row_elems: int, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """src/csrc/cuda_kernel.cpp:524-543."""
    row_elems = int(row_elems)
    _check(x.dim() in (2, 3), "x must have shape [M, K] or [B, S, K]")
    _check(blocks.dim() == 3, "blocks must have shape [N, K_blocks, 34]")
    _check(blocks.size(2) == 34, "q8_0 block size must be 34 bytes")
    _check(row_elems > 0, "row_elems must be positive")
    _check(x.size(-1) == row_elems, "inner dimension mismatch")
    _check(blocks.size(1) * 32 >= row_elems, "blocks do not cover row_elems")
    _check(x.is_cuda and blocks.is_cuda, "all tensors must be CUDA tensors")
    _check(x.is_contiguous(), "x must be contiguous")
    _check(blocks.dtype == torch.uint8, "blocks has unexpected dtype")
    _check(blocks.is_contiguous(), "blocks must be contiguous")
    _check_x(x)
    rows = x.numel() // row_elems
    n = blocks.size(0)
    y = torch.empty(*x.shape[:-1], n, dtype=out_dtype, device=x.device)
    if rows == 0 or n == 0:
        return y
    lib = _lib()
    with torch.cuda.device(x.device):
        ws_bytes = lib.pllm_q8_0_gemm_workspace_bytes(rows, row_elems, n, blocks.size(1))
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_q8_0_gemm(x.data_ptr(), _DTYPE_CODE[x.dtype], blocks.data_ptr(), y.data_ptr(), _DTYPE_CODE[out_dtype],
                                rows, row_elems, n, blocks.size(1), ws.data_ptr(), ws_bytes, _stream(x.device))
    _ffi.check(st, "q8_0_gemm_forward")
    return y


def _dense_checks(x, blocks, row_elems, type_id, signed_grid) -> None:
    # src/csrc/cuda_kernel.cpp:566-589
    _check(x.dim() in (2, 3), "x must have shape [M, K] or [B, S, K]")
    _check(blocks.dim() == 3, "blocks must have shape [N, K_blocks, block_bytes]")
    _check_type(type_id)
    _check(row_elems > 0, "row_elems must be positive")
    _check(x.size(-1) == row_elems, "inner dimension mismatch")
    _check(blocks.size(1) * 256 >= row_elems, "blocks do not cover row_elems")
    _check(blocks.size(2) == GGUF_BLOCK_BYTES[type_id], "unexpected GGUF block size for type_id")
    _check(x.is_cuda and blocks.is_cuda, "x and blocks must be CUDA tensors")
    _check(x.is_contiguous() and blocks.is_contiguous(), "x and blocks must be contiguous")
    _check(blocks.dtype == torch.uint8, "blocks has unexpected dtype")
    _check_x(x)
    _check_grid(signed_grid, type_id, "signed_grid")


def _dense_gemm(name, x, blocks, row_elems, type_id, signed_grid, out_dtype):
    row_elems, type_id = int(row_elems), int(type_id)
    _dense_checks(x, blocks, row_elems, type_id, signed_grid)
    rows = x.numel() // row_elems
    n = blocks.size(0)
    y = torch.empty(*x.shape[:-1], n, dtype=out_dtype, device=x.device)
    if rows == 0 or n == 0:
        return y
    lib = _lib()
    with torch.cuda.device(x.device):
        ws_bytes = lib.pllm_gguf_quant_gemm_workspace_bytes(type_id, rows, row_elems, n, blocks.size(1))
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_quant_gemm(x.data_ptr(), _DTYPE_CODE[x.dtype], blocks.data_ptr(), type_id, y.data_ptr(),
                                      _DTYPE_CODE[out_dtype], rows, row_elems, n, blocks.size(1), ws.data_ptr(), ws_bytes,
                                      _stream(x.device))
    _ffi.check(st, name)
    return y


def gguf_quant_gemm_forward(x, blocks, row_elems, type_id, signed_grid, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Decode-regime operator, src/csrc/cuda_kernel.cpp:566-589.  Any row count is accepted."""
    return _dense_gemm("gguf_quant_gemm_forward", x, blocks, row_elems, type_id, signed_grid, out_dtype)


def gguf_quant_gemm_prefill_forward(x, blocks, row_elems, type_id, signed_grid, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Prefill-regime operator, src/csrc/cuda_kernel.cpp:591-614."""
    return _dense_gemm("gguf_quant_gemm_prefill_forward", x, blocks, row_elems, type_id, signed_grid, out_dtype)


def gguf_q2k_gemm_dp4a_forward(x, blocks, row_elems, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """src/csrc/cuda_kernel.cpp:545-564."""
    _check(blocks.dim() == 3, "blocks must have shape [N, K_blocks, 84]")
    _check(blocks.size(2) == 84, "q2_k block size must be 84 bytes")
    empty = torch.empty(0, dtype=torch.int8, device=x.device)
    return _dense_gemm("gguf_q2k_gemm_dp4a_forward", x, blocks, row_elems, 1, empty, out_dtype)
