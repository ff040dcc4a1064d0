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


def gguf_dequantize_rows(blocks: torch.Tensor, type_id: int, row_elems: int, row_ids: torch.Tensor | None = None, *,
                         out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Dequantize whole or selected rows of a raw-block matrix (type_id _ffi.TYPE_Q8_0 for Q8_0 blocks).

    No direct counterpart in the reference extension: it is the device form of the numpy decoders of
    src/loader/gguf/tensor_reader.py:543-1009, with bit-identical float32 results.
    """
    type_id, row_elems = int(type_id), int(row_elems)
    q8 = type_id == _ffi.TYPE_Q8_0
    if not q8:
        _check_type(type_id)
    _check(blocks.dim() == 3 and blocks.is_cuda and blocks.dtype == torch.uint8 and blocks.is_contiguous(),
           "blocks must be a contiguous CUDA uint8 tensor [N, K_blocks, block_bytes]")
    _check(blocks.size(2) == (34 if q8 else GGUF_BLOCK_BYTES[type_id]), "unexpected GGUF block size for type_id")
    _check(row_elems > 0 and blocks.size(1) * (32 if q8 else 256) >= row_elems, "blocks do not cover row_elems")
    if row_ids is not None:
        _check(row_ids.is_cuda and row_ids.dtype == torch.int64 and row_ids.is_contiguous(), "row_ids must be contiguous CUDA int64")
        lead, count = tuple(row_ids.shape), row_ids.numel()
    else:
        lead, count = (blocks.size(0),), blocks.size(0)
    out = torch.empty(*lead, row_elems, dtype=out_dtype, device=blocks.device)
    if count == 0:
        return out
    with torch.cuda.device(blocks.device):
        st = _lib().pllm_gguf_dequantize_rows(None if row_ids is None else row_ids.data_ptr(), count, blocks.data_ptr(), type_id,
                                              blocks.size(0), row_elems, blocks.size(1), out.data_ptr(), _DTYPE_CODE[out_dtype],
                                              _stream(blocks.device))
    _ffi.check(st, "gguf_dequantize_rows")
    return out


def gguf_quant_embedding_forward(token_ids, blocks, row_elems, type_id, signed_grid, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """src/csrc/cuda_kernel.cpp:669-687.  The reference serves q4_k/q5_k only; every implemented type works here."""
    row_elems, type_id = int(row_elems), int(type_id)
    _check(token_ids.dim() in (1, 2), "token_ids must have shape [T] or [B, S]")
    _check(blocks.dim() == 3, "blocks must have shape [V, K_blocks, block_bytes]")
    _check_type(type_id)
    _check(row_elems > 0, "row_elems must be positive")
    _check(blocks.size(1) * 256 >= row_elems, "blocks do not cover row_elems")
    _check(blocks.size(2) == GGUF_BLOCK_BYTES[type_id], "unexpected GGUF block size for type_id")
    _check(token_ids.is_cuda and blocks.is_cuda, "token_ids and blocks must be CUDA tensors")
    _check(token_ids.is_contiguous() and blocks.is_contiguous(), "token_ids and blocks must be contiguous")
    _check(token_ids.dtype == torch.int64, "token_ids must be int64")
    _check(blocks.dtype == torch.uint8, "blocks has unexpected dtype")
    _check_grid(signed_grid, type_id, "signed_grid")
    return gguf_dequantize_rows(blocks, type_id, row_elems, token_ids, out_dtype=out_dtype)


def fp8_block_dequantize(weight: torch.Tensor, scale: torch.Tensor, *, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """W[r, c] = f32(code) * scale[r // 128, c // 128]  (src/kernels/ops.py:144-147)."""
    w8 = _fp8_bytes(weight)
    n, k = w8.shape
    _check(scale.is_cuda and scale.dtype == torch.float32 and scale.is_contiguous(), "scale must be a contiguous CUDA float32 tensor")
    _check(tuple(scale.shape) == ((n + 127) // 128, (k + 127) // 128), "scale must have shape [ceil(N/128), ceil(K/128)]")
    out = torch.empty(n, k, dtype=out_dtype, device=w8.device)
    with torch.cuda.device(w8.device):
        st = _lib().pllm_fp8_block_dequantize(w8.data_ptr(), scale.data_ptr(), n, k, out.data_ptr(), _DTYPE_CODE[out_dtype], _stream(w8.device))
    _ffi.check(st, "fp8_block_dequantize")
    return out


def _fp8_bytes(weight: torch.Tensor) -> torch.Tensor:
    _check(weight.dim() == 2 and weight.is_cuda and weight.is_contiguous(), "weight must be a contiguous CUDA tensor [N, K]")
    if weight.dtype == torch.float8_e4m3fn:
        return weight.view(torch.uint8)
    _check(weight.dtype == torch.uint8, "weight must be float8_e4m3fn (or its uint8 bytes)")
    return weight


def fp8_block_gemm_forward(x: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, *, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """y = x @ (f32(weight) * block scales)^T from the FP8 bytes (src/kernels/ops.py:641-648)."""
    w8 = _fp8_bytes(weight)
    n, k = w8.shape
    _check(x.is_cuda and x.is_contiguous() and x.size(-1) == k, "x must be a contiguous CUDA tensor [..., K]")
    _check_x(x)
    _check(scale.is_cuda and scale.dtype == torch.float32 and scale.is_contiguous(), "scale must be a contiguous CUDA float32 tensor")
    _check(tuple(scale.shape) == ((n + 127) // 128, (k + 127) // 128), "scale must have shape [ceil(N/128), ceil(K/128)]")
    rows = x.numel() // k
    y = torch.empty(*x.shape[:-1], n, dtype=out_dtype, device=x.device)
    if rows == 0:
        return y
    with torch.cuda.device(x.device):
        st = _lib().pllm_fp8_block_gemm(x.data_ptr(), _DTYPE_CODE[x.dtype], w8.data_ptr(), scale.data_ptr(), y.data_ptr(),
                                        _DTYPE_CODE[out_dtype], rows, k, n, _stream(x.device))
    _ffi.check(st, "fp8_block_gemm_forward")
    return y


def fp8_act_quant_forward(x: torch.Tensor, eps: float = 1e-4, round_scale_pow2: bool = False):
    """Per-(row, 128) FP8 activation quantizer (src/kernels/ops.py:501-516): returns (float8_e4m3fn codes, float32 scales)."""
    _check(x.is_cuda and x.is_contiguous(), "x must be a contiguous CUDA tensor")
    _check_x(x)
    k = x.size(-1)
    _check(k % 128 == 0, "last dimension must be a multiple of 128")
    rows = x.numel() // k
    codes = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    scales = torch.empty(*x.shape[:-1], k // 128, dtype=torch.float32, device=x.device)
    if rows:
        with torch.cuda.device(x.device):
            st = _lib().pllm_fp8_act_quant(x.data_ptr(), _DTYPE_CODE[x.dtype], rows, k, codes.data_ptr(), scales.data_ptr(),
                                           float(eps), int(bool(round_scale_pow2)), _stream(x.device))
        _ffi.check(st, "fp8_act_quant_forward")
    return codes.view(torch.float8_e4m3fn), scales
