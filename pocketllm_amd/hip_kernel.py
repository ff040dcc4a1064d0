"""The native operator module: reference operator names over the libpllm_hip C ABI.

Each function keeps the positional signature, argument meaning, output shape/dtype and error
behaviour (RuntimeError with the reference's message) of the operator it replaces in the
reference's `cuda_kernel` extension (src/csrc/cuda_kernel.cpp:1987-2038).  Outputs are fresh torch
tensors; kernels are enqueued on torch's current stream of x's device and return asynchronously.

One extension over the reference: a keyword-only `out_dtype` (default the reference's dtype) so that
parity checks can read the float32 accumulators before the bf16 rounding.
"""
from __future__ import annotations

import contextlib
import ctypes

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


def _on_device(device: torch.device):
    """Device guard for the launch: torch's context manager only when the tensor's device is not the current one (entering
    and leaving it costs a few microseconds of host time per call, which shows in eager decode loops)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return contextlib.nullcontext()
    return torch.cuda.device(device)


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
    elif type_id in (5, 6):
        _check(grid.is_cuda, f"{name} must be CUDA for iq2_xs/iq3_xxs")
        _check(grid.dtype == torch.int8, f"{name} must be int8")
        _check(grid.is_contiguous(), f"{name} must be contiguous")
        _check(grid.numel() >= 512 * 128 * 8 + 256 * 128 * 8,
               f"{name} must contain packed iq2_xs and iq3_xxs signed grids")


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
    with _on_device(x.device):
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
    with _on_device(x.device):
        ws_bytes = lib.pllm_gguf_quant_gemm_workspace_bytes(type_id, rows, row_elems, n, blocks.size(1))
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_quant_gemm(x.data_ptr(), _DTYPE_CODE[x.dtype], blocks.data_ptr(), type_id, y.data_ptr(),
                                      _DTYPE_CODE[out_dtype], rows, row_elems, n, blocks.size(1), ws.data_ptr(), ws_bytes,
                                      _stream(x.device))
    _ffi.check(st, name)
    return y


def gguf_quant_gemm_q8_forward(x, blocks, row_elems, type_id, signed_grid, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Q4_K / Q5_K matmul with the int8 activation semantics of the reference's MMA prefill path
    (src/csrc/llama_mmq/gguf_mma_wrapper.cu:257-322): activations quantized to 32-value int8 blocks, integer group dots on the
    int8 matrix cores, float32 scales.  gguf_quant_gemm_prefill_forward states the same operator with float activations."""
    row_elems, type_id = int(row_elems), int(type_id)
    _dense_checks(x, blocks, row_elems, type_id, signed_grid)
    _check(type_id in (3, 4), "int8-activation matmul serves q4_k and q5_k")
    rows = x.numel() // row_elems
    n = blocks.size(0)
    y = torch.empty(*x.shape[:-1], n, dtype=out_dtype, device=x.device)
    if rows == 0 or n == 0:
        return y
    lib = _lib()
    with _on_device(x.device):
        ws_bytes = lib.pllm_gguf_quant_gemm_q8_workspace_bytes(type_id, rows, row_elems, n, blocks.size(1))
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_quant_gemm_q8(x.data_ptr(), _DTYPE_CODE[x.dtype], blocks.data_ptr(), type_id, y.data_ptr(), _DTYPE_CODE[out_dtype],
                                         rows, row_elems, n, blocks.size(1), ws.data_ptr(), ws_bytes, _stream(x.device))
    _ffi.check(st, "gguf_quant_gemm_q8_forward")
    return y


STATIC_SCRATCH_BYTES = 16 << 20


def gguf_quant_gemm_static_scratch_forward(x, blocks, row_elems, type_id, signed_grid, y: torch.Tensor) -> torch.Tensor:
    """gguf_quant_gemm_forward / gguf_quant_gemm_prefill_forward into a caller-owned y, through the entry point that allocates no
    device memory (pllm_gguf_quant_gemm_static_scratch: its activation image and staging live in a 16 MiB array the library
    holds on the device).  For callers that cannot allocate: code under graph capture, tight serving loops.  Raises RuntimeError
    ("workspace too small") for calls that need more than the array; calls that overlap on one GPU race."""
    row_elems, type_id = int(row_elems), int(type_id)
    _dense_checks(x, blocks, row_elems, type_id, signed_grid)
    rows = x.numel() // row_elems
    n = blocks.size(0)
    _check(y.is_cuda and y.device == x.device and y.is_contiguous() and y.dtype in _DTYPE_CODE, "y must be a contiguous CUDA tensor of float16, bfloat16 or float32")
    _check(tuple(y.shape) == (*x.shape[:-1], n), "y must have x's leading shape and blocks.size(0) columns")
    if rows == 0 or n == 0:
        return y
    with _on_device(x.device):
        st = _lib().pllm_gguf_quant_gemm_static_scratch(x.data_ptr(), _DTYPE_CODE[x.dtype], blocks.data_ptr(), type_id, y.data_ptr(),
                                                        _DTYPE_CODE[y.dtype], rows, row_elems, n, blocks.size(1), _stream(x.device))
    _ffi.check(st, "gguf_quant_gemm_static_scratch_forward")
    return y


def gguf_quant_gemm_forward(x, blocks, row_elems, type_id, signed_grid, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Decode-regime operator, src/csrc/cuda_kernel.cpp:566-589.  Any row count is accepted."""
    return _dense_gemm("gguf_quant_gemm_forward", x, blocks, row_elems, type_id, signed_grid, out_dtype)


def gguf_quant_gemm_multi_forward(x, blocks_list, row_elems, type_id, signed_grid, *, norm_weight=None, eps: float = 1e-6,
                                  round_fp16: bool = True, out_dtype: torch.dtype = torch.bfloat16):
    """Several projections of one activation tensor, [gguf_quant_gemm_forward(x, b, ...) for b in blocks_list] (with norm_weight:
    gguf_quant_gemm_rmsnorm_forward), as ONE launch where the library has one: up to four matrices of any heights and one format
    (any but Q2_K) at decode row counts.  The generalization of gguf_quant_gemm_pair_forward (src/csrc/cuda_kernel.cpp:615-666) to q / k / v.
    Everything else runs one operator call per matrix.  Returns the list of outputs."""
    row_elems, type_id = int(row_elems), int(type_id)
    blocks_list = list(blocks_list)
    _check(len(blocks_list) >= 1, "blocks_list must hold at least one matrix")
    for b in blocks_list:
        _dense_checks(x, b, row_elems, type_id, signed_grid)
        _check(b.size(1) == blocks_list[0].size(1), "all matrices must have the same number of blocks per row")
    if norm_weight is not None:
        _check(norm_weight.dim() == 1 and norm_weight.size(0) == row_elems, "fused_rms_norm: weight.size(0) must == dim")
        _check(norm_weight.is_cuda and norm_weight.dtype == torch.float32 and norm_weight.is_contiguous(), "fused_rms_norm: weight must be fp32")
    rows = x.numel() // row_elems

    def one_by_one():
        if norm_weight is None:
            return [_dense_gemm("gguf_quant_gemm_multi_forward", x, b, row_elems, type_id, signed_grid, out_dtype) for b in blocks_list]
        return [gguf_quant_gemm_rmsnorm_forward(x, norm_weight, eps, b, row_elems, type_id, signed_grid, round_fp16=round_fp16, out_dtype=out_dtype)
                for b in blocks_list]

    count = len(blocks_list)
    if rows == 0 or count > 4 or any(b.size(0) == 0 for b in blocks_list):
        return one_by_one()
    ys = [torch.empty(*x.shape[:-1], b.size(0), dtype=out_dtype, device=x.device) for b in blocks_list]
    lib = _lib()
    bpr = blocks_list[0].size(1)
    with _on_device(x.device):
        ws_bytes = lib.pllm_activation_image_bytes(rows, bpr)
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_quant_gemm_multi(
            x.data_ptr(), _DTYPE_CODE[x.dtype], norm_weight.data_ptr() if norm_weight is not None else None, float(eps), int(bool(round_fp16)),
            count, (ctypes.c_void_p * count)(*[b.data_ptr() for b in blocks_list]), (ctypes.c_int64 * count)(*[b.size(0) for b in blocks_list]),
            type_id, (ctypes.c_void_p * count)(*[t.data_ptr() for t in ys]), _DTYPE_CODE[out_dtype], rows, row_elems, bpr,
            ws.data_ptr(), ws_bytes, _stream(x.device))
    if st == _ffi.PLLM_ERR_UNSUPPORTED:      # no single launch for this format or row count
        return one_by_one()
    _ffi.check(st, "gguf_quant_gemm_multi_forward")
    return ys


def gguf_quant_gemm_accumulate_forward(x, blocks, row_elems, type_id, signed_grid, y: torch.Tensor) -> torch.Tensor:
    """y += gguf_quant_gemm_forward(x, ...) in place, the residual connection of a transformer block
    (src/models/minimax_m2/architecture.py:412-413) folded into the projection: one launch for decode calls, the sum formed in
    float32 and rounded to y's type once.  Row counts that the plain operator hands to the tile kernel run it and add separately."""
    row_elems, type_id = int(row_elems), int(type_id)
    _dense_checks(x, blocks, row_elems, type_id, signed_grid)
    rows = x.numel() // row_elems
    n = blocks.size(0)
    _check(y.is_cuda and y.device == x.device and y.is_contiguous() and y.dtype in _DTYPE_CODE, "y must be a contiguous CUDA tensor of float16, bfloat16 or float32")
    _check(tuple(y.shape) == (*x.shape[:-1], n), "y must have x's leading shape and blocks.size(0) columns")
    if rows == 0 or n == 0:
        return y
    lib = _lib()
    with _on_device(x.device):
        ws_bytes = lib.pllm_gguf_quant_gemm_workspace_bytes(type_id, rows, row_elems, n, blocks.size(1))
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_quant_gemm_accumulate(x.data_ptr(), _DTYPE_CODE[x.dtype], blocks.data_ptr(), type_id, y.data_ptr(),
                                                 _DTYPE_CODE[y.dtype], rows, row_elems, n, blocks.size(1), ws.data_ptr(), ws_bytes,
                                                 _stream(x.device))
    if st == _ffi.PLLM_ERR_UNSUPPORTED:      # a row count of the tile kernel
        prod = _dense_gemm("gguf_quant_gemm_accumulate_forward", x, blocks, row_elems, type_id, signed_grid, torch.float32)
        y.copy_((y.float() + prod).to(y.dtype))
        return y
    _ffi.check(st, "gguf_quant_gemm_accumulate_forward")
    return y


def gguf_quant_gemm_prefill_forward(x, blocks, row_elems, type_id, signed_grid, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """Prefill-regime operator, src/csrc/cuda_kernel.cpp:591-614."""
    return _dense_gemm("gguf_quant_gemm_prefill_forward", x, blocks, row_elems, type_id, signed_grid, out_dtype)


def fused_rms_norm_forward(x: torch.Tensor, weight: torch.Tensor, eps: float, *, out_dtype: torch.dtype = torch.float16) -> torch.Tensor:
    """src/csrc/cuda_kernel_impl.cu:9699-9730: fp16 [batch, dim] = x * rsqrt(mean(x^2) + eps) * weight."""
    _check(x.dim() == 2, "fused_rms_norm: x must be 2D [batch, dim]")
    _check(weight.dim() == 1, "fused_rms_norm: weight must be 1D [dim]")
    _check(weight.dtype == torch.float32, "fused_rms_norm: weight must be fp32")
    _check(weight.size(0) == x.size(1), "fused_rms_norm: weight.size(0) must == dim")
    _check(x.is_cuda and weight.is_cuda, "fused_rms_norm: tensors must be CUDA tensors")
    _check_x(x)
    x, weight = x.contiguous(), weight.contiguous()
    y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    if x.numel() == 0:
        return y
    with _on_device(x.device):
        st = _lib().pllm_fused_rms_norm(x.data_ptr(), _DTYPE_CODE[x.dtype], weight.data_ptr(), y.data_ptr(), _DTYPE_CODE[out_dtype],
                                        x.size(0), x.size(1), float(eps), _stream(x.device))
    _ffi.check(st, "fused_rms_norm_forward")
    return y


def attention_decode_forward(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, pos: int, *,
                             q_norm_weight: torch.Tensor | None = None, k_norm_weight: torch.Tensor | None = None, eps: float = 1e-6,
                             cos_row: torch.Tensor | None = None, sin_row: torch.Tensor | None = None, rope_dim: int = 0) -> torch.Tensor:
    """One decode step of grouped-query attention (the framework operators of src/models/minimax_m2/architecture.py:158-266 for
    one query position): q [batch, heads * head_dim], k_new / v_new [batch, kv_heads * head_dim]; keys / values
    [>= batch, kv_heads, capacity, head_dim] are the stores, whose position `pos` this call writes.  RMS normalisation of q and k
    over their whole width when weights are given, rotary phases from the float32 rows cos_row / sin_row (head_dim values each
    for this position).  Returns [batch, heads * head_dim] in q's dtype."""
    _check(q.dim() == 2 and k_new.dim() == 2 and v_new.dim() == 2, "attention_decode: q, k_new, v_new must be 2D [batch, width]")
    _check(keys.dim() == 4 and values.shape == keys.shape, "attention_decode: stores must be [batch, kv_heads, capacity, head_dim]")
    _check(q.dtype in (torch.float16, torch.bfloat16), "attention_decode: float16 or bfloat16 only")
    _check(all(t.dtype == q.dtype for t in (k_new, v_new, keys, values)), "attention_decode: one dtype for q, k, v and the stores")
    _check(all(t.is_cuda for t in (q, k_new, v_new, keys, values)), "attention_decode: tensors must be CUDA tensors")
    batch, kv_heads, capacity, head_dim = q.size(0), keys.size(1), keys.size(2), keys.size(3)
    pos = int(pos)
    _check(0 <= pos < capacity and keys.size(0) >= batch, "attention_decode: position or batch outside the stores")
    _check(q.size(1) % head_dim == 0 and k_new.shape == (batch, kv_heads * head_dim) and v_new.shape == k_new.shape,
           "attention_decode: widths do not match the stores")
    heads = q.size(1) // head_dim
    _check(keys.stride(3) == 1 and keys.stride(2) == head_dim and values.stride() == keys.stride(), "attention_decode: stores must be dense per head")
    for w, width in ((q_norm_weight, heads * head_dim), (k_norm_weight, kv_heads * head_dim)):
        _check(w is None or (w.is_cuda and w.dtype == torch.float32 and w.is_contiguous() and w.numel() == width), "attention_decode: norm weights must be fp32 [width]")
    if rope_dim:
        for r in (cos_row, sin_row):
            _check(r is not None and r.is_cuda and r.dtype == torch.float32 and r.is_contiguous() and r.numel() == head_dim,
                   "attention_decode: cos_row / sin_row must be fp32 [head_dim]")
    q, k_new, v_new = q.contiguous(), k_new.contiguous(), v_new.contiguous()
    out = torch.empty_like(q)
    lib = _lib()
    need = lib.pllm_attention_decode_workspace_bytes(batch, heads, pos)
    ws = _workspace(need, q.device)
    with _on_device(q.device):
        st = lib.pllm_attention_decode(q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), _DTYPE_CODE[q.dtype],
                                       None if q_norm_weight is None else q_norm_weight.data_ptr(),
                                       None if k_norm_weight is None else k_norm_weight.data_ptr(), float(eps),
                                       None if not rope_dim else cos_row.data_ptr(), None if not rope_dim else sin_row.data_ptr(), int(rope_dim),
                                       keys.data_ptr(), values.data_ptr(), keys.stride(0), keys.stride(1), batch, heads, kv_heads, head_dim, pos,
                                       out.data_ptr(), ws.data_ptr(), need, _stream(q.device))
    _ffi.check(st, "attention_decode_forward")
    return out


def gguf_quant_gemm_rmsnorm_forward(x, norm_weight, eps, blocks, row_elems, type_id, signed_grid, *, round_fp16: bool = True,
                                    out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """gguf_quant_gemm_forward(fused_rms_norm_forward(x, norm_weight, eps), ...) as one operator (decode: one launch).
    round_fp16=True rounds the normalized activations through fp16 like the two-operator chain, False keeps them in float32."""
    row_elems, type_id = int(row_elems), int(type_id)
    _dense_checks(x, blocks, row_elems, type_id, signed_grid)
    _check(norm_weight.dim() == 1 and norm_weight.size(0) == row_elems, "fused_rms_norm: weight.size(0) must == dim")
    _check(norm_weight.is_cuda and norm_weight.dtype == torch.float32 and norm_weight.is_contiguous(), "fused_rms_norm: weight must be fp32")
    rows = x.numel() // row_elems
    n = blocks.size(0)
    y = torch.empty(*x.shape[:-1], n, dtype=out_dtype, device=x.device)
    if rows == 0 or n == 0:
        return y
    lib = _lib()
    with _on_device(x.device):
        ws_bytes = lib.pllm_gguf_quant_gemm_rmsnorm_workspace_bytes(type_id, rows, row_elems, n, blocks.size(1))
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_quant_gemm_rmsnorm(x.data_ptr(), _DTYPE_CODE[x.dtype], norm_weight.data_ptr(), float(eps), int(bool(round_fp16)),
                                              blocks.data_ptr(), type_id, y.data_ptr(), _DTYPE_CODE[out_dtype], rows, row_elems, n,
                                              blocks.size(1), ws.data_ptr(), ws_bytes, _stream(x.device))
    _ffi.check(st, "gguf_quant_gemm_rmsnorm_forward")
    return y


def gguf_q2k_gemm_dp4a_forward(x, blocks, row_elems, *, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """src/csrc/cuda_kernel.cpp:545-564."""
    _check(blocks.dim() == 3, "blocks must have shape [N, K_blocks, 84]")
    _check(blocks.size(2) == 84, "q2_k block size must be 84 bytes")
    empty = torch.empty(0, dtype=torch.int8, device=x.device)
    return _dense_gemm("gguf_q2k_gemm_dp4a_forward", x, blocks, row_elems, 1, empty, out_dtype)


def gguf_dequantize_rows(blocks: torch.Tensor, type_id: int, row_elems: int, row_ids: torch.Tensor | None = None, *,
                         out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Dequantize whole or selected rows of a raw-block matrix (type_id _ffi.TYPE_Q8_0 for Q8_0 blocks, _ffi.TYPE_Q3_K for Q3_K).

    No direct counterpart in the reference extension: it is the device form of the numpy decoders of
    src/loader/gguf/tensor_reader.py:543-1009, with bit-identical float32 results.
    """
    type_id, row_elems = int(type_id), int(row_elems)
    q8, q3 = type_id == _ffi.TYPE_Q8_0, type_id == _ffi.TYPE_Q3_K
    if not (q8 or q3):
        _check_type(type_id)
    _check(blocks.dim() == 3 and blocks.is_cuda and blocks.dtype == torch.uint8 and blocks.is_contiguous(),
           "blocks must be a contiguous CUDA uint8 tensor [N, K_blocks, block_bytes]")
    _check(blocks.size(2) == (34 if q8 else 110 if q3 else GGUF_BLOCK_BYTES[type_id]), "unexpected GGUF block size for type_id")
    _check(row_elems > 0 and blocks.size(1) * (32 if q8 else 256) >= row_elems, "blocks do not cover row_elems")
    if row_ids is not None:
        _check(row_ids.is_cuda and row_ids.dtype == torch.int64 and row_ids.is_contiguous(), "row_ids must be contiguous CUDA int64")
        lead, count = tuple(row_ids.shape), row_ids.numel()
    else:
        lead, count = (blocks.size(0),), blocks.size(0)
    out = torch.empty(*lead, row_elems, dtype=out_dtype, device=blocks.device)
    if count == 0:
        return out
    with _on_device(blocks.device):
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
    with _on_device(w8.device):
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
    with _on_device(x.device):
        ws_bytes = _lib().pllm_fp8_block_gemm_workspace_bytes(rows, k, n)
        ws = _workspace(ws_bytes, x.device) if ws_bytes else None
        st = _lib().pllm_fp8_block_gemm(x.data_ptr(), _DTYPE_CODE[x.dtype], w8.data_ptr(), scale.data_ptr(), y.data_ptr(),
                                        _DTYPE_CODE[out_dtype], rows, k, n, ws.data_ptr() if ws is not None else None, ws_bytes,
                                        _stream(x.device))
    _ffi.check(st, "fp8_block_gemm_forward")
    return y


def fp8_block_gemm_accumulate_forward(x: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """y += fp8_block_gemm_forward(x, weight, scale) in place (a block's residual connection folded into the projection): one
    launch for decode calls; row counts of the tile kernel run it and add separately."""
    w8 = _fp8_bytes(weight)
    n, k = w8.shape
    _check(x.is_cuda and x.is_contiguous() and x.size(-1) == k, "x must be a contiguous CUDA tensor [..., K]")
    _check_x(x)
    _check(scale.is_cuda and scale.dtype == torch.float32 and scale.is_contiguous(), "scale must be a contiguous CUDA float32 tensor")
    _check(tuple(scale.shape) == ((n + 127) // 128, (k + 127) // 128), "scale must have shape [ceil(N/128), ceil(K/128)]")
    _check(y.is_cuda and y.device == x.device and y.is_contiguous() and y.dtype in _DTYPE_CODE, "y must be a contiguous CUDA tensor of float16, bfloat16 or float32")
    _check(tuple(y.shape) == (*x.shape[:-1], n), "y must have x's leading shape and weight.size(0) columns")
    rows = x.numel() // k
    if rows == 0:
        return y
    with _on_device(x.device):
        st = _lib().pllm_fp8_block_gemm_accumulate(x.data_ptr(), _DTYPE_CODE[x.dtype], w8.data_ptr(), scale.data_ptr(), y.data_ptr(),
                                                   _DTYPE_CODE[y.dtype], rows, k, n, _stream(x.device))
    if st == _ffi.PLLM_ERR_UNSUPPORTED:      # a row count of the tile kernel
        y.copy_((y.float() + fp8_block_gemm_forward(x, weight, scale, out_dtype=torch.float32)).to(y.dtype))
        return y
    _ffi.check(st, "fp8_block_gemm_accumulate_forward")
    return y


def fp8_gemm_forward(a: torch.Tensor, a_scale: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, *,
                     out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """fp8_gemm(a, a_s, b, b_s) of src/kernels/ops.py:1043-1051 on the native FP8 matrix path: `a` / `a_scale` are the
    codes and 128-wide scales of fp8_act_quant_forward, `weight` / `scale` the block-scaled FP8 weight."""
    _check(a.dtype in (torch.float8_e4m3fn, torch.uint8), "a must be float8_e4m3fn (or its uint8 bytes)")
    a8 = a.view(torch.uint8) if a.dtype == torch.float8_e4m3fn else a
    w8 = _fp8_bytes(weight)
    n, k = w8.shape
    _check(a8.is_cuda and a8.is_contiguous() and a8.dim() >= 1 and a8.size(-1) == k, "a must be a contiguous CUDA FP8 tensor [..., K]")
    _check(k % 128 == 0, "fp8_gemm needs K to be a multiple of 128")
    rows = a8.numel() // k
    _check(a_scale.is_cuda and a_scale.dtype == torch.float32 and a_scale.is_contiguous() and a_scale.numel() == rows * (k // 128),
           "a_scale must be a contiguous CUDA float32 tensor [..., K/128]")
    _check(scale.is_cuda and scale.dtype == torch.float32 and scale.is_contiguous(), "scale must be a contiguous CUDA float32 tensor")
    _check(tuple(scale.shape) == ((n + 127) // 128, k // 128), "scale must have shape [ceil(N/128), K/128]")
    y = torch.empty(*a8.shape[:-1], n, dtype=out_dtype, device=a8.device)
    if rows == 0:
        return y
    with _on_device(a8.device):
        need = int(_lib().pllm_fp8_gemm_workspace_bytes(rows, k, n))
        ws = torch.empty(need, dtype=torch.uint8, device=a8.device) if need else None
        st = _lib().pllm_fp8_gemm_ws(a8.data_ptr(), a_scale.data_ptr(), w8.data_ptr(), scale.data_ptr(), y.data_ptr(), _DTYPE_CODE[out_dtype],
                                     rows, k, n, ws.data_ptr() if ws is not None else None, need, _stream(a8.device))
    _ffi.check(st, "fp8_gemm_forward")
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
        with _on_device(x.device):
            st = _lib().pllm_fp8_act_quant(x.data_ptr(), _DTYPE_CODE[x.dtype], rows, k, codes.data_ptr(), scales.data_ptr(),
                                           float(eps), int(bool(round_scale_pow2)), _stream(x.device))
        _ffi.check(st, "fp8_act_quant_forward")
    return codes.view(torch.float8_e4m3fn), scales


def gguf_quant_gemm_pair_forward(x, blocks0, row_elems0, type_id0, blocks1, row_elems1, type_id1, signed_grid, *,
                                 out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """src/csrc/cuda_kernel.cpp:615-666: returns the stack [2, ..., N]."""
    row_elems0, row_elems1, type_id0, type_id1 = int(row_elems0), int(row_elems1), int(type_id0), int(type_id1)
    _check(x.dim() in (2, 3), "x must have shape [M, K] or [B, S, K]")
    _check(blocks0.dim() == 3 and blocks1.dim() == 3, "blocks must have shape [N, K_blocks, block_bytes]")
    _check_type(type_id0, "type_id0")
    _check_type(type_id1, "type_id1")
    uses_iq2 = type_id0 == 0 or type_id1 == 0
    uses_iq1 = type_id0 == 2 or type_id1 == 2
    uses_xs = type_id0 in (5, 6) or type_id1 in (5, 6)
    _check(not (uses_iq2 and uses_iq1), "paired GEMM cannot mix iq2_xxs and iq1_m because they require different grids")
    _check(not (uses_iq2 and uses_xs), "paired GEMM cannot mix iq2_xxs with iq2_xs/iq3_xxs because they require different grids")
    _check(not (uses_iq1 and uses_xs), "paired GEMM cannot mix iq1_m with iq2_xs/iq3_xxs because they require different grids")
    _check(row_elems0 > 0 and row_elems1 > 0, "row_elems must be positive")
    _check(row_elems0 == row_elems1, "paired GGUF GEMM requires matching input dimensions")
    _check(x.size(-1) == row_elems0, "inner dimension mismatch")
    _check(blocks0.size(0) == blocks1.size(0), "paired blocks must have same output rows")
    _check(blocks0.size(1) * 256 >= row_elems0 and blocks1.size(1) * 256 >= row_elems1, "blocks do not cover row_elems")
    _check(blocks0.size(2) == GGUF_BLOCK_BYTES[type_id0], "unexpected blocks0 GGUF block size")
    _check(blocks1.size(2) == GGUF_BLOCK_BYTES[type_id1], "unexpected blocks1 GGUF block size")
    _check(x.is_cuda and blocks0.is_cuda and blocks1.is_cuda, "x and blocks must be CUDA tensors")
    _check(x.is_contiguous() and blocks0.is_contiguous() and blocks1.is_contiguous(), "x and blocks must be contiguous")
    _check(blocks0.dtype == torch.uint8, "blocks0 has unexpected dtype")
    _check(blocks1.dtype == torch.uint8, "blocks1 has unexpected dtype")
    _check_x(x)
    _check(blocks0.size(1) == blocks1.size(1), "paired blocks must have the same number of blocks per row")
    if uses_iq2:
        _check_grid(signed_grid, 0, "signed_grid")
    elif uses_iq1:
        _check_grid(signed_grid, 2, "signed_grid")
    elif uses_xs:
        _check_grid(signed_grid, 5, "signed_grid")
    rows = x.numel() // row_elems0
    n = blocks0.size(0)
    y = torch.empty(2, *x.shape[:-1], n, dtype=out_dtype, device=x.device)
    if rows == 0 or n == 0:
        return y
    lib = _lib()
    with _on_device(x.device):
        ws_bytes = lib.pllm_activation_image_bytes(rows, blocks0.size(1))
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_quant_gemm_pair(x.data_ptr(), _DTYPE_CODE[x.dtype], blocks0.data_ptr(), type_id0, blocks1.data_ptr(), type_id1,
                                           y.data_ptr(), _DTYPE_CODE[out_dtype], rows, row_elems0, n, blocks0.size(1),
                                           ws.data_ptr(), ws_bytes, _stream(x.device))
    _ffi.check(st, "gguf_quant_gemm_pair_forward")
    return y


# ---- routed experts --------------------------------------------------------------------------------

_MOE_TYPES = IMPLEMENTED_TYPE_IDS   # iq2_xxs, q2_k, iq1_m have fused expert kernels; the other six run route by route or as tile matmuls

# codebook families: one grid tensor serves a family (src/csrc/cuda_kernel.cpp:717-722)
_GRID_FAMILY = {0: 0, 2: 2, 5: 5, 6: 5}
_FAMILY_NAME = {0: "iq2_xxs", 2: "iq1_m", 5: "iq2_xs/iq3_xxs"}


def _grids_ok(grid, type_ids, name: str) -> None:
    """The reference takes ONE grid tensor and refuses to mix codebook families (iq2_xxs, iq1_m, iq2_xs/iq3_xxs:
    src/csrc/cuda_kernel.cpp:717-722).  Passing a tuple/list of grids lifts that limit: one entry per family in use,
    in the order iq2_xxs, iq1_m, iq2_xs/iq3_xxs, each checked like the reference checks its single grid."""
    need = sorted({_GRID_FAMILY[t] for t in type_ids if t in _GRID_FAMILY})
    if isinstance(grid, (tuple, list)):
        _check(len(grid) >= len(need), f"{name}: one grid per codebook type in use is required")
        for g, t in zip(grid, need):
            _check_grid(g, t, name)
        return
    if len(need) > 1:
        a, b = _FAMILY_NAME[need[0]], _FAMILY_NAME[need[1]]
        joiner = "and" if (need[0], need[1]) == (0, 2) else "with"
        _check(False, f"grouped GGUF kernel cannot mix {a} {joiner} {b} because they require different grids")
    if need:
        _check_grid(grid, need[0], name)


def _moe_call(name, x, tokens, route_tokens, route_experts, seg_starts, route_weights, w1, w3, w2, w13_type, w2_type, swiglu_limit):
    dim, inter, n_experts, routes = x.size(-1), w1.size(1), w1.size(0), route_weights.numel()
    y = torch.empty(tokens, dim, dtype=torch.float32, device=x.device)
    lib = _lib()
    with _on_device(x.device):
        ws_bytes = lib.pllm_gguf_moe_workspace_bytes(tokens, routes, dim, inter)
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_moe_forward(
            x.data_ptr(), _DTYPE_CODE[x.dtype], tokens, dim, inter,
            None if route_tokens is None else route_tokens.data_ptr(),
            None if route_experts is None else route_experts.data_ptr(),
            None if seg_starts is None else seg_starts.data_ptr(), n_experts,
            route_weights.data_ptr(), routes, w1.data_ptr(), w3.data_ptr(), w13_type, w2.data_ptr(), w2_type,
            float(swiglu_limit), y.data_ptr(), ws.data_ptr(), ws_bytes, _stream(x.device))
    _ffi.check(st, name)
    return y


def gguf_moe_prefill_grouped_forward(x, route_tokens, route_weights_sorted, seg_starts, w1_blocks, w3_blocks, w2_blocks,
                                     w1_row_elems, w1_type_id, w3_row_elems, w3_type_id, w2_row_elems, w2_type_id,
                                     signed_grid, swiglu_limit) -> torch.Tensor:
    """src/csrc/cuda_kernel.cpp:689-767: float32 [T, D]."""
    w1_type_id, w3_type_id, w2_type_id = int(w1_type_id), int(w3_type_id), int(w2_type_id)
    _check(x.dim() == 2, "x must have shape [T, D]")
    _check(route_tokens.dim() == 1, "route_tokens must have shape [R]")
    _check(route_weights_sorted.dim() == 1, "route_weights_sorted must have shape [R]")
    _check(seg_starts.dim() == 1, "seg_starts must have shape [E + 1]")
    _check(w1_blocks.dim() == 4 and w3_blocks.dim() == 4 and w2_blocks.dim() == 4, "GGUF blocks must have shape [E, N, K_blocks, block_bytes]")
    _check(route_tokens.size(0) == route_weights_sorted.size(0), "route count mismatch")
    _check(seg_starts.size(0) == w1_blocks.size(0) + 1, "seg_starts/expert count mismatch")
    _check(w1_blocks.size(0) == w3_blocks.size(0) == w2_blocks.size(0), "expert count mismatch")
    _check(w1_blocks.size(2) * 256 >= w1_row_elems and w3_blocks.size(2) * 256 >= w3_row_elems and w2_blocks.size(2) * 256 >= w2_row_elems,
           "blocks do not cover row_elems")
    for t, nm in ((w1_type_id, "w1"), (w3_type_id, "w3"), (w2_type_id, "w2")):
        _check(t in GGUF_BLOCK_BYTES, f"unsupported {nm} GGUF type: {t}")
        _check(t in _MOE_TYPES, f"{nm} GGUF type {t} has no fused expert kernel in this build")
    _grids_ok(signed_grid, (w1_type_id, w3_type_id, w2_type_id), "signed_grid")
    _check(w1_type_id == w3_type_id, "w1 and w3 must share a GGUF type in this build")
    _check(w1_blocks.size(3) == GGUF_BLOCK_BYTES[w1_type_id], "unexpected w1 GGUF block size")
    _check(w3_blocks.size(3) == GGUF_BLOCK_BYTES[w3_type_id], "unexpected w3 GGUF block size")
    _check(w2_blocks.size(3) == GGUF_BLOCK_BYTES[w2_type_id], "unexpected w2 GGUF block size")
    _check(w1_row_elems == x.size(1) and w3_row_elems == x.size(1), "w1/w3 input dimension mismatch")
    _check(w2_row_elems == w1_blocks.size(1) and w1_blocks.size(1) == w3_blocks.size(1), "w2 input dimension mismatch")
    _check(w2_blocks.size(1) == x.size(1), "w2 output dimension mismatch")
    _check(x.is_cuda and route_tokens.is_cuda and route_weights_sorted.is_cuda and seg_starts.is_cuda, "route tensors must be CUDA tensors")
    _check(w1_blocks.is_cuda and w3_blocks.is_cuda and w2_blocks.is_cuda, "GGUF blocks must be CUDA tensors")
    _check(x.is_contiguous() and route_tokens.is_contiguous() and route_weights_sorted.is_contiguous() and seg_starts.is_contiguous(),
           "route tensors must be contiguous")
    _check(w1_blocks.is_contiguous() and w3_blocks.is_contiguous() and w2_blocks.is_contiguous(), "GGUF blocks must be contiguous")
    _check_x(x)
    _check(route_tokens.dtype == torch.int64, "route_tokens must be int64")
    _check(route_weights_sorted.dtype == torch.float32, "route_weights_sorted must be float32")
    _check(seg_starts.dtype in (torch.int32, torch.int64), "seg_starts must be int32 or int64")
    for b, nm in ((w1_blocks, "w1_blocks"), (w3_blocks, "w3_blocks"), (w2_blocks, "w2_blocks")):
        _check(b.dtype == torch.uint8, f"{nm} has unexpected dtype")
    seg32 = seg_starts if seg_starts.dtype == torch.int32 else seg_starts.to(torch.int32)
    return _moe_call("gguf_moe_prefill_grouped_forward", x, x.size(0), route_tokens, None, seg32, route_weights_sorted,
                     w1_blocks, w3_blocks, w2_blocks, w1_type_id, w2_type_id, swiglu_limit)


def _single_token_checks(x, route_slots, route_weights, w1, w3, w2):
    _check(x.dim() == 2 and x.size(0) == 1, "x must have shape [1, D]")
    _check(route_slots.dim() == 1, "route_slots must have shape [K]")
    _check(route_weights.dim() == 1, "route_weights must have shape [K]")
    _check(route_slots.size(0) == route_weights.size(0), "route_slots/route_weights length mismatch")
    _check(w1.dim() == 4 and w3.dim() == 4 and w2.dim() == 4, "GGUF blocks must have shape [E, N, K_blocks, block_bytes]")
    _check(w1.size(0) == w3.size(0) == w2.size(0), "expert count mismatch")
    _check(w1.size(1) == w3.size(1), "w1/w3 inter_dim mismatch")
    _check(w1.size(2) == w3.size(2), "w1/w3 block count mismatch")
    _check(w1.size(2) * 256 >= x.size(1), "w1/w3 blocks do not cover x dim")
    _check(w2.size(1) == x.size(1), "w2 output dimension mismatch")
    _check(w2.size(2) * 256 >= w1.size(1), "w2 blocks do not cover inter dim")
    _check(x.is_cuda and route_slots.is_cuda and route_weights.is_cuda, "x/route tensors must be CUDA tensors")
    _check(w1.is_cuda and w3.is_cuda and w2.is_cuda, "GGUF blocks must be CUDA tensors")
    _check(x.is_contiguous() and route_slots.is_contiguous() and route_weights.is_contiguous(), "x/route tensors must be contiguous")
    _check(w1.is_contiguous() and w3.is_contiguous() and w2.is_contiguous(), "GGUF blocks must be contiguous")
    _check_x(x)
    _check(route_slots.dtype == torch.int64, "route_slots must be int64")
    _check(route_weights.dtype == torch.float32, "route_weights must be float32")
    for b, nm in ((w1, "w1_blocks"), (w3, "w3_blocks"), (w2, "w2_blocks")):
        _check(b.dtype == torch.uint8, f"{nm} has unexpected dtype")


_TYPE_OF_BLOCK_BYTES = {GGUF_BLOCK_BYTES[t]: t for t in IMPLEMENTED_TYPE_IDS}   # the nine block sizes are distinct


def gguf_moe_single_token_forward(x, route_slots, route_weights, w1_blocks, w3_blocks, w2_blocks, swiglu_limit) -> torch.Tensor:
    """Single-token routed experts for any mix of IQ2_XXS / Q2_K / IQ1_M matrices (types read off the
    block sizes): the case the reference cannot express because its operators take one grid tensor."""
    _single_token_checks(x, route_slots, route_weights, w1_blocks, w3_blocks, w2_blocks)
    _check(w1_blocks.size(3) == w3_blocks.size(3) and w1_blocks.size(3) in _TYPE_OF_BLOCK_BYTES, "w1/w3 must be blocks of one supported GGUF type")
    _check(w2_blocks.size(3) in _TYPE_OF_BLOCK_BYTES, "w2 must be blocks of a supported GGUF type")
    return _moe_call("gguf_moe_single_token_forward", x, 1, None, route_slots, None, route_weights, w1_blocks, w3_blocks, w2_blocks,
                     _TYPE_OF_BLOCK_BYTES[w1_blocks.size(3)], _TYPE_OF_BLOCK_BYTES[w2_blocks.size(3)], swiglu_limit)


def gguf_moe_single_token_accumulate_forward(x, route_slots, route_weights, w1_blocks, w3_blocks, w2_blocks, swiglu_limit, y: torch.Tensor) -> bool:
    """y [1, D] (float16, bfloat16 or float32) += the routed experts of the one token x, inside the down projection's launch
    (no counterpart in the reference, whose block converts and adds afterwards: src/models/minimax_m2/architecture.py:404-413).
    Returns False, with y untouched, when the shape or the type pair has no such kernel: take gguf_moe_single_token_forward and add."""
    _single_token_checks(x, route_slots, route_weights, w1_blocks, w3_blocks, w2_blocks)
    _check(w1_blocks.size(3) == w3_blocks.size(3) and w1_blocks.size(3) in _TYPE_OF_BLOCK_BYTES, "w1/w3 must be blocks of one supported GGUF type")
    _check(w2_blocks.size(3) in _TYPE_OF_BLOCK_BYTES, "w2 must be blocks of a supported GGUF type")
    _check(y.is_cuda and y.is_contiguous() and y.numel() == x.size(-1) and y.dtype in _DTYPE_CODE, "y must be a contiguous CUDA tensor of D values (float16, bfloat16 or float32)")
    dim, inter, routes = x.size(-1), w1_blocks.size(1), route_weights.numel()
    lib = _lib()
    with _on_device(x.device):
        ws_bytes = lib.pllm_gguf_moe_workspace_bytes(1, routes, dim, inter)
        ws = _workspace(ws_bytes, x.device)
        st = lib.pllm_gguf_moe_single_token_accumulate(
            x.data_ptr(), _DTYPE_CODE[x.dtype], dim, inter, route_slots.data_ptr(), route_weights.data_ptr(), routes,
            w1_blocks.data_ptr(), w3_blocks.data_ptr(), _TYPE_OF_BLOCK_BYTES[w1_blocks.size(3)], w2_blocks.data_ptr(),
            _TYPE_OF_BLOCK_BYTES[w2_blocks.size(3)], float(swiglu_limit), y.data_ptr(), _DTYPE_CODE[y.dtype], ws.data_ptr(), ws_bytes, _stream(x.device))
    if st == _ffi.PLLM_ERR_UNSUPPORTED:
        return False
    _ffi.check(st, "gguf_moe_single_token_accumulate_forward")
    return True


def gguf_moe_single_token_iq2_q2k_forward(x, route_slots, route_weights, w1_blocks, w3_blocks, w2_blocks, signed_grid, swiglu_limit) -> torch.Tensor:
    """src/csrc/cuda_kernel.cpp:769-818: float32 [1, D]."""
    _single_token_checks(x, route_slots, route_weights, w1_blocks, w3_blocks, w2_blocks)
    _check(w1_blocks.size(3) == 66 and w3_blocks.size(3) == 66, "w1/w3 must be IQ2_XXS blocks")
    _check(w2_blocks.size(3) in (66, 84), "w2 must be IQ2_XXS or Q2_K blocks")
    _check(signed_grid.is_cuda, "signed_grid must be CUDA for IQ2_XXS")
    _check(signed_grid.is_contiguous(), "signed_grid must be contiguous")
    _check(signed_grid.dtype == torch.int8, "signed_grid has unexpected dtype")
    _check(signed_grid.numel() == 256 * 128 * 8, "signed_grid must contain 256*128*8 entries")
    return _moe_call("gguf_moe_single_token_iq2_q2k_forward", x, 1, None, route_slots, None, route_weights, w1_blocks, w3_blocks, w2_blocks,
                     0, _TYPE_OF_BLOCK_BYTES[w2_blocks.size(3)], swiglu_limit)


def gguf_moe_single_token_iq1m_forward(x, route_slots, route_weights, w1_blocks, w3_blocks, w2_blocks, iq1_grid, swiglu_limit) -> torch.Tensor:
    """src/csrc/cuda_kernel.cpp:820-865: float32 [1, D]."""
    _single_token_checks(x, route_slots, route_weights, w1_blocks, w3_blocks, w2_blocks)
    _check(w1_blocks.size(3) == 56 and w3_blocks.size(3) == 56 and w2_blocks.size(3) == 56, "w1/w3/w2 must be IQ1_M blocks")
    _check_grid(iq1_grid, 2, "iq1_grid")
    return _moe_call("gguf_moe_single_token_iq1m_forward", x, 1, None, route_slots, None, route_weights, w1_blocks, w3_blocks, w2_blocks,
                     2, 2, swiglu_limit)


def moe_group_routes(indices, weights, experts_start_idx, n_local_experts):
    """src/csrc/cuda_kernel.cpp:1228-1242: [local_ids int64, route_tokens int64 [R], route_weights float32 [R], seg_starts int32 [E+1]].
    Like the reference it reads the route count back to size the outputs (one host sync)."""
    _check(indices.dim() == 2, "indices must have shape [T, K]")
    _check(weights.dim() == 2, "weights must have shape [T, K]")
    _check(indices.shape == weights.shape, "indices/weights shape mismatch")
    _check(indices.is_cuda and weights.is_cuda, "indices and weights must be CUDA tensors")
    _check(indices.is_contiguous() and weights.is_contiguous(), "indices and weights must be contiguous")
    _check(weights.dtype == torch.float32, "weights must be float32")
    _check(indices.dtype in (torch.int64, torch.int32), "indices must be int64 or int32")
    n_local = int(n_local_experts)
    _check(n_local > 0, "n_local_experts must be positive")
    t, k = indices.shape
    dev = indices.device
    seg = torch.empty(n_local + 1, dtype=torch.int32, device=dev)
    cap = max(t * k, 1)
    toks = torch.empty(cap, dtype=torch.int64, device=dev)
    wts = torch.empty(cap, dtype=torch.float32, device=dev)
    exps = torch.empty(cap, dtype=torch.int32, device=dev)
    if t * k:
        with _on_device(dev):
            st = _lib().pllm_moe_group_routes(indices.data_ptr(), int(indices.dtype == torch.int64), weights.data_ptr(), t, k,
                                              int(experts_start_idx), n_local, seg.data_ptr(), toks.data_ptr(), wts.data_ptr(),
                                              exps.data_ptr(), _stream(dev))
        _ffi.check(st, "moe_group_routes")
    else:
        seg.zero_()
    routes = int(seg[-1].item())
    local_ids = (seg[1:] > seg[:-1]).nonzero().flatten().to(torch.long)
    return [local_ids, toks[:routes], wts[:routes], seg]


def moe_route(x_flat: torch.Tensor, gate_weight: torch.Tensor, gate_bias, top_k: int, *, softmax: bool = False):
    """MiniMaxMoE.route (src/models/minimax_m2/architecture.py:291-298) in two launches: (indices int64 [T, top_k],
    weights float32 [T, top_k]) from x_flat [T, dim], gate_weight float32 [E, dim] and an optional gate_bias [E].
    softmax=True picks the top_k logits and returns their softmax instead (the renormalised softmax routing)."""
    _check(x_flat.dim() == 2 and gate_weight.dim() == 2 and x_flat.size(1) == gate_weight.size(1), "x_flat [T, dim] and gate_weight [E, dim] must agree on dim")
    _check(x_flat.is_cuda and gate_weight.is_cuda and x_flat.is_contiguous() and gate_weight.is_contiguous(), "x_flat and gate_weight must be contiguous CUDA tensors")
    _check_x(x_flat)
    _check(gate_weight.dtype == torch.float32, "gate_weight must be float32")
    if gate_bias is not None:
        _check(gate_bias.is_cuda and gate_bias.dtype == torch.float32 and gate_bias.is_contiguous() and gate_bias.numel() == gate_weight.size(0),
               "gate_bias must be a contiguous CUDA float32 tensor [E]")
    t, e, k = x_flat.size(0), gate_weight.size(0), int(top_k)
    _check(0 < k <= e, "top_k must be in 1..E")
    dev = x_flat.device
    indices = torch.empty(t, k, dtype=torch.int64, device=dev)
    weights = torch.empty(t, k, dtype=torch.float32, device=dev)
    if t == 0:
        return indices, weights
    logits = torch.empty(t, e, dtype=torch.float32, device=dev)
    with _on_device(dev):
        st = _lib().pllm_moe_route(x_flat.data_ptr(), _DTYPE_CODE[x_flat.dtype], t, x_flat.size(1), gate_weight.data_ptr(),
                                   gate_bias.data_ptr() if gate_bias is not None else None, e, k, int(bool(softmax)),
                                   logits.data_ptr(), indices.data_ptr(), weights.data_ptr(), _stream(dev))
    _ffi.check(st, "moe_route")
    return indices, weights


def moe_route_rmsnorm(x_flat: torch.Tensor, norm_weight: torch.Tensor, eps: float, gate_weight: torch.Tensor, gate_bias, top_k: int, *,
                      out_dtype: torch.dtype = torch.float16, softmax: bool = False):
    """RMS normalisation of the decode rows x_flat [T <= 4, dim] and moe_route on the result (the decoder block's ffn_norm and
    MiniMaxMoE.route, src/models/minimax_m2/architecture.py:291-298, 405-412) in two launches instead of three:
    (indices, weights, normalized rows in out_dtype), or None where the library has no such launch (the caller then runs the two
    operators)."""
    _check(x_flat.dim() == 2 and gate_weight.dim() == 2 and x_flat.size(1) == gate_weight.size(1), "x_flat [T, dim] and gate_weight [E, dim] must agree on dim")
    _check(x_flat.is_cuda and gate_weight.is_cuda and x_flat.is_contiguous() and gate_weight.is_contiguous(), "x_flat and gate_weight must be contiguous CUDA tensors")
    _check_x(x_flat)
    _check(gate_weight.dtype == torch.float32, "gate_weight must be float32")
    _check(norm_weight.is_cuda and norm_weight.dtype == torch.float32 and norm_weight.is_contiguous() and norm_weight.numel() == x_flat.size(1),
           "norm_weight must be a contiguous CUDA float32 tensor [dim]")
    _check(out_dtype in _DTYPE_CODE, "out_dtype must be float32, float16 or bfloat16")
    if gate_bias is not None:
        _check(gate_bias.is_cuda and gate_bias.dtype == torch.float32 and gate_bias.is_contiguous() and gate_bias.numel() == gate_weight.size(0),
               "gate_bias must be a contiguous CUDA float32 tensor [E]")
    t, e, k = x_flat.size(0), gate_weight.size(0), int(top_k)
    _check(0 < k <= e, "top_k must be in 1..E")
    if t == 0 or t > 4:
        return None
    dev = x_flat.device
    indices = torch.empty(t, k, dtype=torch.int64, device=dev)
    weights = torch.empty(t, k, dtype=torch.float32, device=dev)
    logits = torch.empty(t, e, dtype=torch.float32, device=dev)
    normed = torch.empty(t, x_flat.size(1), dtype=out_dtype, device=dev)
    with _on_device(dev):
        st = _lib().pllm_moe_route_rmsnorm(x_flat.data_ptr(), _DTYPE_CODE[x_flat.dtype], norm_weight.data_ptr(), float(eps), normed.data_ptr(),
                                           _DTYPE_CODE[out_dtype], t, x_flat.size(1), gate_weight.data_ptr(),
                                           gate_bias.data_ptr() if gate_bias is not None else None, e, k, int(bool(softmax)),
                                           logits.data_ptr(), indices.data_ptr(), weights.data_ptr(), _stream(dev))
    if st == _ffi.PLLM_ERR_UNSUPPORTED:
        return None
    _ffi.check(st, "moe_route_rmsnorm")
    return indices, weights, normed


def gguf_single_token_route_slots(indices, weights, experts_start_idx, n_local_experts):
    """Host-side compaction of one token's routes (src/csrc/cuda_kernel.cpp:1244-1327):
    [local_ids (CPU int64), route_tokens, route_weights, route_slots, compact_starts (int32)]."""
    _check(indices.dim() == 2 and indices.size(0) == 1, "indices must have shape [1, K]")
    _check(weights.dim() == 2 and weights.size(0) == 1, "weights must have shape [1, K]")
    _check(indices.size(1) == weights.size(1), "indices/weights shape mismatch")
    _check(indices.is_cuda and weights.is_cuda, "indices and weights must be CUDA tensors")
    _check(indices.is_contiguous() and weights.is_contiguous(), "indices and weights must be contiguous")
    _check(weights.dtype == torch.float32, "weights must be float32")
    _check(indices.dtype in (torch.int64, torch.int32), "indices must be int64 or int32")
    _check(int(n_local_experts) > 0, "n_local_experts must be positive")
    by_local: dict[int, list[int]] = {}
    for pos, ex in enumerate(indices.view(-1).tolist()):
        local = int(ex) - int(experts_start_idx)
        if 0 <= local < int(n_local_experts):
            by_local.setdefault(local, []).append(pos)
    local_ids, slots, positions, starts = [], [], [], [0]
    for slot, local in enumerate(sorted(by_local)):
        local_ids.append(local)
        for pos in by_local[local]:
            slots.append(slot)
            positions.append(pos)
        starts.append(len(slots))
    dev = indices.device
    route_positions = torch.tensor(positions, dtype=torch.int64, device=dev)
    return [torch.tensor(local_ids, dtype=torch.int64), torch.zeros(len(slots), dtype=torch.int64, device=dev),
            weights.view(-1).index_select(0, route_positions), torch.tensor(slots, dtype=torch.int64, device=dev),
            torch.tensor(starts, dtype=torch.int32, device=dev)]


def quantize_activations(x: torch.Tensor, blocks_per_row: int) -> torch.Tensor:
    """Pre-quantize activations [..., K] for the super-block matmuls: returns the opaque uint8 image
    (one row per activation row) that gguf_quant_gemm_prequantized reads."""
    _check(x.is_cuda and x.is_contiguous(), "x must be a contiguous CUDA tensor")
    _check_x(x)
    k, bpr = x.size(-1), int(blocks_per_row)
    _check(bpr * 256 >= k, "blocks do not cover row_elems")
    rows = x.numel() // k
    lib = _lib()
    nbytes = lib.pllm_activation_image_bytes(rows, bpr)
    image = torch.empty(rows, nbytes // max(rows, 1), dtype=torch.uint8, device=x.device)
    with _on_device(x.device):
        st = lib.pllm_quantize_activations(x.data_ptr(), _DTYPE_CODE[x.dtype], rows, k, bpr, image.data_ptr(), nbytes, _stream(x.device))
    _ffi.check(st, "quantize_activations")
    return image


def swiglu_quantize_activations(gate: torch.Tensor, up: torch.Tensor, blocks_per_row: int, *, swiglu_limit: float = 0.0,
                                round_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """The activation image of SiLU(gate) * up for the down projection (gguf_quant_gemm_prequantized), one launch in place of the
    activation, the multiplication and the quantization pre-pass.  swiglu_limit > 0 caps gate and clamps up as the fused expert
    operators do (src/csrc/cuda_kernel_impl.cu:241-262); round_dtype float16 / bfloat16 rounds the product through that type
    first, as a chain that forms it in the model's dtype does."""
    _check(gate.is_cuda and up.is_cuda and gate.is_contiguous() and up.is_contiguous(), "gate and up must be contiguous CUDA tensors")
    _check(gate.shape == up.shape and gate.dtype == up.dtype, "gate and up must agree in shape and dtype")
    _check_x(gate)
    _check(round_dtype in _DTYPE_CODE, "round_dtype must be float16, bfloat16, or float32")
    k, bpr = gate.size(-1), int(blocks_per_row)
    _check(bpr * 256 >= k, "blocks do not cover row_elems")
    rows = gate.numel() // max(k, 1)
    _check(rows > 0 and k > 0, "gate and up must not be empty")
    lib = _lib()
    nbytes = lib.pllm_activation_image_bytes(rows, bpr)
    image = torch.empty(rows, nbytes // rows, dtype=torch.uint8, device=gate.device)
    with _on_device(gate.device):
        st = lib.pllm_swiglu_quantize_activations(gate.data_ptr(), up.data_ptr(), _DTYPE_CODE[gate.dtype], rows, k, bpr, float(swiglu_limit),
                                                  _DTYPE_CODE[round_dtype], image.data_ptr(), nbytes, _stream(gate.device))
    _ffi.check(st, "swiglu_quantize_activations")
    return image


def gguf_quant_gemm_prequantized(image: torch.Tensor, blocks: torch.Tensor, type_id: int, *, out_dtype: torch.dtype = torch.bfloat16,
                                 accumulate_into: torch.Tensor = None) -> torch.Tensor:
    """y [rows, N] from an activation image and raw super-blocks [N, K_blocks, block_bytes]; with accumulate_into the product is
    added to that tensor in place (the residual connection) and it is returned."""
    type_id = int(type_id)
    _check_type(type_id)
    _check(image.is_cuda and image.dtype == torch.uint8 and image.dim() == 2 and image.is_contiguous(), "image must come from quantize_activations")
    _check(blocks.dim() == 3 and blocks.is_cuda and blocks.dtype == torch.uint8 and blocks.is_contiguous(),
           "blocks must be a contiguous CUDA uint8 tensor [N, K_blocks, block_bytes]")
    _check(blocks.size(2) == GGUF_BLOCK_BYTES[type_id], "unexpected GGUF block size for type_id")
    lib = _lib()
    rows, n = image.size(0), blocks.size(0)
    _check(image.size(1) * rows == lib.pllm_activation_image_bytes(rows, blocks.size(1)), "image does not match blocks_per_row")
    if accumulate_into is not None:
        y = accumulate_into
        _check(y.is_cuda and y.device == image.device and y.is_contiguous() and y.dtype in _DTYPE_CODE and y.numel() == rows * n and y.size(-1) == n,
               "accumulate_into must be a contiguous CUDA tensor [rows, N] of float16, bfloat16 or float32")
        fn = lib.pllm_gguf_quant_gemm_prequantized_accumulate
    else:
        y = torch.empty(rows, n, dtype=out_dtype, device=image.device)
        fn = lib.pllm_gguf_quant_gemm_prequantized
    with _on_device(image.device):
        st = fn(image.data_ptr(), blocks.data_ptr(), type_id, y.data_ptr(), _DTYPE_CODE[y.dtype], rows, n, blocks.size(1), _stream(image.device))
    _ffi.check(st, "gguf_quant_gemm_prequantized")
    return y
