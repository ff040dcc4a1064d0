"""Quantized-op layer: the Q8_0 and FP8 functions of the reference's src/kernels/ops.py, over HIP kernels.

Same names, arguments and result dtypes as the reference functions cited below.  Differences, all on
purpose: every function runs the native HIP library and raises RuntimeError when it is missing or
when its tensors are not on the GPU (the reference silently falls back to dequantize-then-matmul in
torch, src/kernels/ops.py:777-792); there is no Triton or backend switch; no full-precision copy of a
weight is ever made inside the matmul functions.
"""
from __future__ import annotations

from typing import Optional

import torch

from pocketllm_amd import _ffi
from pocketllm_amd.cuda_loader import load_cuda_kernel


def _kernel():
    mod = load_cuda_kernel()
    if mod is None:
        raise RuntimeError("the native HIP library is unavailable (python -m pocketllm_amd.build)")
    return mod


def _on_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("this build has no CPU path: tensors must live on the GPU")


# ---- Q8_0 ---------------------------------------------------------------------------------------

def q8_0_weight_dequantize(blocks: torch.Tensor, row_elems: int | None = None) -> torch.Tensor:
    """uint8 [N, K/32, 34] -> float32 [N, row_elems]  (src/kernels/ops.py:734-741)."""
    assert blocks.dtype == torch.uint8 and blocks.dim() == 3 and blocks.size(-1) == 34
    _on_gpu(blocks)
    row_elems = int(blocks.size(1) * 32 if row_elems is None else row_elems)
    return _kernel().gguf_dequantize_rows(blocks.contiguous(), _ffi.TYPE_Q8_0, row_elems)


def q8_0_weight_gemm_cuda_ext(x: torch.Tensor, blocks: torch.Tensor, *, row_elems: int,
                              out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """src/kernels/ops.py:744-763."""
    mod = load_cuda_kernel()
    if mod is None or not hasattr(mod, "q8_0_gemm_forward"):
        raise RuntimeError("Q8_0 CUDA extension is unavailable")
    y = mod.q8_0_gemm_forward(x.contiguous(), blocks.contiguous(), int(row_elems))
    return y.to(torch.get_default_dtype() if out_dtype is None else out_dtype)


def q8_0_weight_gemm(x: torch.Tensor, blocks: torch.Tensor, *, row_elems: int | None = None, chunk_rows: int = 0,
                     out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """y = x W^T straight from the raw blocks, for any number of activation rows (src/kernels/ops.py:766-792).

    `chunk_rows` is accepted for signature compatibility; nothing is chunked because no dequantized
    copy exists.  The result is computed in float32 and cast once.
    """
    assert blocks.dtype == torch.uint8 and blocks.dim() == 3 and blocks.size(-1) == 34
    _on_gpu(x, blocks)
    row_elems = int(blocks.size(1) * 32 if row_elems is None else row_elems)
    y = _kernel().q8_0_gemm_forward(x.contiguous(), blocks.contiguous(), row_elems, out_dtype=torch.float32)
    return y.to(torch.get_default_dtype() if out_dtype is None else out_dtype)


# ---- FP8 E4M3 with 128 x 128 block scales --------------------------------------------------------

def soft_fp8_blockfp8_weight_dequant(weight: torch.Tensor, scale: torch.Tensor, block_size: int = 128, impl: str = "auto") -> torch.Tensor:
    """src/kernels/ops.py:572-590 / 144-147: float32 [N, K]."""
    assert block_size == 128
    _on_gpu(weight, scale)
    return _kernel().fp8_block_dequantize(weight.contiguous(), scale.to(torch.float32).contiguous())


soft_fp8_blockfp8_weight_dequant_torch = soft_fp8_blockfp8_weight_dequant


def soft_fp8_blockfp8_gemm(x: torch.Tensor, weight: torch.Tensor, scale: torch.Tensor, impl: str = "auto") -> torch.Tensor:
    """y = x (f32(W) * scales)^T in float32, cast to the default dtype (src/kernels/ops.py:641-648, 937-946)."""
    _on_gpu(x, weight, scale)
    y = _kernel().fp8_block_gemm_forward(x.contiguous(), weight.contiguous(), scale.to(torch.float32).contiguous())
    return y.to(torch.get_default_dtype())


soft_fp8_blockfp8_gemm_torch = soft_fp8_blockfp8_gemm


def blockfp8_act_quant(x: torch.Tensor, *, block_size: int = 128, round_scale_to_pow2: bool = False, eps: float = 1e-4,
                       impl: str = "auto") -> tuple[torch.Tensor, torch.Tensor]:
    """src/kernels/ops.py:501-516, 548-569."""
    assert block_size == 128 and x.shape[-1] % block_size == 0
    _on_gpu(x)
    return _kernel().fp8_act_quant_forward(x.contiguous(), eps=eps, round_scale_pow2=round_scale_to_pow2)


blockfp8_act_quant_torch = blockfp8_act_quant


def act_quant(x: torch.Tensor, block_size: int = 128, scale_fmt: Optional[str] = None,
              scale_dtype: torch.dtype = torch.float32, inplace: bool = False):
    """src/kernels/ops.py:982-1001."""
    quant, scales = blockfp8_act_quant(x, block_size=block_size, round_scale_to_pow2=scale_fmt is not None, eps=1e-4)
    if inplace:
        scale_full = scales.repeat_interleave(block_size, dim=-1)
        x.copy_((quant.to(torch.float32) * scale_full).to(x.dtype).view_as(x))
        return x
    return quant, scales.to(scale_dtype)


def _dequant_fp8_acts(a: torch.Tensor, a_s: torch.Tensor, block_size: int = 128) -> torch.Tensor:
    """src/kernels/ops.py:138-141."""
    return a.to(torch.float32) * a_s.to(torch.float32).repeat_interleave(block_size, dim=-1)[..., :a.size(-1)]


def fp8_gemm(a: torch.Tensor, a_s: torch.Tensor, b: torch.Tensor, b_s: torch.Tensor,
             scale_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """FP8 activations (codes + per-128 scales) times block-scaled FP8 weights (src/kernels/ops.py:1043-1051)."""
    _on_gpu(a, a_s, b, b_s)
    if a.shape[-1] % 128 == 0:
        # the matrix cores multiply the FP8 codes directly; the two scales meet the float32 block sums
        y = _kernel().fp8_gemm_forward(a.contiguous(), a_s.to(torch.float32).contiguous(), b.contiguous(), b_s.to(torch.float32).contiguous())
        return y.to(torch.get_default_dtype())
    return soft_fp8_blockfp8_gemm(_dequant_fp8_acts(a, a_s, 128).contiguous(), b, b_s)
