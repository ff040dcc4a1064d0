"""FP8 E4M3 weights with fp16 block scales: the reference C++ engine's raw-pointer operators over libpllm_hip.

The reference declares these in cpp_engine/include/qwen_cuda_ops.hpp:59-170 as
`bool f(const float* d_x, const uint8_t* d_weight, const uint16_t* d_scale_fp16, float* d_y, int rows, int cols,
int weight_stride, int scale_stride, void* stream)`: device pointers, caller-owned output, `false` for bad
arguments or a failed launch, never an exception.  The functions here keep that contract with torch tensors
standing in for the device pointers (any tensor whose storage holds the bytes; only `data_ptr()` is used):
`rows` counts OUTPUT rows, `cols` is the inner dimension, pitches are in elements, the output is written in
place and the return value is the reference's bool.  The `_f16` variants of the reference (fp16 activations
and outputs) are the same calls with fp16 tensors: the dtype is read from the tensors.
"""
from __future__ import annotations

import torch

from pocketllm_amd import _ffi

_DTYPE_CODE = {torch.float32: _ffi.DTYPE_F32, torch.float16: _ffi.DTYPE_F16, torch.bfloat16: _ffi.DTYPE_BF16}


def _lib():
    lib = _ffi.load_library()
    if lib is None:
        raise RuntimeError("libpllm_hip.so is not built (run `python -m pocketllm_amd.build`)")
    return lib


def _ptr(t):
    return t.data_ptr() if t is not None else None


def _on_one_gpu(*tensors) -> bool:
    return all(t is not None and t.is_cuda and t.device == tensors[0].device for t in tensors)


def _codes_ok(x, y) -> bool:
    return x.dtype in _DTYPE_CODE and y.dtype in _DTYPE_CODE


def qwen_fp8_e4m3_fp16scale_matvec(x, weight, scale_fp16, y, rows: int, cols: int, weight_stride: int, scale_stride: int) -> bool:
    """y[r] = sum_c x[c] * f32(weight[r, c]) * f32(scale[r // 128, c // 128]) (qwen_cuda_ops.hpp:59-69, 102-111)."""
    if not _on_one_gpu(x, weight, scale_fp16, y) or not _codes_ok(x, y):
        return False
    with torch.cuda.device(x.device):
        st = _lib().pllm_fp8_fp16scale_matvec(_ptr(x), _DTYPE_CODE[x.dtype], _ptr(weight), _ptr(scale_fp16), _ptr(y), _DTYPE_CODE[y.dtype],
                                              int(rows), int(cols), int(weight_stride), int(scale_stride),
                                              torch.cuda.current_stream(x.device).cuda_stream)
    return st == 0


def qwen_fp8_e4m3_fp16scale_swiglu_matvec(x, gate_weight, gate_scale_fp16, up_weight, up_scale_fp16, y, rows: int, cols: int,
                                          weight_stride: int, scale_stride: int, *, batch: int = 1, x_stride: int | None = None,
                                          y_stride: int | None = None) -> bool:
    """y[b, r] = silu(gate[r] . x_b) * (up[r] . x_b) (qwen_cuda_ops.hpp:72-83, 113-124; with batch > 1 and pitches the
    small-batch form, 126-140)."""
    if not _on_one_gpu(x, gate_weight, gate_scale_fp16, up_weight, up_scale_fp16, y) or not _codes_ok(x, y):
        return False
    with torch.cuda.device(x.device):
        st = _lib().pllm_fp8_fp16scale_swiglu_matvec(_ptr(x), _DTYPE_CODE[x.dtype], _ptr(gate_weight), _ptr(gate_scale_fp16), _ptr(up_weight),
                                                     _ptr(up_scale_fp16), _ptr(y), _DTYPE_CODE[y.dtype], int(batch), int(rows), int(cols),
                                                     int(cols if x_stride is None else x_stride), int(rows if y_stride is None else y_stride),
                                                     int(weight_stride), int(scale_stride), torch.cuda.current_stream(x.device).cuda_stream)
    return st == 0


def qwen_fp8_e4m3_fp16scale_matmul_rows(x, weight, scale_fp16, y, batch: int, rows: int, cols: int, x_stride: int, y_stride: int,
                                        weight_stride: int, scale_stride: int) -> bool:
    """The matvec over `batch` activation rows (qwen_cuda_ops.hpp:85-97, 142-170).  The workspace of the tile-kernel
    path is a torch tensor made here, so stream order and lifetime follow torch's allocator."""
    if not _on_one_gpu(x, weight, scale_fp16, y) or not _codes_ok(x, y):
        return False
    lib = _lib()
    with torch.cuda.device(x.device):
        ws_bytes = lib.pllm_fp8_fp16scale_matmul_rows_workspace_bytes(int(batch), int(rows), int(cols))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
        st = lib.pllm_fp8_fp16scale_matmul_rows(_ptr(x), _DTYPE_CODE[x.dtype], _ptr(weight), _ptr(scale_fp16), _ptr(y), _DTYPE_CODE[y.dtype],
                                                int(batch), int(rows), int(cols), int(x_stride), int(y_stride), int(weight_stride),
                                                int(scale_stride), _ptr(ws), ws_bytes, torch.cuda.current_stream(x.device).cuda_stream)
    return st == 0


def qwen_fp8_e4m3_bf16_matmul_rows(x, weight, scale_bf16, y, batch: int, rows: int, cols: int, x_stride: int, y_stride: int,
                                   weight_stride: int, scale_stride: int) -> bool:
    """The compatibility forms with bf16 scale bits (qwen_cuda_ops.hpp:172-197); batch 1 is qwen_fp8_e4m3_bf16_matvec_cuda."""
    if not _on_one_gpu(x, weight, scale_bf16, y) or not _codes_ok(x, y):
        return False
    with torch.cuda.device(x.device):
        st = _lib().pllm_fp8_bf16scale_matmul_rows(_ptr(x), _DTYPE_CODE[x.dtype], _ptr(weight), _ptr(scale_bf16), _ptr(y), _DTYPE_CODE[y.dtype],
                                                   int(batch), int(rows), int(cols), int(x_stride), int(y_stride), int(weight_stride),
                                                   int(scale_stride), torch.cuda.current_stream(x.device).cuda_stream)
    return st == 0


def qwen_fp8_e4m3_bf16_matvec(x, weight, scale_bf16, y, rows: int, cols: int, weight_stride: int, scale_stride: int) -> bool:
    return qwen_fp8_e4m3_bf16_matmul_rows(x, weight, scale_bf16, y, 1, rows, cols, cols, rows, weight_stride, scale_stride)
