"""ctypes binding of libpllm_hip.so (the C ABI declared in include/pllm_hip.h)."""
from __future__ import annotations

import ctypes
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libpllm_hip.so"

PLLM_OK = 0
PLLM_ERR_UNSUPPORTED = -2        # include/pllm_hip.h: type id or shape outside what the kernels implement
PLLM_ERR_WORKSPACE = -4          # the caller's workspace (or the library's static array) is too small
DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
TYPE_Q8_0 = 100
TYPE_Q3_K = 101   # dequantization only (the reference decodes it in numpy and gives it no id)

_c_void_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_size_t = ctypes.c_size_t

# name -> (restype, argtypes); must list every symbol include/pllm_hip.h declares
SIGNATURES = {
    "pllm_status_string": (ctypes.c_char_p, [_int]),
    "pllm_abi_version": (_int, []),
    "pllm_gguf_block_bytes": (_int, [_int]),
    "pllm_q8_0_gemm": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_q8_0_gemm_workspace_bytes": (_size_t, [_i64, _i64, _i64, _i64]),
    "pllm_gguf_quant_gemm": (_int, [_c_void_p, _int, _c_void_p, _int, _c_void_p, _int, _i64, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_quant_gemm_multi": (_int, [_c_void_p, _int, _c_void_p, ctypes.c_float, _int, _int, _c_void_p, _c_void_p, _int, _c_void_p, _int,
                                          _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_quant_gemm_accumulate": (_int, [_c_void_p, _int, _c_void_p, _int, _c_void_p, _int, _i64, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_quant_gemm_q8": (_int, [_c_void_p, _int, _c_void_p, _int, _c_void_p, _int, _i64, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_quant_gemm_q8_workspace_bytes": (_size_t, [_int, _i64, _i64, _i64, _i64]),
    "pllm_gguf_quant_gemm_static_scratch": (_int, [_c_void_p, _int, _c_void_p, _int, _c_void_p, _int, _i64, _i64, _i64, _i64, _c_void_p]),
    "pllm_gguf_quant_gemm_workspace_bytes": (_size_t, [_int, _i64, _i64, _i64, _i64]),
    "pllm_activation_image_bytes": (_size_t, [_i64, _i64]),
    "pllm_quantize_activations": (_int, [_c_void_p, _int, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_quant_gemm_prequantized": (_int, [_c_void_p, _c_void_p, _int, _c_void_p, _int, _i64, _i64, _i64, _c_void_p]),
    "pllm_gguf_quant_gemm_prequantized_accumulate": (_int, [_c_void_p, _c_void_p, _int, _c_void_p, _int, _i64, _i64, _i64, _c_void_p]),
    "pllm_swiglu_quantize_activations": (_int, [_c_void_p, _c_void_p, _int, _i64, _i64, _i64, ctypes.c_float, _int, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_quant_gemm_pair": (_int, [_c_void_p, _int, _c_void_p, _int, _c_void_p, _int, _c_void_p, _int, _i64, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_moe_workspace_bytes": (_size_t, [_i64, _i64, _i64, _i64]),
    "pllm_gguf_moe_forward": (_int, [_c_void_p, _int, _i64, _i64, _i64, _c_void_p, _c_void_p, _c_void_p, _i64, _c_void_p, _i64,
                                     _c_void_p, _c_void_p, _int, _c_void_p, _int, ctypes.c_float, _c_void_p, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_moe_single_token_accumulate": (_int, [_c_void_p, _int, _i64, _i64, _c_void_p, _c_void_p, _i64, _c_void_p, _c_void_p, _int, _c_void_p, _int,
                                                     ctypes.c_float, _c_void_p, _int, _c_void_p, _size_t, _c_void_p]),
    "pllm_moe_group_routes": (_int, [_c_void_p, _int, _c_void_p, _i64, _i64, _i64, _i64, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "pllm_gguf_dequantize_rows": (_int, [_c_void_p, _i64, _c_void_p, _int, _i64, _i64, _i64, _c_void_p, _int, _c_void_p]),
    "pllm_fp8_block_dequantize": (_int, [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _int, _c_void_p]),
    "pllm_fp8_block_gemm": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_fp8_block_gemm_accumulate": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _c_void_p]),
    "pllm_fp8_block_gemm_workspace_bytes": (_size_t, [_i64, _i64, _i64]),
    "pllm_fp8_fp16scale_matvec": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _i64, _c_void_p]),
    "pllm_fp8_fp16scale_swiglu_matvec": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int,
                                                _i64, _i64, _i64, _i64, _i64, _i64, _i64, _c_void_p]),
    "pllm_fp8_fp16scale_matmul_rows": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                              _c_void_p, _size_t, _c_void_p]),
    "pllm_fp8_fp16scale_matmul_rows_workspace_bytes": (_size_t, [_i64, _i64, _i64]),
    "pllm_fp8_bf16scale_matmul_rows": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _c_void_p]),
    "pllm_fp8_gemm": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _c_void_p]),
    "pllm_fp8_gemm_workspace_bytes": (_size_t, [_i64, _i64, _i64]),
    "pllm_fp8_gemm_ws": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_fused_rms_norm": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _int, _i64, _i64, ctypes.c_float, _c_void_p]),
    "pllm_attention_decode_workspace_bytes": (_size_t, [_i64, _i64, _i64]),
    "pllm_attention_decode": (_int, [_c_void_p, _c_void_p, _c_void_p, _int, _c_void_p, _c_void_p, ctypes.c_float, _c_void_p, _c_void_p, _i64,
                                     _c_void_p, _c_void_p, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _c_void_p, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_quant_gemm_rmsnorm": (_int, [_c_void_p, _int, _c_void_p, ctypes.c_float, _int, _c_void_p, _int, _c_void_p, _int,
                                            _i64, _i64, _i64, _i64, _c_void_p, _size_t, _c_void_p]),
    "pllm_gguf_quant_gemm_rmsnorm_workspace_bytes": (_size_t, [_int, _i64, _i64, _i64, _i64]),
    "pllm_moe_route": (_int, [_c_void_p, _int, _i64, _i64, _c_void_p, _c_void_p, _i64, _i64, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "pllm_moe_route_rmsnorm": (_int, [_c_void_p, _int, _c_void_p, ctypes.c_float, _c_void_p, _int, _i64, _i64, _c_void_p, _c_void_p, _i64, _i64, _int,
                                      _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "pllm_fp8_act_quant": (_int, [_c_void_p, _int, _i64, _i64, _c_void_p, _c_void_p, ctypes.c_float, _int, _c_void_p]),
}

_LIB = None


def load_library():
    """Returns the loaded library, or None when libpllm_hip.so has not been built."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not LIB_PATH.exists():
        return None
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _LIB = lib
    return lib


def check(status: int, what: str) -> None:
    if status != PLLM_OK:
        lib = load_library()
        msg = lib.pllm_status_string(status).decode() if lib is not None else str(status)
        raise RuntimeError(f"{what}: {msg} (status {status})")
