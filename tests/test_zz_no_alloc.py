"""The entry point that allocates nothing (pllm_gguf_quant_gemm_static_scratch) against pllm_gguf_quant_gemm, through the C ABI:
same bits on calls in a row, the later ones smaller than the first, for a decode call on a pre-quantized image and for a prefill
call on the tile kernel (both keep their temporaries in the library's device array); oversize calls are refused."""
import ctypes

import numpy as np
import pytest
import torch

from pocketllm_amd import _ffi, block_codec as C
from pocketllm_amd.cuda_loader import load_cuda_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
CODE = {torch.float32: _ffi.DTYPE_F32, torch.float16: _ffi.DTYPE_F16, torch.bfloat16: _ffi.DTYPE_BF16}


def _both(lib, x, blocks, type_id, k):
    rows, n, bpr = x.shape[0], blocks.shape[0], blocks.shape[1]
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.pllm_gguf_quant_gemm_workspace_bytes(type_id, rows, k, n, bpr)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device=DEV)
    want = torch.full((rows, n), float("nan"), dtype=torch.float32, device=DEV)
    got = torch.full((rows, n), float("nan"), dtype=torch.float32, device=DEV)
    st = lib.pllm_gguf_quant_gemm(x.data_ptr(), CODE[x.dtype], blocks.data_ptr(), type_id, want.data_ptr(), _ffi.DTYPE_F32,
                                  rows, k, n, bpr, ws.data_ptr(), need, stream)
    assert st == _ffi.PLLM_OK
    st = lib.pllm_gguf_quant_gemm_static_scratch(x.data_ptr(), CODE[x.dtype], blocks.data_ptr(), type_id, got.data_ptr(), _ffi.DTYPE_F32,
                                                 rows, k, n, bpr, stream)
    assert st == _ffi.PLLM_OK
    torch.cuda.synchronize()
    return need, want, got


def test_static_scratch_entry_point_matches_the_workspace_one():
    assert load_cuda_kernel() is not None and torch.cuda.is_available()
    lib = _ffi.load_library()
    rng = np.random.default_rng(91)
    enc = {3: C.quantize_q4_k, 4: C.quantize_q5_k}
    # (type id, rows, n, k): a decode call of 8 rows (activation image in the array), then smaller ones; a prefill call of 96
    # rows (staged fp16 rows and partial tiles in the array), then a smaller one
    for type_id, rows, n, k in ((3, 8, 640, 2048), (3, 6, 200, 1024), (4, 5, 48, 512), (4, 96, 520, 1536), (3, 33, 130, 768)):
        blocks = torch.from_numpy(enc[type_id]((rng.standard_normal((n, k)) * 0.02).astype(np.float32))).to(DEV)
        x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(DEV).to(torch.bfloat16)
        print(f"case static scratch type={type_id} rows={rows} n={n} k={k}", flush=True)
        need, want, got = _both(lib, x, blocks, type_id, k)
        assert need > 0, "the case no longer uses a workspace"
        assert not torch.isnan(want).any()
        assert torch.equal(got, want)
    # more than the array holds: refused with the workspace status, nothing launched
    rows, n, k = 4096, 4096, 4096
    assert lib.pllm_gguf_quant_gemm_workspace_bytes(3, rows, k, n, k // 256) > (16 << 20)
    st = lib.pllm_gguf_quant_gemm_static_scratch(ctypes.c_void_p(256), _ffi.DTYPE_BF16, ctypes.c_void_p(256), 3, ctypes.c_void_p(256), _ffi.DTYPE_F32,
                                                 rows, k, n, k // 256, None)
    assert st == _ffi.PLLM_ERR_WORKSPACE
    assert b"workspace" in lib.pllm_status_string(st)
