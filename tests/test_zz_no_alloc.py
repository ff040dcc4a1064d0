"""The entry point that allocates nothing (pllm_gguf_quant_gemm_static_scratch) against pllm_gguf_quant_gemm, through the C ABI:
same bits on calls in a row, the later ones smaller than the first, for every kind of call that keeps temporaries in the library's
device array: decode calls whose activation image is written there by the pre-pass (float32 activations of 5 - 8 rows, and a
Q6_K call of 7 bf16 rows; 16-bit rows of Q4_K / Q5_K at these counts run a kernel without workspace and would test nothing), a
33-row call (staged fp16 rows and the partial sums of its K slices) and a 96-row call on the tile kernel (staged rows and partial
tiles); oversize calls are refused."""
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
    enc = {3: C.quantize_q4_k, 4: C.quantize_q5_k, 8: C.quantize_q6_k}
    # (type id, rows, n, k, activation type): decode calls on an activation image in the array, each smaller than the one before;
    # then the two prefill forms, the larger first
    for type_id, rows, n, k, dt in ((3, 8, 640, 2048, torch.float32), (3, 6, 200, 1024, torch.float32), (4, 5, 48, 512, torch.float32),
                                    (8, 7, 96, 512, torch.bfloat16), (4, 96, 520, 1536, torch.bfloat16), (3, 33, 130, 768, torch.bfloat16)):
        blocks = torch.from_numpy(enc[type_id]((rng.standard_normal((n, k)) * 0.02).astype(np.float32))).to(DEV)
        x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(DEV).to(dt)
        print(f"case static scratch type={type_id} rows={rows} n={n} k={k} {dt}", flush=True)
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
