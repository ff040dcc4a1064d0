"""RMS normalisation ahead of the quantized projections: the stand-alone operator and the form fused into the decode matvec."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as O
from pocketllm_amd import block_codec as C, codebooks
from pocketllm_amd.cuda_loader import load_cuda_kernel

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture(scope="module")
def mod():
    m = load_cuda_kernel()
    assert m is not None and torch.cuda.is_available()
    return m


@pytest.mark.parametrize("rows,dim", [(1, 3072), (5, 1000), (3, 17408), (2, 7)])
def test_fused_rms_norm_matches_float64(mod, rows, dim):
    rng = np.random.default_rng(rows + dim)
    w = torch.from_numpy(rng.uniform(0.5, 1.5, size=dim).astype(np.float32)).to(DEV)
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        x = torch.from_numpy((rng.standard_normal((rows, dim)) * 3.0).astype(np.float32)).to(DEV).to(dt)
        y = mod.fused_rms_norm_forward(x, w, 1e-6)
        assert y.dtype == torch.float16 and tuple(y.shape) == (rows, dim)
        want = O.rms_norm(x.float().cpu().numpy(), w.cpu().numpy(), 1e-6)
        got = y.float().cpu().numpy().astype(np.float64)
        assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -10 + 1e-7)      # one fp16 rounding of a float32 result
        y32 = mod.fused_rms_norm_forward(x, w, 1e-6, out_dtype=torch.float32)
        np.testing.assert_allclose(y32.cpu().numpy(), want, rtol=3e-6, atol=1e-7)
    with pytest.raises(RuntimeError, match="weight must be fp32"):
        mod.fused_rms_norm_forward(x, w.half(), 1e-6)
    with pytest.raises(RuntimeError, match="must == dim"):
        mod.fused_rms_norm_forward(x, w[:-1], 1e-6)


def _blocks(rng, type_name, n, k):
    bpr = (k + 255) // 256
    if type_name in ("q4_k", "q5_k", "q2_k"):
        w = np.zeros((n, bpr * 256), dtype=np.float32)
        w[:, :k] = rng.standard_normal((n, k)) * 0.02
        return {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k, "q2_k": C.quantize_q2_k}[type_name](w)
    if type_name == "iq2_xxs":
        return C.random_iq2_xxs(rng, n, bpr)
    if type_name == "iq1_m":
        return C.random_iq1_m(rng, n, bpr)
    return C.random_blocks(rng, type_name, n, bpr)


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k", "q2_k", "q6_k", "iq4_xs", "iq2_xxs", "iq1_m", "iq2_xs", "iq3_xxs"])
def test_rmsnorm_fused_into_the_projection(mod, type_name):
    """One operator for normalisation + projection: against float64 (with and without the fp16 rounding of the normalized
    activations) and against the two operators run one after the other; 1 - 4 rows take the in-kernel form, 20 the workspace one."""
    rng = np.random.default_rng(len(type_name) * 13)
    tid = O.TYPE_IDS[type_name]
    grid = codebooks.grid_tensor_for_type(tid).to(DEV)
    for n, k, rows in ((48, 5120, 1), (130, 1002, 3), (16, 17408, 2), (64, 768, 20)):
        blocks_np = _blocks(rng, type_name, n, k)
        blocks = torch.from_numpy(blocks_np).to(DEV)
        wq = O.dequant_rows(blocks_np, type_name, k).astype(np.float64)
        gamma = torch.from_numpy(rng.uniform(0.5, 1.5, size=k).astype(np.float32)).to(DEV)
        for dt in (torch.bfloat16, torch.float32):
            x = torch.from_numpy((rng.standard_normal((rows, k)) * 2.0).astype(np.float32)).to(DEV).to(dt)
            print(f"case rmsnorm {type_name} n={n} k={k} rows={rows} {dt}", flush=True)
            normed = O.rms_norm(x.float().cpu().numpy(), gamma.cpu().numpy(), 1e-5)
            y_round = mod.gguf_quant_gemm_rmsnorm_forward(x, gamma, 1e-5, blocks, k, tid, grid, out_dtype=torch.float32)
            want_round = normed.astype(np.float32).astype(np.float16).astype(np.float64) @ wq.T
            assert O.rel_l2(y_round.cpu().numpy(), want_round) <= 1e-3
            chain = mod.gguf_quant_gemm_forward(mod.fused_rms_norm_forward(x, gamma, 1e-5), blocks, k, tid, grid, out_dtype=torch.float32)
            assert O.rel_l2(y_round.cpu().numpy(), chain.cpu().numpy().astype(np.float64)) <= 2e-4
            if rows <= 4:
                y_f32 = mod.gguf_quant_gemm_rmsnorm_forward(x, gamma, 1e-5, blocks, k, tid, grid, round_fp16=False, out_dtype=torch.float32)
                assert O.rel_l2(y_f32.cpu().numpy(), normed @ wq.T) <= 2e-4
    with pytest.raises(RuntimeError, match="weight must be fp32"):
        mod.gguf_quant_gemm_rmsnorm_forward(x, gamma.half(), 1e-5, blocks, k, tid, grid)
