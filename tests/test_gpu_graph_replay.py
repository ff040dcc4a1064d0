"""The decode operators under HIP graph capture: captured once, replayed several times with new inputs and with eager work and
synchronisations in between, every replay compared with the eager result (bit for bit: the kernels are deterministic)."""
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


def _replay_matches_eager(fn, static_inputs, fresh_inputs):
    """fn() reads the tensors of static_inputs; fresh_inputs: lists of tensors to copy into them before each replay."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                          # warm-up outside capture (allocator, function attributes)
        for _ in range(2):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    for step, fresh in enumerate(fresh_inputs):
        for dst, src in zip(static_inputs, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = fn()                                        # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {step} differs from the eager call"


@pytest.mark.parametrize("type_name,n,k", [("q4_k", 256, 5120), ("q5_k", 64, 17408), ("q2_k", 128, 1024), ("iq4_xs", 96, 2048), ("q6_k", 80, 1536)])
def test_decode_matvec_replays(mod, type_name, n, k):
    rng = np.random.default_rng(n + k)
    enc = {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k, "q2_k": C.quantize_q2_k, "q6_k": C.quantize_q6_k, "iq4_xs": C.quantize_iq4_xs}[type_name]
    blocks = torch.from_numpy(enc((rng.standard_normal((n, k)) * 0.02).astype(np.float32))).to(DEV)
    tid = O.TYPE_IDS[type_name]
    grid = codebooks.grid_tensor_for_type(tid).to(DEV)
    gamma = torch.from_numpy(rng.uniform(0.5, 1.5, size=k).astype(np.float32)).to(DEV)
    for rows in (1, 6):                                    # in-kernel quantization / activation pre-pass
        x = torch.randn(rows, k, device=DEV, dtype=torch.bfloat16)
        fresh = [[torch.randn(rows, k, device=DEV, dtype=torch.bfloat16)] for _ in range(3)]
        print(f"case graph {type_name} rows={rows}", flush=True)
        _replay_matches_eager(lambda: mod.gguf_quant_gemm_forward(x, blocks, k, tid, grid, out_dtype=torch.float32), [x], fresh)
        _replay_matches_eager(lambda: mod.gguf_quant_gemm_rmsnorm_forward(x, gamma, 1e-6, blocks, k, tid, grid, out_dtype=torch.float32), [x], fresh)


def test_single_token_experts_and_router_replay(mod):
    rng = np.random.default_rng(5)
    e, d, inter, topk = 16, 1024, 768, 4
    w1 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(DEV)
    w3 = torch.from_numpy(C.random_iq2_xxs(rng, e, inter, d // 256, d_range=(0.002, 0.006))).to(DEV)
    w2 = torch.from_numpy(C.random_iq1_m(rng, e, d, inter // 256, d_range=(0.002, 0.006))).to(DEV)
    gate = torch.randn(e, d, device=DEV) * d ** -0.5
    x = torch.randn(1, d, device=DEV, dtype=torch.bfloat16)

    def step():
        idx, w = mod.moe_route(x, gate, None, topk)
        return mod.gguf_moe_single_token_forward(x, idx[0], w[0], w1, w3, w2, 0.0)

    _replay_matches_eager(step, [x], [[torch.randn(1, d, device=DEV, dtype=torch.bfloat16)] for _ in range(3)])


def test_fp8_and_q8_0_replay(mod):
    rng = np.random.default_rng(6)
    n, k = 256, 1024
    codes, scale = C.quantize_fp8_block((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    codes, scale = torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV)
    q8 = torch.from_numpy(C.pack_q8_0((rng.standard_normal((n, k)) * 0.02).astype(np.float32))).to(DEV)
    x = torch.randn(1, k, device=DEV)
    fresh = [[torch.randn(1, k, device=DEV)] for _ in range(3)]
    _replay_matches_eager(lambda: mod.fp8_block_gemm_forward(x, codes, scale), [x], fresh)
    _replay_matches_eager(lambda: mod.q8_0_gemm_forward(x, q8, k, out_dtype=torch.float32), [x], fresh)
