"""The one-operator decode step of attention (pllm_attention_decode through attention_decode_forward) against a float64
statement of the same arithmetic (reference: src/models/minimax_m2/architecture.py:158-266 for one query position): RMS
normalisation of q and k over their whole width, half-split rotary phases, the new row in the stores, grouped-query softmax
attention over positions 0 .. pos.  Tolerance: rel-L2 <= 3e-3 in fp16 and <= 1.5e-2 in bf16 (the operator rounds the normalized
and the turned values and its output to the 16-bit type; the statement does not)."""
import numpy as np
import pytest
import torch

from pocketllm_amd.attention_core import RotaryTable
from pocketllm_amd.cuda_loader import load_cuda_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _statement(q, k_new, v_new, keys, values, pos, heads, kv_heads, qw, kw, eps, cos, sin, rope_dim):
    """float64 on the CPU; keys / values [batch, kv_heads, >= pos, 128] hold positions 0 .. pos - 1."""
    q, k_new, v_new, keys, values = (t.double().cpu() for t in (q, k_new, v_new, keys, values))
    batch, dim = q.size(0), 128
    half = rope_dim // 2

    def norm(x, w):
        return x if w is None else x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w.double().cpu()

    def turn(x):                                  # [batch, heads, 128]
        if rope_dim == 0:
            return x
        partner = torch.cat((x[..., half:2 * half], x[..., :half], x[..., 2 * half:]), dim=-1)
        return x * cos.double().cpu() + partner * sin.double().cpu()

    qh = turn(norm(q, qw).view(batch, heads, dim))
    kh = turn(norm(k_new, kw).view(batch, kv_heads, dim))
    all_k = torch.cat((keys[:batch, :, :pos], kh.unsqueeze(2)), dim=2)              # [batch, kv_heads, pos + 1, 128]
    all_v = torch.cat((values[:batch, :, :pos], v_new.view(batch, kv_heads, 1, dim)), dim=2)
    group = heads // kv_heads
    qg = qh.view(batch, kv_heads, group, dim)
    scores = torch.einsum("bkgd,bkld->bkgl", qg, all_k) / np.sqrt(dim)
    out = torch.einsum("bkgl,bkld->bkgd", torch.softmax(scores, dim=-1), all_v)
    return out.reshape(batch, heads * dim), kh


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 3e-3), (torch.bfloat16, 1.5e-2)])
def test_decode_step_matches_the_float64_statement(dtype, tol):
    mod = load_cuda_kernel()
    assert mod is not None and torch.cuda.is_available()
    gen = torch.Generator(device="cpu").manual_seed(11)
    cases = (  # heads, kv_heads, rope_dim, batch, positions, norm weights
        (48, 8, 64, 1, (0, 5, 63, 64, 65, 700, 2047), True),
        (16, 2, 128, 2, (1, 64, 130), True),
        (8, 8, 0, 3, (3, 127, 128), False),
        (12, 4, 32, 1, (255, 256), True),
    )
    for heads, kv_heads, rope_dim, batch, positions, with_norm in cases:
        capacity = max(positions) + 1
        table = RotaryTable(rope_dim, 1.0e4, torch.device(DEV), head_dim=128, positions=capacity)
        qw = (torch.rand(heads * 128, generator=gen) + 0.5).to(DEV) if with_norm else None
        kw = (torch.rand(kv_heads * 128, generator=gen) + 0.5).to(DEV) if with_norm else None
        for pos in positions:
            keys = (torch.randn(batch + 1, kv_heads, capacity, 128, generator=gen) * 0.7).to(DEV).to(dtype)
            values = torch.randn(batch + 1, kv_heads, capacity, 128, generator=gen).to(DEV).to(dtype)
            q = (torch.randn(batch, heads * 128, generator=gen) * 2.0).to(DEV).to(dtype)
            k_new = torch.randn(batch, kv_heads * 128, generator=gen).to(DEV).to(dtype)
            v_new = torch.randn(batch, kv_heads * 128, generator=gen).to(DEV).to(dtype)
            cos, sin = table.rows(pos)
            want, want_k = _statement(q, k_new, v_new, keys, values, pos, heads, kv_heads, qw, kw, 1e-6, cos, sin, rope_dim)
            keys_before, values_before = keys.clone(), values.clone()
            print(f"case attention decode {dtype} heads={heads}/{kv_heads} rope={rope_dim} batch={batch} pos={pos}", flush=True)
            got = mod.attention_decode_forward(q, k_new, v_new, keys, values, pos, q_norm_weight=qw, k_norm_weight=kw, eps=1e-6,
                                               cos_row=cos, sin_row=sin, rope_dim=rope_dim)
            torch.cuda.synchronize()
            assert got.shape == (batch, heads * 128) and got.dtype == dtype
            err = (got.double().cpu() - want).norm() / want.norm()
            assert err <= tol, f"rel-L2 {err:.3e}"
            # the stores: position pos of the first `batch` sequences holds the new rows, nothing else moved
            new_k = keys[:batch, :, pos].double().cpu()
            assert (new_k - want_k).norm() / want_k.norm() <= tol
            assert torch.equal(values[:batch, :, pos], v_new.view(batch, kv_heads, 128))
            keys_before[:batch, :, pos] = keys[:batch, :, pos]
            values_before[:batch, :, pos] = values[:batch, :, pos]
            assert torch.equal(keys, keys_before) and torch.equal(values, values_before)


def test_decode_step_rejects_what_it_does_not_take():
    mod = load_cuda_kernel()
    keys = torch.zeros(1, 2, 8, 64, device=DEV, dtype=torch.float16)       # 64-wide heads
    q = torch.zeros(1, 4 * 64, device=DEV, dtype=torch.float16)
    kv = torch.zeros(1, 2 * 64, device=DEV, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        mod.attention_decode_forward(q, kv, kv, keys, keys.clone(), 0)
    keys = torch.zeros(1, 1, 8, 128, device=DEV, dtype=torch.float16)      # sixteen query heads on one key/value head
    q = torch.zeros(1, 16 * 128, device=DEV, dtype=torch.float16)
    kv = torch.zeros(1, 128, device=DEV, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        mod.attention_decode_forward(q, kv, kv, keys, keys.clone(), 0)
    with pytest.raises(RuntimeError):                                      # position outside the stores
        mod.attention_decode_forward(torch.zeros(1, 128, device=DEV, dtype=torch.float16), kv, kv, keys, keys.clone(), 8)
