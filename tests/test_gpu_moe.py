"""GPU parity of the routed-expert operators, route grouping and the paired projection."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as O
from pocketllm_amd import _ffi, block_codec as C, codebooks
from pocketllm_amd.cuda_loader import load_cuda_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-3
GEN = {"iq2_xxs": C.random_iq2_xxs, "iq1_m": C.random_iq1_m}


@pytest.fixture(scope="module")
def mod():
    m = load_cuda_kernel()
    assert m is not None and torch.cuda.is_available()
    return m


def _expert_blocks(rng, type_name, e, n, k):
    if type_name == "q2_k":
        w = (rng.standard_normal((e * n, k)) * 0.05).astype(np.float32)
        return C.quantize_q2_k(w).reshape(e, n, k // 256, 84)
    # scales sized so that the hidden activations stay O(1)
    return GEN[type_name](rng, e, n, (k + 255) // 256, d_range=(0.002, 0.006))


def _route(rng, t, e, topk):
    logits = rng.standard_normal((t, e)).astype(np.float32)
    p = np.exp(logits - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    idx = np.argsort(-p, axis=1)[:, :topk].astype(np.int64)
    w = np.take_along_axis(p, idx, axis=1)
    return idx, (w / w.sum(axis=1, keepdims=True)).astype(np.float32)


@pytest.mark.parametrize("t13,t2", [("iq2_xxs", "iq1_m"), ("iq2_xxs", "iq2_xxs"), ("iq2_xxs", "q2_k"), ("iq1_m", "iq1_m")])
@pytest.mark.parametrize("limit", [0.0, 0.6])
def test_single_token_experts(mod, t13, t2, limit):
    rng = np.random.default_rng(100 + len(t13) + len(t2))
    e, d, inter, topk = 8, 512, 768, 4
    w1 = _expert_blocks(rng, t13, e, inter, d)
    w3 = _expert_blocks(rng, t13, e, inter, d)
    w2 = _expert_blocks(rng, t2, e, d, inter)
    idx, wts = _route(rng, 1, e, topk)
    x = torch.from_numpy(rng.standard_normal((1, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    slots = torch.from_numpy(idx[0]).to(DEV)
    rw = torch.from_numpy(wts[0]).to(DEV)
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    print(f"case single {t13}/{t2} limit={limit}", flush=True)
    y = mod.gguf_moe_single_token_forward(x, slots, rw, dw1, dw3, dw2, limit)
    torch.cuda.synchronize()
    want = O.moe_forward(x.float().cpu().numpy(), np.zeros(topk, dtype=np.int64), wts[0], idx[0], w1, w3, w2, t13, t13, t2, limit)
    assert y.dtype == torch.float32 and tuple(y.shape) == (1, d)
    assert O.rel_l2(y.cpu().numpy(), want) <= TOL
    # the reference-named operators where they apply
    if t13 == "iq2_xxs" and t2 in ("iq2_xxs", "q2_k"):
        grid = codebooks.get_iq2xxs_signed_grid_tensor().to(DEV)
        y2 = mod.gguf_moe_single_token_iq2_q2k_forward(x, slots, rw, dw1, dw3, dw2, grid, limit)
        assert torch.equal(y2, y)
    if t13 == "iq1_m" and t2 == "iq1_m":
        y2 = mod.gguf_moe_single_token_iq1m_forward(x, slots, rw, dw1, dw3, dw2, codebooks.get_iq1_grid_tensor().to(DEV), limit)
        assert torch.equal(y2, y)


@pytest.mark.parametrize("t13,t2", [("iq2_xxs", "iq1_m"), ("iq2_xxs", "q2_k")])
def test_grouped_experts_and_route_grouping(mod, t13, t2):
    rng = np.random.default_rng(7)
    e, d, inter, topk, t = 12, 512, 512, 3, 9
    w1 = _expert_blocks(rng, t13, e, inter, d)
    w3 = _expert_blocks(rng, t13, e, inter, d)
    w2 = _expert_blocks(rng, t2, e, d, inter)
    idx, wts = _route(rng, t, e + 4, topk)                 # experts 0..15, local window 2..13
    start = 2
    x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    local_ids, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), start, e)
    o_ids, o_toks, o_rws, o_seg = O.group_routes(idx, wts, start, e)
    assert local_ids.cpu().tolist() == o_ids.tolist()
    np.testing.assert_array_equal(seg.cpu().numpy(), o_seg)
    np.testing.assert_array_equal(toks.cpu().numpy(), o_toks)          # stable order: same as the oracle's
    np.testing.assert_array_equal(rws.cpu().numpy(), o_rws)
    # int32 indices give the same grouping
    _, toks32, _, seg32 = mod.moe_group_routes(torch.from_numpy(idx.astype(np.int32)).to(DEV), torch.from_numpy(wts).to(DEV), start, e)
    assert torch.equal(toks32, toks) and torch.equal(seg32, seg)

    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), codebooks.get_iq1_grid_tensor().to(DEV))
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid[t13], d, tid[t13], inter, tid[t2], grids, 0.0)
    torch.cuda.synchronize()
    route_experts = np.repeat(np.arange(e), np.diff(o_seg))
    want = O.moe_forward(x.float().cpu().numpy(), o_toks, o_rws, route_experts, w1, w3, w2, t13, t13, t2, 0.0)
    assert O.rel_l2(y.cpu().numpy(), want) <= TOL
    # run-to-run bitwise determinism (the reference's atomics cannot promise this)
    y2 = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg.to(torch.int64), dw1, dw3, dw2, d, tid[t13], d, tid[t13], inter, tid[t2], grids, 0.0)
    assert torch.equal(y, y2)
    if t2 == "iq1_m":
        with pytest.raises(RuntimeError, match="cannot mix iq2_xxs and iq1_m"):
            mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, 0, d, 0, inter, 2, grids[0], 0.0)


def test_no_routes_gives_zeros(mod):
    e, d, inter = 2, 256, 256
    z = torch.zeros(e, inter, 1, 66, dtype=torch.uint8, device=DEV)
    z2 = torch.zeros(e, d, 1, 66, dtype=torch.uint8, device=DEV)
    x = torch.randn(3, d, device=DEV)
    y = mod.gguf_moe_prefill_grouped_forward(x, torch.empty(0, dtype=torch.int64, device=DEV), torch.empty(0, device=DEV),
                                             torch.zeros(e + 1, dtype=torch.int32, device=DEV), z, z, z2, d, 0, d, 0, inter, 0,
                                             codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), 0.0)
    assert tuple(y.shape) == (3, d) and float(y.abs().max()) == 0.0


def test_baseline_config_single_token_shapes(mod):
    """BASELINE config 5 at T = 1 with 16 of the 256 experts materialised (routing only touches 8)."""
    rng = np.random.default_rng(1005)
    e, d, inter, topk = 16, 3072, 1536, 8
    w1 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w3 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w2 = _expert_blocks(rng, "iq1_m", e, d, inter)
    idx, wts = _route(rng, 1, e, topk)
    x = torch.from_numpy(rng.standard_normal((1, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    y = mod.gguf_moe_single_token_forward(x, torch.from_numpy(idx[0]).to(DEV), torch.from_numpy(wts[0]).to(DEV),
                                          *(torch.from_numpy(a).to(DEV) for a in (w1, w3, w2)), 0.0)
    torch.cuda.synchronize()
    want = O.moe_forward(x.float().cpu().numpy(), np.zeros(topk, dtype=np.int64), wts[0], idx[0], w1, w3, w2, "iq2_xxs", "iq2_xxs", "iq1_m", 0.0)
    assert O.rel_l2(y.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_single_token_experts_added_into_the_residual_stream(mod, dtype):
    """y += experts(x) inside the down projection's launch: the float32 sum of what y held and the result of the plain operator
    (bit for bit the same routes' sum), rounded once to y's type; shapes or type pairs without such a kernel report False and
    leave y alone."""
    rng = np.random.default_rng(2718)
    e, d, inter, topk = 16, 3072, 1536, 8
    w1 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w3 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w2 = _expert_blocks(rng, "iq1_m", e, d, inter)
    idx, wts = _route(rng, 1, e, topk)
    x = torch.from_numpy(rng.standard_normal((1, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    slots, rw = torch.from_numpy(idx[0]).to(DEV), torch.from_numpy(wts[0]).to(DEV)
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    plain = mod.gguf_moe_single_token_forward(x, slots, rw, dw1, dw3, dw2, 0.0)
    stream = torch.from_numpy(rng.standard_normal((1, d)).astype(np.float32)).to(DEV).to(dtype)
    y = stream.clone()
    print(f"case accumulate {dtype}", flush=True)
    assert mod.gguf_moe_single_token_accumulate_forward(x, slots, rw, dw1, dw3, dw2, 0.0, y) is True
    torch.cuda.synchronize()
    assert torch.equal(y, (stream.float() + plain).to(dtype))
    # types without fused expert kernels: the down projection with the routes as its waves adds into y
    for t13, t2 in (("q4_k", "q6_k"), ("q5_k", "q4_k")):
        g1, g3, g2 = (torch.from_numpy(_any_expert_blocks(rng, t, 4, n, k)).to(DEV) for t, n, k in ((t13, 512, 768), (t13, 512, 768), (t2, 768, 512)))
        xs = x[:, :768].contiguous()
        few = torch.tensor([3, 0, 2], dtype=torch.int64, device=DEV)
        fw = torch.tensor([0.5, 0.3, 0.2], device=DEV)
        plain_g = mod.gguf_moe_single_token_forward(xs, few, fw, g1, g3, g2, 0.0)
        base = stream[:, :768].contiguous()
        yg = base.clone()
        assert mod.gguf_moe_single_token_accumulate_forward(xs, few, fw, g1, g3, g2, 0.0, yg) is True
        assert torch.equal(yg, (base.float() + plain_g).to(dtype))
    # a type pair whose down projection has no such kernel: refused, y untouched
    w2q = torch.from_numpy(_expert_blocks(rng, "q2_k", e, d, inter)).to(DEV)
    y2 = stream.clone()
    assert mod.gguf_moe_single_token_accumulate_forward(x, slots, rw, dw1, dw3, w2q, 0.0, y2) is False
    assert torch.equal(y2, stream)


def test_baseline_config_grouped_256_tokens_256_experts(mod):
    """BASELINE config 5 at T = 256: 256 experts, top-8 softmax routing, 2048 routes, every weight tensor at its full size.
    The oracle restates the operator for 32 sampled tokens (their 256 routes, full output rows); every other token is
    covered by the determinism check and by the finite, non-zero rows.  The same full-size tensors then serve the single-token
    operator on routes to the far end of the expert range (ids above 200: offsets of hundreds of megabytes into w1 / w3 / w2)."""
    rng = np.random.default_rng(1005)
    e, d, inter, topk, t = 256, 3072, 1536, 8, 256
    w1 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w3 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w2 = _expert_blocks(rng, "iq1_m", e, d, inter)
    idx, wts = _route(rng, t, e, topk)
    x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    _, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), 0, e)
    _, o_toks, o_rws, o_seg = O.group_routes(idx, wts, 0, e)
    np.testing.assert_array_equal(seg.cpu().numpy(), o_seg)
    np.testing.assert_array_equal(toks.cpu().numpy(), o_toks)
    assert len(o_toks) == t * topk
    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), codebooks.get_iq1_grid_tensor().to(DEV))
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    print("case grouped experts 256 tokens x 256 experts", flush=True)
    y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid["iq2_xxs"], d, tid["iq2_xxs"], inter, tid["iq1_m"], grids, 0.0)
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    assert got.shape == (t, d) and np.isfinite(got).all() and (np.abs(got).max(axis=1) > 0).all()
    route_experts = np.repeat(np.arange(e), np.diff(o_seg))
    sample = rng.choice(t, size=32, replace=False)
    keep = np.isin(o_toks, sample)
    want = O.moe_forward(x.float().cpu().numpy(), o_toks[keep], o_rws[keep], route_experts[keep], w1, w3, w2, "iq2_xxs", "iq2_xxs", "iq1_m", 0.0)
    assert O.rel_l2(got[sample], want[sample]) <= TOL
    for tok in sample:
        assert O.rel_l2(got[tok], want[tok]) <= 2 * TOL, tok
    y2 = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid["iq2_xxs"], d, tid["iq2_xxs"], inter, tid["iq1_m"], grids, 0.0)
    assert torch.equal(y, y2)
    # T = 1 on the same 256-expert tensors, routed to experts at the far end of the range
    far = np.array([255, 201, 230, 7, 248, 213, 128, 254], dtype=np.int64)
    fw = rng.uniform(0.05, 0.3, size=topk).astype(np.float32)
    print("case single token, experts above 200 of 256", flush=True)
    y1 = mod.gguf_moe_single_token_forward(x[:1].contiguous(), torch.from_numpy(far).to(DEV), torch.from_numpy(fw).to(DEV), dw1, dw3, dw2, 0.0)
    torch.cuda.synchronize()
    want1 = O.moe_forward(x[:1].float().cpu().numpy(), np.zeros(topk, dtype=np.int64), fw, far, w1, w3, w2, "iq2_xxs", "iq2_xxs", "iq1_m", 0.0)
    assert O.rel_l2(y1.cpu().numpy(), want1) <= TOL


def test_grouped_experts_more_routes_than_the_reduction_lists(mod):
    """More than 2048 routes (the route-sum kernel reads the route table in pieces of 2048: two pieces, then three) and 60 / 120 routes
    per expert on average (every expert's routes pass through the matrix-row kernels in several batches of 16)."""
    rng = np.random.default_rng(17)
    e, d, inter, topk = 40, 256, 256, 8
    w1 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w3 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w2 = _expert_blocks(rng, "iq1_m", e, d, inter)
    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), codebooks.get_iq1_grid_tensor().to(DEV))
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    for t in (300, 600):
        idx, wts = _route(rng, t, e, topk)
        x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
        _, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), 0, e)
        _, o_toks, o_rws, o_seg = O.group_routes(idx, wts, 0, e)
        assert len(o_toks) == 8 * t
        print(f"case grouped experts {8 * t} routes", flush=True)
        y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid["iq2_xxs"], d, tid["iq2_xxs"], inter, tid["iq1_m"], grids, 0.0)
        torch.cuda.synchronize()
        route_experts = np.repeat(np.arange(e), np.diff(o_seg))
        want = O.moe_forward(x.float().cpu().numpy(), o_toks, o_rws, route_experts, w1, w3, w2, "iq2_xxs", "iq2_xxs", "iq1_m", 0.0)
        assert O.rel_l2(y.cpu().numpy(), want) <= TOL


def test_route_slots_host_compaction(mod):
    idx = torch.tensor([[9, 3, 12, 4, 3]], device=DEV)
    w = torch.tensor([[0.1, 0.2, 0.3, 0.25, 0.15]], device=DEV)
    local_ids, toks, rw, slots, starts = mod.gguf_single_token_route_slots(idx, w, 3, 8)     # local window 3..10
    assert local_ids.tolist() == [0, 1, 6] and not local_ids.is_cuda
    assert slots.cpu().tolist() == [0, 0, 1, 2] and starts.cpu().tolist() == [0, 2, 3, 4]
    assert toks.cpu().tolist() == [0, 0, 0, 0]
    np.testing.assert_allclose(rw.cpu().numpy(), [0.2, 0.15, 0.25, 0.1])


def test_paired_projection(mod):
    rng = np.random.default_rng(21)
    n, k = 48, 1024
    wa = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    wb = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = torch.randn(1, 3, k, device=DEV, dtype=torch.bfloat16)
    grid = torch.empty(0, dtype=torch.int8, device=DEV)
    for tid, enc in ((3, C.quantize_q4_k), (4, C.quantize_q5_k)):
        ba, bb = torch.from_numpy(enc(wa)).to(DEV), torch.from_numpy(enc(wb)).to(DEV)
        y = mod.gguf_quant_gemm_pair_forward(x, ba, k, tid, bb, k, tid, grid)
        assert y.dtype == torch.bfloat16 and tuple(y.shape) == (2, 1, 3, n)
        # pair == the two separate calls, bit for bit (the reference's own test: tests/test_gguf_quantized_ops_cuda.py:83-92)
        assert torch.equal(y[0], mod.gguf_quant_gemm_prefill_forward(x, ba, k, tid, grid))
        assert torch.equal(y[1], mod.gguf_quant_gemm_prefill_forward(x, bb, k, tid, grid))
    # one launch over both matrices: also with rows that take the activation pre-pass and with mixed types (two launches)
    for rows, ta, tb in ((1, 4, 4), (6, 3, 3), (2, 3, 4)):
        xr = torch.randn(rows, k, device=DEV, dtype=torch.bfloat16)
        ea, eb = ({3: C.quantize_q4_k, 4: C.quantize_q5_k}[t] for t in (ta, tb))
        ba, bb = torch.from_numpy(ea(wa)).to(DEV), torch.from_numpy(eb(wb)).to(DEV)
        y = mod.gguf_quant_gemm_pair_forward(xr, ba, k, ta, bb, k, tb, grid, out_dtype=torch.float32)
        assert torch.equal(y[0], mod.gguf_quant_gemm_forward(xr, ba, k, ta, grid, out_dtype=torch.float32))
        assert torch.equal(y[1], mod.gguf_quant_gemm_forward(xr, bb, k, tb, grid, out_dtype=torch.float32))
    with pytest.raises(RuntimeError, match="paired blocks must have same output rows"):
        mod.gguf_quant_gemm_pair_forward(x, ba, k, 4, bb[:8], k, 4, grid)


def test_linear_modules(mod):
    from pocketllm_amd.quantized_ops import Q8_0GGUFLinear, QuantizedGGUFEmbedding, QuantizedGGUFLinear
    from pocketllm_amd.quantized_tensor import QuantizedGGUFTensor
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((64, 512)) * 0.02).astype(np.float32)
    blocks = C.quantize_q5_k(w)
    t = QuantizedGGUFTensor.from_blocks(torch.from_numpy(blocks).to(DEV), "q5_k", 512, source_name="proj")
    lin = QuantizedGGUFLinear(t)
    assert (lin.in_dim, lin.out_dim, lin.row_start) == (512, 64, 0)
    ref = O.dequant_rows(blocks, "q5_k")
    for shape in ((1, 512), (5, 512), (2, 3, 512)):
        x = torch.randn(*shape, device=DEV, dtype=torch.float16)
        y = lin(x)
        assert y.dtype == torch.float16 and tuple(y.shape) == shape[:-1] + (64,)
        want = O.matmul_f(x.float().cpu().numpy().reshape(-1, 512), ref).reshape(shape[:-1] + (64,))
        assert np.abs(y.float().cpu().numpy() - want).max() < 2e-2       # the reference's bound for this wrapper
    with pytest.raises(ValueError, match="expected input dim 512"):
        lin(torch.randn(1, 256, device=DEV))
    y0, y1 = QuantizedGGUFLinear.pair(lin, lin, torch.randn(1, 512, device=DEV, dtype=torch.float16))
    assert torch.equal(y0, y1)
    emb = QuantizedGGUFEmbedding(t)
    assert emb.dim == 512 and tuple(emb(torch.tensor([1, 2, 3], device=DEV, dtype=torch.int32)).shape) == (3, 512)
    # the two table-free types the reference's linear wrapper also serves (it passes an empty grid)
    for name, enc in (("q6_k", C.quantize_q6_k), ("iq4_xs", C.quantize_iq4_xs)):
        bl = enc(w)
        lin2 = QuantizedGGUFLinear(QuantizedGGUFTensor.from_blocks(torch.from_numpy(bl).to(DEV), name, 512, source_name=name))
        x = torch.randn(3, 512, device=DEV, dtype=torch.float16)
        want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(bl, name))
        assert np.abs(lin2(x).float().cpu().numpy() - want).max() < 2e-2
    # the codebook types: the module brings the grid of its type itself (one upload per type and device)
    for name in ("iq2_xxs", "iq1_m", "iq2_xs", "iq3_xxs"):
        bl = GEN[name](rng, 64, 2) if name in GEN else C.random_blocks(rng, name, 64, 2)
        lin3 = QuantizedGGUFLinear(QuantizedGGUFTensor.from_blocks(torch.from_numpy(bl).to(DEV), name, 512, source_name=name))
        lin4 = QuantizedGGUFLinear(QuantizedGGUFTensor.from_blocks(torch.from_numpy(bl).to(DEV), name, 512, source_name=name))
        assert lin3._grid.data_ptr() == lin4._grid.data_ptr()
        x = torch.randn(3, 512, device=DEV, dtype=torch.float16)
        want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(bl, name))
        got = lin3(x).float().cpu().numpy()
        assert O.rel_l2(got, want) < 2e-3, name
        emb3 = QuantizedGGUFEmbedding(QuantizedGGUFTensor.from_blocks(torch.from_numpy(bl).to(DEV), name, 512, source_name=name))
        rows = emb3(torch.tensor([5, 63], device=DEV, dtype=torch.int32)).float().cpu().numpy()
        assert O.rel_l2(rows, O.dequant_rows(bl[[5, 63]], name)) < 2e-3, name
    q8 = Q8_0GGUFLinear(torch.from_numpy(C.pack_q8_0(w)).to(DEV), 512, source_name="q8")
    x = torch.randn(2, 512, device=DEV, dtype=torch.float16)
    want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(C.pack_q8_0(w), "q8_0"))
    assert np.abs(q8(x).float().cpu().numpy() - want).max() < 2e-2
    with pytest.raises(ValueError, match="q8_0 blocks must be"):
        Q8_0GGUFLinear(torch.zeros(4, 2, 33, dtype=torch.uint8, device=DEV), 64)


@pytest.mark.parametrize("t13,e,d,inter,topk,t,limit", [("iq2_xxs", 6, 3072, 1536, 2, 24, 0.0), ("iq2_xxs", 5, 768, 1072, 3, 14, 0.5),
                                                        ("iq1_m", 7, 1024, 512, 2, 28, 0.0), ("iq2_xxs", 3, 256, 256, 3, 2, 0.0)])
def test_grouped_experts_matrix_core_path(mod, t13, e, d, inter, topk, t, limit):
    """Up to 8 routes per expert on average with an IQ1_M down projection: every expert's blocks are decoded once and its
    routes pass through in batches (several batches for the busier experts, an intermediate size that is not a multiple of 256)."""
    rng = np.random.default_rng(13 + t)
    w1 = _expert_blocks(rng, t13, e, inter, d)
    w3 = _expert_blocks(rng, t13, e, inter, d)
    w2 = _expert_blocks(rng, "iq1_m", e, d, inter)
    idx, wts = _route(rng, t, e + 2, topk)                 # local window 1..e
    x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    _, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), 1, e)
    _, o_toks, o_rws, o_seg = O.group_routes(idx, wts, 1, e)
    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), codebooks.get_iq1_grid_tensor().to(DEV))
    if t13 == "iq1_m":
        grids = grids[1]
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    print(f"case matrix-core grouped {t13} e={e} d={d} inter={inter} t={t} routes={len(o_toks)}", flush=True)
    assert 1 < t and len(o_toks) <= 8 * e, "shape no longer selects the grouped matrix-core kernels"
    assert t == 2 or np.diff(o_seg).max() > 4, "no expert with more than one batch of routes"
    y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid[t13], d, tid[t13], inter, tid["iq1_m"], grids, limit)
    torch.cuda.synchronize()
    route_experts = np.repeat(np.arange(e), np.diff(o_seg))
    want = O.moe_forward(x.float().cpu().numpy(), o_toks, o_rws, route_experts, w1, w3, w2, t13, t13, "iq1_m", limit)
    assert O.rel_l2(y.cpu().numpy(), want) <= TOL
    y2 = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid[t13], d, tid[t13], inter, tid["iq1_m"], grids, limit)
    assert torch.equal(y, y2)


@pytest.mark.parametrize("d", [512, 1024, 2048, 3072])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_grouped_experts_routes_as_matrix_rows(mod, dtype, d):
    """IQ2_XXS / IQ1_M experts at 1.5 routes per expert or more take the half-precision form (routes = rows of the matrix-core
    product): one expert with 21 routes (two batches of 16, three of 8 for float32 activations, which go in as two terms),
    experts without routes, an intermediate size that is not a multiple of 256, every activation dtype, rows scaled far
    away from 1 (the rows are brought into half-precision range by a power of two per token)."""
    rng = np.random.default_rng(77)
    e, inter, t = 6, 400, 24           # d: rows of 2, 4, 8 and 12 super-blocks (the gate/up kernel has a form per divisibility of the row)
    w1 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w3 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w2 = _expert_blocks(rng, "iq1_m", e, d, inter)
    idx = np.zeros((t, 2), dtype=np.int64)
    idx[:21, 0] = 0                                         # 21 tokens choose expert 0 first
    idx[21:, 0] = 2
    idx[:, 1] = 1 + 2 * (np.arange(t) % 2) + 2 * (np.arange(t) % 3 == 0)   # second choices over experts 1, 3, 5; expert 4 stays empty
    wts = rng.uniform(0.1, 0.9, size=(t, 2)).astype(np.float32)
    xf = rng.standard_normal((t, d)).astype(np.float32)
    xf[3] *= 3.0e4 if dtype != torch.float16 else 40.0      # (its hidden values) beyond half-precision range before scaling
    xf[5] *= 2.0e-6                                         # half-precision subnormals before scaling
    xf[7] = 0.0
    x = torch.from_numpy(xf).to(DEV).to(dtype)
    _, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), 0, e)
    _, o_toks, o_rws, o_seg = O.group_routes(idx, wts, 0, e)
    counts = np.diff(o_seg)
    assert counts[0] == 21 and counts[4] == 0 and 2 * len(o_toks) >= 3 * e and len(o_toks) <= 8 * e
    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), codebooks.get_iq1_grid_tensor().to(DEV))
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    print(f"case routes as matrix rows {dtype} d={d}", flush=True)
    y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid["iq2_xxs"], d, tid["iq2_xxs"], inter, tid["iq1_m"], grids, 0.0)
    torch.cuda.synchronize()
    route_experts = np.repeat(np.arange(e), counts)
    want = O.moe_forward(x.float().cpu().numpy(), o_toks, o_rws, route_experts, w1, w3, w2, "iq2_xxs", "iq2_xxs", "iq1_m", 0.0)
    got = y.float().cpu().numpy()
    for tok in range(t):                                    # per token: the rows differ by ten orders of magnitude
        if np.abs(want[tok]).max() > 0:
            assert O.rel_l2(got[tok], want[tok]) <= TOL, tok
        else:
            assert not got[tok].any(), tok


def test_grouped_experts_below_the_matrix_row_threshold(mod):
    """Fewer than 1.5 routes per expert: the integer form (one decode per expert, the routes one after the other)."""
    rng = np.random.default_rng(78)
    e, d, inter, topk, t = 12, 512, 512, 2, 7
    w1 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w3 = _expert_blocks(rng, "iq2_xxs", e, inter, d)
    w2 = _expert_blocks(rng, "iq1_m", e, d, inter)
    idx, wts = _route(rng, t, e, topk)
    x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    _, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), 0, e)
    _, o_toks, o_rws, o_seg = O.group_routes(idx, wts, 0, e)
    assert 2 * len(o_toks) < 3 * e
    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), codebooks.get_iq1_grid_tensor().to(DEV))
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    print("case grouped experts below the matrix-row threshold", flush=True)
    y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid["iq2_xxs"], d, tid["iq2_xxs"], inter, tid["iq1_m"], grids, 0.0)
    torch.cuda.synchronize()
    route_experts = np.repeat(np.arange(e), np.diff(o_seg))
    want = O.moe_forward(x.float().cpu().numpy(), o_toks, o_rws, route_experts, w1, w3, w2, "iq2_xxs", "iq2_xxs", "iq1_m", 0.0)
    assert O.rel_l2(y.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("t13,t2,limit", [("iq2_xxs", "iq1_m", 0.0), ("iq2_xxs", "q2_k", 0.7), ("iq1_m", "iq1_m", 0.0)])
def test_grouped_experts_tile_path(mod, t13, t2, limit):
    """Sixteen tokens or more: the routes of every expert go through the MFMA tile kernel as one batch of matmuls
    (some experts idle, one token count that is not a multiple of the tile)."""
    rng = np.random.default_rng(11)
    e, d, inter, topk, t = 10, 768, 512, 3, 77
    w1 = _expert_blocks(rng, t13, e, inter, d)
    w3 = _expert_blocks(rng, t13, e, inter, d)
    w2 = _expert_blocks(rng, t2, e, d, inter)
    idx, wts = _route(rng, t, e + 6, topk)                 # experts 0..15, local window 3..12
    start = 3
    x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    _, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), start, e)
    _, o_toks, o_rws, o_seg = O.group_routes(idx, wts, start, e)
    grids = (codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), codebooks.get_iq1_grid_tensor().to(DEV))
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    if t13 == t2:                                          # one codebook in use: one grid, as the reference takes it
        grids = grids[0] if t13 == "iq2_xxs" else grids[1]
    print(f"case tile path {t13}/{t2} limit={limit}", flush=True)
    y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid[t13], d, tid[t13], inter, tid[t2], grids, limit)
    torch.cuda.synchronize()
    route_experts = np.repeat(np.arange(e), np.diff(o_seg))
    want = O.moe_forward(x.float().cpu().numpy(), o_toks, o_rws, route_experts, w1, w3, w2, t13, t13, t2, limit)
    assert O.rel_l2(y.cpu().numpy(), want) <= TOL
    y2 = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid[t13], d, tid[t13], inter, tid[t2], grids, limit)
    assert torch.equal(y, y2)


@pytest.mark.parametrize("tokens,dim,n_experts,top_k", [(1, 3072, 256, 8), (7, 3072, 256, 8), (3, 1000, 60, 6), (2, 257, 1024, 64), (5, 64, 8, 8),
                                                        (16, 3072, 256, 8), (80, 1024, 60, 6), (256, 3072, 256, 8), (97, 48, 20, 4), (90, 1000, 60, 6),
                                                        (81, 16, 5, 2)])
def test_router_matches_the_reference_statement(mod, tokens, dim, n_experts, top_k):
    """MiniMaxMoE.route on the device: logits against float64, then selection and weights against the oracle evaluated on the
    device's own logits (a float dot in another order may legitimately swap two experts whose scores differ in the last bits,
    so the integer part of the comparison starts from identical inputs), sigmoid with and without bias and the softmax form."""
    rng = np.random.default_rng(tokens * 31 + n_experts)
    x = torch.from_numpy(rng.standard_normal((tokens, dim)).astype(np.float32)).to(DEV)
    gate = torch.from_numpy((rng.standard_normal((n_experts, dim)) / np.sqrt(dim)).astype(np.float32)).to(DEV)
    bias = torch.from_numpy(rng.uniform(-0.3, 0.3, size=n_experts).astype(np.float32)).to(DEV)
    lib = _ffi.load_library()
    for xd in (x, x.to(torch.bfloat16)):
        for b, softmax in ((None, False), (bias, False), (None, True)):
            print(f"case route t={tokens} dim={dim} e={n_experts} k={top_k} {xd.dtype} bias={b is not None} softmax={softmax}", flush=True)
            logits = torch.empty(tokens, n_experts, device=DEV)
            idx = torch.empty(tokens, top_k, dtype=torch.int64, device=DEV)
            w = torch.empty(tokens, top_k, device=DEV)
            st = lib.pllm_moe_route(xd.data_ptr(), {torch.float32: _ffi.DTYPE_F32, torch.bfloat16: _ffi.DTYPE_BF16}[xd.dtype], tokens, dim,
                                    gate.data_ptr(), b.data_ptr() if b is not None else None, n_experts, top_k, int(softmax),
                                    logits.data_ptr(), idx.data_ptr(), w.data_ptr(), torch.cuda.current_stream().cuda_stream)
            assert st == 0
            torch.cuda.synchronize()
            want_logits = xd.double().cpu().numpy() @ gate.double().cpu().numpy().T
            assert O.rel_l2(logits.cpu().numpy(), want_logits) < 1e-6
            want_idx, want_w = O.route_topk(logits.cpu().numpy(), None if b is None else b.cpu().numpy(), top_k, softmax)
            # float32 sigmoid on the device against float64 in the oracle: equal picks unless two scores sit within 1e-6
            got_idx = idx.cpu().numpy()
            if not np.array_equal(got_idx, want_idx):
                l64 = logits.double().cpu().numpy()
                sc = l64 if softmax else 1.0 / (1.0 + np.exp(-l64)) + (0.0 if b is None else b.double().cpu().numpy()[None, :])
                for t in range(tokens):
                    assert sorted(got_idx[t].tolist()) == sorted(want_idx[t].tolist()) or \
                        np.abs(np.sort(np.take(sc[t], got_idx[t])) - np.sort(np.take(sc[t], want_idx[t]))).max() < 1e-6
                    assert np.all(np.diff(np.take(sc[t], got_idx[t])) <= 1e-6)      # descending
            else:
                np.testing.assert_allclose(w.cpu().numpy(), want_w, rtol=2e-6, atol=1e-8)
            assert np.allclose(w.sum(dim=1).cpu().numpy(), 1.0, atol=1e-5)
    # the operator form, and what the reference's own op chain gives
    i2, w2 = mod.moe_route(x, gate, bias, top_k)
    probs = torch.sigmoid(x @ gate.t())
    _, ri = torch.topk(probs + bias, k=top_k, dim=-1)
    rw = torch.gather(probs, -1, ri)
    rw = rw / rw.sum(dim=-1, keepdim=True).clamp_min(1e-20)
    same = (i2 == ri).all(dim=1)
    assert same.float().mean() >= 0.5                      # rows without near-ties agree pick for pick
    assert torch.allclose(w2[same], rw[same], rtol=1e-4, atol=1e-7)
    with pytest.raises(RuntimeError, match="top_k must be in"):
        mod.moe_route(x, gate, None, n_experts + 1)


@pytest.mark.parametrize("tokens,dim,n_experts,top_k", [(1, 3072, 256, 8), (4, 3072, 256, 8), (3, 1000, 60, 6), (2, 260, 1024, 64), (1, 64, 8, 8)])
@pytest.mark.parametrize("x_dtype,out_dtype", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.float16),
                                               (torch.float32, torch.float32)])
def test_router_on_rows_normalized_in_the_same_launch(mod, tokens, dim, n_experts, top_k, x_dtype, out_dtype):
    """ffn_norm + MiniMaxMoE.route of a decode step in two launches: the normalized rows against the oracle's float64
    normalisation (one rounding to the output type), the logits against float64 on the rows the kernel itself wrote, picks and
    weights against the oracle on the device's logits, and all three against the two-operator chain."""
    rng = np.random.default_rng(tokens * 131 + dim + n_experts)
    x = torch.from_numpy((rng.standard_normal((tokens, dim)) * 3.0).astype(np.float32)).to(DEV).to(x_dtype)
    gamma = torch.from_numpy(rng.uniform(0.5, 1.5, size=dim).astype(np.float32)).to(DEV)
    gate = torch.from_numpy((rng.standard_normal((n_experts, dim)) / np.sqrt(dim)).astype(np.float32)).to(DEV)
    bias = torch.from_numpy(rng.uniform(-0.3, 0.3, size=n_experts).astype(np.float32)).to(DEV)
    eps = 1e-6
    lib = _ffi.load_library()
    code = {torch.float32: _ffi.DTYPE_F32, torch.bfloat16: _ffi.DTYPE_BF16, torch.float16: _ffi.DTYPE_F16}
    logits = torch.empty(tokens, n_experts, device=DEV)
    idx = torch.empty(tokens, top_k, dtype=torch.int64, device=DEV)
    w = torch.empty(tokens, top_k, device=DEV)
    normed = torch.empty(tokens, dim, dtype=out_dtype, device=DEV)
    print(f"case route+norm t={tokens} dim={dim} e={n_experts} k={top_k} {x_dtype} -> {out_dtype}", flush=True)
    st = lib.pllm_moe_route_rmsnorm(x.data_ptr(), code[x_dtype], gamma.data_ptr(), eps, normed.data_ptr(), code[out_dtype], tokens, dim,
                                    gate.data_ptr(), bias.data_ptr(), n_experts, top_k, 0, logits.data_ptr(), idx.data_ptr(), w.data_ptr(),
                                    torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    want_rows = O.rms_norm(x.float().cpu().numpy(), gamma.cpu().numpy(), eps)
    ulp = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8, torch.float32: 2.0 ** -22}[out_dtype]
    got_rows = normed.double().cpu().numpy()
    atol = 2.0 ** -25 if out_dtype == torch.float16 else 1e-30          # (fp16 values below 6.1e-5 are spaced 2^-24 apart)
    assert np.all(np.abs(got_rows - want_rows) <= ulp * np.abs(want_rows) * 1.01 + atol)
    want_logits = got_rows @ gate.double().cpu().numpy().T
    assert O.rel_l2(logits.cpu().numpy(), want_logits) < 1e-6
    want_idx, want_w = O.route_topk(logits.cpu().numpy(), bias.cpu().numpy(), top_k, False)
    got_idx = idx.cpu().numpy()
    if np.array_equal(got_idx, want_idx):
        np.testing.assert_allclose(w.cpu().numpy(), want_w, rtol=2e-6, atol=1e-8)
    else:                                                  # two scores within float32 rounding of each other
        sc = 1.0 / (1.0 + np.exp(-logits.double().cpu().numpy())) + bias.double().cpu().numpy()[None, :]
        for t in range(tokens):
            assert np.abs(np.sort(np.take(sc[t], got_idx[t])) - np.sort(np.take(sc[t], want_idx[t]))).max() < 1e-6
    # the two-operator chain: same rows up to one unit of the output type where the row's scale rounded the other way, then
    # the same picks wherever the rows are the same bits
    rows2 = mod.fused_rms_norm_forward(x, gamma, eps, out_dtype=out_dtype)
    assert np.all(np.abs(rows2.double().cpu().numpy() - got_rows) <= 2.0 * ulp * np.abs(got_rows) + 2.0 * atol)
    i2, w2 = mod.moe_route(rows2, gate, bias, top_k)
    for t in range(tokens):
        if torch.equal(rows2[t], normed[t]):
            assert torch.equal(i2[t], idx[t]) and torch.allclose(w2[t], w[t], rtol=1e-5, atol=1e-8)
    # the operator form
    out = mod.moe_route_rmsnorm(x, gamma, eps, gate, bias, top_k, out_dtype=out_dtype)
    assert out is not None and torch.equal(out[0], idx) and torch.equal(out[1], w) and torch.equal(out[2], normed)


def test_router_with_normalisation_declines_what_it_has_no_launch_for(mod):
    gate = torch.randn(16, 4096, device=DEV)
    assert mod.moe_route_rmsnorm(torch.randn(1, 4096, device=DEV), torch.ones(4096, device=DEV), 1e-6, gate, None, 4) is None      # wider than a wave holds
    gate = torch.randn(16, 512, device=DEV)
    assert mod.moe_route_rmsnorm(torch.randn(5, 512, device=DEV), torch.ones(512, device=DEV), 1e-6, gate, None, 4) is None        # more than four rows
    gate = torch.randn(16, 510, device=DEV)
    assert mod.moe_route_rmsnorm(torch.randn(1, 510, device=DEV), torch.ones(510, device=DEV), 1e-6, gate, None, 4) is None        # not whole vectors
    out = mod.moe_route_rmsnorm(torch.randn(2, 512, device=DEV), torch.ones(512, device=DEV), 1e-6, torch.randn(16, 512, device=DEV), None, 4)
    assert out is not None and tuple(out[2].shape) == (2, 512)


def _any_expert_blocks(rng, type_name, e, n, k):
    if type_name in ("iq2_xxs", "iq1_m", "q2_k"):
        return _expert_blocks(rng, type_name, e, n, k)
    bpr = (k + 255) // 256
    if type_name in ("iq2_xs", "iq3_xxs"):
        return C.random_blocks(rng, type_name, e, n, bpr, d_range=(0.002, 0.006))
    enc = {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k, "q6_k": C.quantize_q6_k, "iq4_xs": C.quantize_iq4_xs}[type_name]
    w = (rng.standard_normal((e * n, bpr * 256)) * 0.05).astype(np.float32)
    w[:, k:] = 0.0
    return enc(w).reshape(e, n, bpr, O.BLOCK_BYTES[type_name])


@pytest.mark.parametrize("t13,t2", [("iq2_xs", "iq3_xxs"), ("q4_k", "q5_k"), ("q6_k", "iq4_xs"), ("iq2_xxs", "q4_k"), ("q5_k", "iq1_m")])
@pytest.mark.parametrize("tokens", [1, 5, 40])
def test_experts_in_every_block_type(mod, t13, t2, tokens):
    """The routed operators accept all nine block types like the reference (src/csrc/cuda_kernel.cpp:714-725): types without a
    fused expert kernel run route by route through the dense decode kernels below 16 tokens and as tile matmuls from 16 on."""
    rng = np.random.default_rng(300 + tokens + len(t13) * 7 + len(t2))
    e, d, inter, topk = 6, 512, 768, 3
    w1 = _any_expert_blocks(rng, t13, e, inter, d)
    w3 = _any_expert_blocks(rng, t13, e, inter, d)
    w2 = _any_expert_blocks(rng, t2, e, d, inter)
    idx, wts = _route(rng, tokens, e, topk)
    x = torch.from_numpy(rng.standard_normal((tokens, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    grids = tuple(codebooks.grid_tensor_for_type(t).to(DEV) for t in (0, 2, 5))
    used = sorted({{0: 0, 2: 1, 5: 2, 6: 2}[tid[t]] for t in (t13, t2) if tid[t] in (0, 2, 5, 6)})
    grid_arg = tuple(grids[i] for i in used) if used else torch.empty(0, dtype=torch.int8, device=DEV)
    print(f"case experts {t13}/{t2} tokens={tokens}", flush=True)
    for limit in (0.0, 0.5):
        if tokens == 1:
            y = mod.gguf_moe_single_token_forward(x, torch.from_numpy(idx[0]).to(DEV), torch.from_numpy(wts[0]).to(DEV), dw1, dw3, dw2, limit)
            want = O.moe_forward(x.float().cpu().numpy(), np.zeros(topk, dtype=np.int64), wts[0], idx[0], w1, w3, w2, t13, t13, t2, limit)
        else:
            _, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), 0, e)
            y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid[t13], d, tid[t13], inter, tid[t2], grid_arg, limit)
            _, o_toks, o_rws, o_seg = O.group_routes(idx, wts, 0, e)
            want = O.moe_forward(x.float().cpu().numpy(), o_toks, o_rws, np.repeat(np.arange(e), np.diff(o_seg)), w1, w3, w2, t13, t13, t2, limit)
        torch.cuda.synchronize()
        assert tuple(y.shape) == (tokens, d) and y.dtype == torch.float32
        assert O.rel_l2(y.cpu().numpy(), want) <= TOL, (t13, t2, tokens, limit)


@pytest.mark.parametrize("t2", ["q4_k", "q5_k", "iq4_xs", "q6_k", "q2_k"])
@pytest.mark.parametrize("topk,inter", [(8, 768), (5, 600), (1, 256)])
def test_one_token_down_projection_with_the_routes_as_waves(mod, t2, topk, inter):
    """One token through experts without fused kernels: the down projection forms SiLU(gate) * up * route weight itself, one wave
    per route, and sums the routes in route order (two launches in all).  Every down format of the single-launch kernels, a row
    length that ends inside its last super-block, one to eight routes, with and without the clamp; bitwise repeatable."""
    rng = np.random.default_rng(900 + topk + inter + len(t2))
    e, d = 12, 512
    w1 = _any_expert_blocks(rng, "q4_k", e, inter, d)
    w3 = _any_expert_blocks(rng, "q4_k", e, inter, d)
    if t2 == "q2_k":                                       # (the helper's Q2_K encoder takes whole super-blocks)
        wd = (rng.standard_normal((e * d, (inter + 255) // 256 * 256)) * 0.05).astype(np.float32)
        wd[:, inter:] = 0.0
        w2 = C.quantize_q2_k(wd).reshape(e, d, (inter + 255) // 256, 84)
    else:
        w2 = _any_expert_blocks(rng, t2, e, d, inter)
    idx, wts = _route(rng, 1, e, topk)
    x = torch.from_numpy(rng.standard_normal((1, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    for limit in (0.0, 0.5):
        print(f"case routes as waves q4_k/{t2} topk={topk} inter={inter} limit={limit}", flush=True)
        y = mod.gguf_moe_single_token_forward(x, torch.from_numpy(idx[0]).to(DEV), torch.from_numpy(wts[0]).to(DEV), dw1, dw3, dw2, limit)
        torch.cuda.synchronize()
        want = O.moe_forward(x.float().cpu().numpy(), np.zeros(topk, dtype=np.int64), wts[0], idx[0], w1, w3, w2, "q4_k", "q4_k", t2, limit)
        assert O.rel_l2(y.cpu().numpy(), want) <= TOL, (t2, topk, inter, limit)
        y2 = mod.gguf_moe_single_token_forward(x, torch.from_numpy(idx[0]).to(DEV), torch.from_numpy(wts[0]).to(DEV), dw1, dw3, dw2, limit)
        assert torch.equal(y, y2)


@pytest.mark.parametrize("t13,t2", [("q4_k", "q6_k"), ("iq4_xs", "q5_k")])
def test_experts_with_few_routes_each_at_sixteen_tokens_or_more(mod, t13, t2):
    """Types without fused expert kernels, 16 tokens or more but under four routes per expert on average: the route-by-route path
    (the tile matmuls would decode every touched expert for one or two rows)."""
    rng = np.random.default_rng(812)
    e, d, inter, topk, tokens = 40, 512, 512, 2, 24
    w1 = _any_expert_blocks(rng, t13, e, inter, d)
    w3 = _any_expert_blocks(rng, t13, e, inter, d)
    w2 = _any_expert_blocks(rng, t2, e, d, inter)
    idx, wts = _route(rng, tokens, e, topk)
    assert tokens * topk < 4 * e
    x = torch.from_numpy(rng.standard_normal((tokens, d)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    dw1, dw3, dw2 = (torch.from_numpy(a).to(DEV) for a in (w1, w3, w2))
    tid = O.TYPE_IDS
    _, toks, rws, seg = mod.moe_group_routes(torch.from_numpy(idx).to(DEV), torch.from_numpy(wts).to(DEV), 0, e)
    print(f"case experts few routes each {t13}/{t2}", flush=True)
    y = mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, dw1, dw3, dw2, d, tid[t13], d, tid[t13], inter, tid[t2],
                                             torch.empty(0, dtype=torch.int8, device=DEV), 0.0)
    torch.cuda.synchronize()
    _, o_toks, o_rws, o_seg = O.group_routes(idx, wts, 0, e)
    want = O.moe_forward(x.float().cpu().numpy(), o_toks, o_rws, np.repeat(np.arange(e), np.diff(o_seg)), w1, w3, w2, t13, t13, t2, 0.0)
    assert O.rel_l2(y.cpu().numpy(), want) <= TOL


def test_expert_grid_families_are_checked(mod):
    e, d, inter = 2, 256, 256
    x = torch.randn(2, d, device=DEV)
    toks = torch.zeros(1, dtype=torch.int64, device=DEV)
    rws = torch.ones(1, device=DEV)
    seg = torch.tensor([0, 1, 1], dtype=torch.int32, device=DEV)
    w_xs = torch.zeros(e, inter, 1, 74, dtype=torch.uint8, device=DEV)
    w_xxs = torch.zeros(e, d, 1, 66, dtype=torch.uint8, device=DEV)
    with pytest.raises(RuntimeError, match="cannot mix iq2_xxs with iq2_xs/iq3_xxs"):
        mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, w_xs, w_xs, w_xxs, d, 5, d, 5, inter, 0, codebooks.grid_tensor_for_type(5).to(DEV), 0.0)
    with pytest.raises(RuntimeError, match="packed iq2_xs and iq3_xxs signed grids"):
        mod.gguf_moe_prefill_grouped_forward(x, toks, rws, seg, w_xs, w_xs, torch.zeros(e, d, 1, 98, dtype=torch.uint8, device=DEV), d, 5, d, 5, inter, 6,
                                             codebooks.get_iq2xxs_signed_grid_tensor().to(DEV), 0.0)
