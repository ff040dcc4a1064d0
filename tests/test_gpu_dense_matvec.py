"""GPU parity of the dense decode matvec operators against the float-activation oracle.

Gate: rel-L2 <= 1e-3 on the float32 outputs (the bar the hot path is held to); the kernels carry the
activations as two int8 terms, so the measured distance is around 1e-5.
"""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as O
from pocketllm_amd import block_codec as C, codebooks
from pocketllm_amd.cuda_loader import load_cuda_kernel

pytestmark = pytest.mark.gpu

TOL = 1e-3
ENCODERS = {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k, "q2_k": C.quantize_q2_k, "q6_k": C.quantize_q6_k, "iq4_xs": C.quantize_iq4_xs}


@pytest.fixture(scope="module")
def mod():
    m = load_cuda_kernel()
    assert m is not None, "libpllm_hip.so missing: build it before running GPU tests"
    assert torch.cuda.is_available()
    return m


def _weights(rng, n, k):
    return (rng.standard_normal((n, k)) * 0.02).astype(np.float32)


def _run_dense(mod, type_name, blocks, x_np, x_dtype, k):
    dev = torch.device("cuda:0")
    x = torch.from_numpy(x_np).to(dev).to(x_dtype).contiguous()
    b = torch.from_numpy(blocks).to(dev)
    grid = codebooks.grid_tensor_for_type(O.TYPE_IDS[type_name]).to(dev)
    y = mod.gguf_quant_gemm_forward(x, b, k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
    torch.cuda.synchronize()
    return x.float().cpu().numpy(), y.cpu().numpy()


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k", "q2_k", "q6_k", "iq4_xs"])
@pytest.mark.parametrize("n,k,rows", [(64, 256, 1), (37, 768, 1), (100, 5120, 1), (16, 2048, 3), (9, 17408, 1), (33, 1000, 2), (20, 33024, 2), (48, 20480, 1)])
def test_kquant_matvec_matches_oracle(mod, type_name, n, k, rows):
    rng = np.random.default_rng(1000 + n + k)
    blocks = ENCODERS[type_name](_weights(rng, n, k))
    x_np = rng.standard_normal((rows, k)).astype(np.float32)
    for dt in (torch.bfloat16, torch.float32, torch.float16):
        print(f"case {type_name} n={n} k={k} rows={rows} {dt}", flush=True)
        x_used, y = _run_dense(mod, type_name, blocks, x_np, dt, k)
        want = O.matmul_f(x_used, O.dequant_rows(blocks, type_name, k))
        err = O.rel_l2(y, want)
        assert err <= TOL, (type_name, n, k, rows, dt, err)
        assert err < 2e-4


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k", "q2_k", "q6_k", "iq4_xs", "iq2_xs", "iq3_xxs"])
def test_kquant_matvec_random_bytes(mod, type_name):
    """Uniformly random block bytes reach every scale/min/high-bit code, not only what the encoder emits."""
    rng = np.random.default_rng(77)
    n, bpr = 48, 5
    bb = O.BLOCK_BYTES[type_name]
    blocks = rng.integers(0, 256, size=(n, bpr, bb), dtype=np.uint8)
    for off in {"q2_k": [80, 82], "q6_k": [208], "iq4_xs": [0], "iq2_xs": [0], "iq3_xxs": [0]}.get(type_name, [0, 2]):
        vals = rng.uniform(0.001, 0.05, size=(n, bpr)) * rng.choice([-1.0, 1.0], size=(n, bpr))
        blocks[..., off:off + 2] = vals.astype("<f2").view(np.uint8).reshape(n, bpr, 2)
    x_np = rng.standard_normal((1, bpr * 256)).astype(np.float32)
    x_used, y = _run_dense(mod, type_name, blocks, x_np, torch.float32, bpr * 256)
    want = O.matmul_f(x_used, O.dequant_rows(blocks, type_name))
    assert O.rel_l2(y, want) <= 2e-4


@pytest.mark.parametrize("type_name,n,k", [("q4_k", 5120, 5120), ("q5_k", 5120, 5120), ("q4_k", 17408, 5120), ("q5_k", 17408, 5120)])
def test_kquant_matvec_baseline_shapes(mod, type_name, n, k):
    rng = np.random.default_rng(1002)
    blocks = ENCODERS[type_name](_weights(rng, n, k))
    x_np = rng.standard_normal((1, k)).astype(np.float32)
    print(f"case {type_name} n={n} k={k}", flush=True)
    x_used, y = _run_dense(mod, type_name, blocks, x_np, torch.bfloat16, k)
    want = O.matmul_f(x_used, O.dequant_rows(blocks, type_name, k))
    assert O.rel_l2(y, want) <= 2e-4


def test_reference_output_dtype_is_bf16(mod):
    rng = np.random.default_rng(5)
    blocks = torch.from_numpy(C.quantize_q4_k(_weights(rng, 32, 512))).cuda()
    x = torch.randn(2, 3, 512, device="cuda", dtype=torch.float16)
    y = mod.gguf_quant_gemm_forward(x, blocks, 512, 3, torch.empty(0, dtype=torch.int8, device="cuda"))
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (2, 3, 32)
    y32 = mod.gguf_quant_gemm_prefill_forward(x, blocks, 512, 3, torch.empty(0, dtype=torch.int8, device="cuda"), out_dtype=torch.float32)
    assert torch.equal(y32.to(torch.bfloat16), y)


# ---------------------------------------------------------------------------------------------
# Q8_0
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("n,k,rows", [(96, 64, 2), (8, 256, 1), (130, 4096, 1), (4096, 4096, 1), (24, 1024, 3), (10, 200, 1), (5, 11008, 1)])
def test_q8_0_matvec_matches_oracle(mod, n, k, rows):
    rng = np.random.default_rng(1001 + n)
    blocks = C.pack_q8_0(_weights(rng, n, k))
    x_np = rng.standard_normal((rows, k)).astype(np.float32)
    dev = torch.device("cuda:0")
    b = torch.from_numpy(blocks).to(dev)
    for dt in (torch.float32, torch.bfloat16):
        print(f"case q8_0 n={n} k={k} rows={rows} {dt}", flush=True)
        x = torch.from_numpy(x_np).to(dev).to(dt)
        y = mod.q8_0_gemm_forward(x, b, k, out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks, "q8_0", k))
        err = O.rel_l2(y.cpu().numpy(), want)
        assert err <= 2e-4, (n, k, rows, dt, err)


@pytest.mark.parametrize("n,k,rows,dt", [(1, 256, 1, torch.float32), (7, 256, 1, torch.float16), (1000, 256, 2, torch.bfloat16),
                                         (4099, 1024, 1, torch.float16), (333, 2304, 3, torch.float32), (517, 5120, 1, torch.bfloat16),
                                         (2050, 24576, 1, torch.float32), (61, 17408, 4, torch.bfloat16)])
def test_q8_0_streamed_rows_straddling_steps(mod, n, k, rows, dt):
    """Rows of a multiple of 256 weights on an aligned base take the single-launch kernel, whose 64-pair steps cut
    through row ends: every output row against the oracle, max-abs as well as norm (a misplaced row would hide in a norm)."""
    rng = np.random.default_rng(77 + n)
    blocks = C.pack_q8_0(_weights(rng, n, k))
    dev = torch.device("cuda:0")
    print(f"case q8_0 streamed n={n} k={k} rows={rows} {dt}", flush=True)
    x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(dev).to(dt)
    y = mod.q8_0_gemm_forward(x, torch.from_numpy(blocks).to(dev), k, out_dtype=torch.float32)
    torch.cuda.synchronize()
    want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks, "q8_0", k))
    got = y.cpu().numpy()
    assert O.rel_l2(got, want) <= 2e-4
    assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max()


def test_q8_0_unaligned_activation_rows_fall_back(mod):
    """An activation view that starts 4 bytes into its allocation cannot be read in vector pieces: same result through the other kernels."""
    rng = np.random.default_rng(5)
    n, k = 64, 512
    blocks = C.pack_q8_0(_weights(rng, n, k))
    dev = torch.device("cuda:0")
    store = torch.from_numpy(rng.standard_normal(k + 1).astype(np.float32)).to(dev)
    x = store[1:].view(1, k)
    y = mod.q8_0_gemm_forward(x, torch.from_numpy(blocks).to(dev), k, out_dtype=torch.float32)
    y2 = mod.q8_0_gemm_forward(x.clone(), torch.from_numpy(blocks).to(dev), k, out_dtype=torch.float32)
    torch.cuda.synchronize()
    want = O.matmul_f(x.cpu().numpy(), O.dequant_rows(blocks, "q8_0", k))
    assert O.rel_l2(y.cpu().numpy(), want) <= 2e-4 and O.rel_l2(y2.cpu().numpy(), want) <= 2e-4


def test_q8_0_random_bytes_and_offset_base(mod):
    rng = np.random.default_rng(3)
    n, bpr = 40, 16
    blocks = rng.integers(0, 256, size=(n + 1, bpr, 34), dtype=np.uint8)
    vals = rng.uniform(0.001, 0.05, size=(n + 1, bpr)) * rng.choice([-1.0, 1.0], size=(n + 1, bpr))
    blocks[..., 0:2] = vals.astype("<f2").view(np.uint8).reshape(n + 1, bpr, 2)
    x_np = rng.standard_normal((1, bpr * 32)).astype(np.float32)
    dev = torch.device("cuda:0")
    full = torch.from_numpy(blocks).to(dev)
    x = torch.from_numpy(x_np).to(dev)
    for view, ref in ((full[:n], blocks[:n]), (full[1:], blocks[1:])):   # second view starts 544 B into the allocation
        y = mod.q8_0_gemm_forward(x, view, bpr * 32, out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = O.matmul_f(x_np, O.dequant_rows(ref, "q8_0"))
        assert O.rel_l2(y.cpu().numpy(), want) <= 2e-4


def test_argument_errors_match_reference_messages(mod):
    dev = torch.device("cuda:0")
    x = torch.randn(1, 512, device=dev)
    blocks = torch.zeros(8, 2, 144, dtype=torch.uint8, device=dev)
    grid = torch.empty(0, dtype=torch.int8, device=dev)
    with pytest.raises(RuntimeError, match="inner dimension mismatch"):
        mod.gguf_quant_gemm_forward(x, blocks, 256, 3, grid)
    with pytest.raises(RuntimeError, match="unexpected GGUF block size for type_id"):
        mod.gguf_quant_gemm_forward(x, blocks, 512, 4, grid)
    with pytest.raises(RuntimeError, match="unsupported GGUF quant type_id"):
        mod.gguf_quant_gemm_forward(x, blocks, 512, 11, grid)
    with pytest.raises(RuntimeError, match="blocks do not cover row_elems"):
        mod.gguf_quant_gemm_forward(torch.randn(1, 1024, device=dev), blocks, 1024, 3, grid)
    with pytest.raises(RuntimeError, match="x must be float16, bfloat16, or float32"):
        mod.gguf_quant_gemm_forward(x.double(), blocks, 512, 3, grid)
    with pytest.raises(RuntimeError, match="q8_0 block size must be 34 bytes"):
        mod.q8_0_gemm_forward(x, blocks, 512)


# ---------------------------------------------------------------------------------------------
# codebook types: IQ2_XXS and IQ1_M (random valid blocks, as the reference's own tests build them)
# ---------------------------------------------------------------------------------------------

def _grid_for(type_name, dev):
    from pocketllm_amd import codebooks
    if type_name == "iq2_xxs":
        return codebooks.get_iq2xxs_signed_grid_tensor().to(dev)
    return codebooks.get_iq1_grid_tensor().to(dev)


@pytest.mark.parametrize("type_name", ["iq2_xxs", "iq1_m"])
@pytest.mark.parametrize("n,k,rows", [(16, 256, 1), (50, 768, 1), (1536, 3072, 1), (3072, 1536, 1), (40, 2048, 3), (7, 5120, 1), (21, 1000, 2),
                                      (176, 768, 2), (208, 5120, 1), (64, 14336, 1),
                                      # rows of 12 and of 6 super-blocks (the streamed kernels built for those lengths): fewer rows than
                                      # one chunk of 64, exactly one, and row counts whose last chunk is moved back over its predecessor
                                      (48, 3072, 1), (64, 3072, 2), (80, 3072, 1), (1552, 3072, 2), (32, 1536, 1), (64, 1536, 1), (208, 1536, 2),
                                      (3088, 1536, 1)])
def test_iq_matvec_matches_oracle(mod, type_name, n, k, rows):
    rng = np.random.default_rng(500 + n + k)
    gen = C.random_iq2_xxs if type_name == "iq2_xxs" else C.random_iq1_m
    blocks = gen(rng, n, (k + 255) // 256)
    x_np = rng.standard_normal((rows, k)).astype(np.float32)
    dev = torch.device("cuda:0")
    grid = _grid_for(type_name, dev)
    b = torch.from_numpy(blocks).to(dev)
    for dt in (torch.bfloat16, torch.float32):
        print(f"case {type_name} n={n} k={k} rows={rows} {dt}", flush=True)
        x = torch.from_numpy(x_np).to(dev).to(dt)
        y = mod.gguf_quant_gemm_forward(x, b, k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks, type_name, k))
        err = O.rel_l2(y.cpu().numpy(), want)
        assert err <= 2e-4, (type_name, n, k, rows, dt, err)


@pytest.mark.parametrize("type_name,n,k", [("iq2_xxs", 35200, 3072), ("iq1_m", 70400, 1536)])
def test_iq_matvec_many_rows(mod, type_name, n, k):
    """More row tiles than workgroups in flight: every workgroup walks several chunks of rows, the last ones
    unevenly.  Checked on the first and last rows and a random sample in between."""
    rng = np.random.default_rng(77)
    gen = C.random_iq2_xxs if type_name == "iq2_xxs" else C.random_iq1_m
    blocks = gen(rng, n, k // 256)
    x_np = rng.standard_normal((1, k)).astype(np.float32)
    dev = torch.device("cuda:0")
    print(f"case {type_name} n={n} k={k}", flush=True)
    y = mod.gguf_quant_gemm_forward(torch.from_numpy(x_np).to(dev), torch.from_numpy(blocks).to(dev), k, O.TYPE_IDS[type_name],
                                    _grid_for(type_name, dev), out_dtype=torch.float32)
    torch.cuda.synchronize()
    pick = np.unique(np.concatenate([np.arange(256), np.arange(n - 256, n), rng.integers(0, n, size=4096)]))
    want = O.matmul_f(x_np, O.dequant_rows(blocks[pick], type_name, k))
    assert O.rel_l2(y.cpu().numpy()[:, pick], want) <= 2e-4
    assert torch.isfinite(y).all()


@pytest.mark.parametrize("type_name", ["iq2_xs", "iq3_xxs"])
@pytest.mark.parametrize("n,k,rows", [(16, 256, 1), (50, 768, 2), (1536, 3072, 1), (7, 5120, 1), (64, 14336, 1)])
def test_iq2xs_iq3xxs_matvec_matches_oracle(mod, type_name, n, k, rows):
    rng = np.random.default_rng(900 + n + k)
    blocks = C.random_blocks(rng, type_name, n, (k + 255) // 256)
    x_np = rng.standard_normal((rows, k)).astype(np.float32)
    dev = torch.device("cuda:0")
    print(f"case {type_name} n={n} k={k} rows={rows}", flush=True)
    y = mod.gguf_quant_gemm_forward(torch.from_numpy(x_np).to(dev).to(torch.bfloat16), torch.from_numpy(blocks).to(dev), k, O.TYPE_IDS[type_name],
                                    codebooks.grid_tensor_for_type(O.TYPE_IDS[type_name]).to(dev), out_dtype=torch.float32)
    torch.cuda.synchronize()
    x_used = torch.from_numpy(x_np).to(torch.bfloat16).float().numpy()
    want = O.matmul_f(x_used, O.dequant_rows(blocks, type_name, k))
    assert O.rel_l2(y.cpu().numpy(), want) <= 2e-4, (type_name, n, k, rows)


def test_iq_fully_random_bytes(mod):
    """Every byte random (all scale codes, all sign patterns, both deltas); only the fp16 scale is kept finite."""
    rng = np.random.default_rng(91)
    dev = torch.device("cuda:0")
    for type_name, bb in (("iq2_xxs", 66), ("iq1_m", 56)):
        n, bpr = 64, 6
        gen = C.random_iq2_xxs if type_name == "iq2_xxs" else C.random_iq1_m
        blocks = gen(rng, n, bpr, d_range=(0.001, 0.08))
        x_np = rng.standard_normal((1, bpr * 256)).astype(np.float32)
        y = mod.gguf_quant_gemm_forward(torch.from_numpy(x_np).to(dev), torch.from_numpy(blocks).to(dev), bpr * 256,
                                        O.TYPE_IDS[type_name], _grid_for(type_name, dev), out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = O.matmul_f(x_np, O.dequant_rows(blocks, type_name))
        assert O.rel_l2(y.cpu().numpy(), want) <= 2e-4, type_name


def test_codebook_grid_argument_is_validated(mod):
    dev = torch.device("cuda:0")
    x = torch.randn(1, 256, device=dev)
    blocks = torch.zeros(4, 1, 66, dtype=torch.uint8, device=dev)
    with pytest.raises(RuntimeError, match="256\\*128\\*8 entries for iq2_xxs"):
        mod.gguf_quant_gemm_forward(x, blocks, 256, 0, torch.empty(0, dtype=torch.int8, device=dev))
    with pytest.raises(RuntimeError, match="2048\\*8 entries for iq1_m"):
        mod.gguf_quant_gemm_forward(x, torch.zeros(4, 1, 56, dtype=torch.uint8, device=dev), 256, 2, torch.empty(0, dtype=torch.int8, device=dev))
    for tid, bb in ((5, 74), (6, 98)):
        with pytest.raises(RuntimeError, match="packed iq2_xs and iq3_xxs signed grids"):
            mod.gguf_quant_gemm_forward(x, torch.zeros(4, 1, bb, dtype=torch.uint8, device=dev), 256, tid,
                                        codebooks.get_iq2xs_signed_grid_tensor().to(dev))
    with pytest.raises(RuntimeError, match="cannot mix iq1_m with iq2_xs/iq3_xxs"):
        mod.gguf_quant_gemm_pair_forward(x, torch.zeros(4, 1, 56, dtype=torch.uint8, device=dev), 256, 2,
                                         torch.zeros(4, 1, 74, dtype=torch.uint8, device=dev), 256, 5, codebooks.get_iq1_grid_tensor().to(dev))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_activation_image_holds_two_int8_terms_per_value(mod, dtype):
    """The image the matvec kernels read: per 32 values x ~= xs * (hi + lo / 254) with xs = amax / 127, plus exact-order float sums
    of every 16 and 32 values.  Checked against the definition (not against another quantizer): reconstruction error below
    amax / 127 / 254 * 0.51 per value, scale and sums as stated, padding zero."""
    rng = np.random.default_rng(77)
    dev = torch.device("cuda:0")
    k, bpr = 1000, 4
    x_np = rng.standard_normal((3, k)).astype(np.float32) * np.array([[1.0], [1e-3], [300.0]], dtype=np.float32)
    x_np[0, 64:96] = 0.0                                       # an all-zero group
    x = torch.from_numpy(x_np).to(dev).to(dtype)
    xf = x.float().cpu().numpy()
    image = mod.quantize_activations(x, bpr).cpu().numpy()
    kpad = bpr * 256
    xp = np.zeros((3, kpad), dtype=np.float32)
    xp[:, :k] = xf
    hi = image[:, :kpad].view(np.int8).astype(np.float32)
    lo = image[:, kpad:2 * kpad].view(np.int8).astype(np.float32)
    gs = image[:, 2 * kpad:2 * kpad + kpad // 32 * 8].copy().view(np.float32).reshape(3, kpad // 32, 2)
    sum16 = image[:, 2 * kpad + kpad // 32 * 8:2 * kpad + kpad // 32 * 8 + kpad // 16 * 4].copy().view(np.float32)
    amax = np.abs(xp).reshape(3, -1, 32).max(axis=2)
    np.testing.assert_allclose(gs[..., 0] * 254.0, amax / 127.0, rtol=3e-7)
    recon = (gs[..., 0:1] * (hi.reshape(3, -1, 32) * 254.0 + lo.reshape(3, -1, 32))).reshape(3, kpad)
    assert np.all(np.abs(recon - xp) <= np.repeat(amax, 32, axis=1) / 127.0 / 254.0 * 0.51 + 1e-30)
    assert np.all(np.abs(hi) <= 127) and np.all(np.abs(lo) <= 127)
    np.testing.assert_allclose(sum16, xp.reshape(3, -1, 16).sum(axis=2), rtol=0, atol=np.abs(xp).max() * 4e-6)
    np.testing.assert_allclose(gs[..., 1], xp.reshape(3, -1, 32).sum(axis=2), rtol=0, atol=np.abs(xp).max() * 8e-6)
    assert not hi[:, k:].any() and not lo[:, k:].any()


def _quantizer_cases(rng, k):
    """Rows that stress the 32-value quantizer: plain, tiny, huge, an all-zero group, values that sit on or next to rounding
    ties of x / scale (half-integer multiples of amax / 127, one float32 step above and below), and a group whose largest
    value is the only non-zero one."""
    rows = [rng.standard_normal(k), rng.standard_normal(k) * 1e-6, rng.standard_normal(k) * 3e4, rng.standard_normal(k)]
    rows[3][64:96] = 0.0
    rows[3][128:160] = 0.0
    rows[3][130] = -2.5
    ties = np.empty(k, dtype=np.float32)
    for g in range(k // 32):
        amax = np.float32(rng.uniform(0.01, 50.0))
        scale = np.float32(amax / np.float32(127.0))
        half = (rng.integers(-126, 126, size=32).astype(np.float32) + np.float32(0.5)) * scale
        nudge = rng.integers(-1, 2, size=32)
        half = np.where(nudge > 0, np.nextafter(half, np.float32(np.inf)), np.where(nudge < 0, np.nextafter(half, np.float32(-np.inf)), half))
        half[0] = amax
        ties[32 * g:32 * g + 32] = half
    rows.append(ties)
    return np.stack(rows).astype(np.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_activation_image_first_term_equals_the_reference_quantizer(mod, dtype):
    """The first int8 term and the scale of the image are the reference's 32-value activation quantizer
    (src/csrc/cuda_kernel_impl.cu:7090-7117, restated as oracle.q8_1_quantize): codes equal bit for bit, the stored figure is
    float32(scale) * float32(1 / 254) bit for bit.  Only an all-zero group differs by design: scale 0 here, 1e-8 there, codes 0
    in both."""
    rng = np.random.default_rng(79)
    dev = torch.device("cuda:0")
    k, bpr = 2048, 8
    x_np = _quantizer_cases(rng, k)
    if dtype == torch.float16:
        x_np = np.clip(x_np, -6e4, 6e4)
    x = torch.from_numpy(x_np).to(dev).to(dtype)
    xf = x.float().cpu().numpy()
    rows = xf.shape[0]
    want_q, want_s = O.q8_1_quantize(xf, 32)
    zero = np.abs(xf).reshape(rows, -1, 32).max(axis=2) == 0
    assert zero.sum() >= 1
    image = mod.quantize_activations(x, bpr).cpu().numpy()
    hi = image[:, :k].view(np.int8)
    gs = image[:, 2 * k:2 * k + k // 32 * 8].copy().view(np.float32).reshape(rows, k // 32, 2)
    np.testing.assert_array_equal(hi, want_q)
    want_gs = np.where(zero, np.float32(0.0), want_s * np.float32(1.0 / 254.0)).astype(np.float32)
    np.testing.assert_array_equal(gs[..., 0].view(np.uint32), want_gs.view(np.uint32))


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k"])
@pytest.mark.parametrize("n,k,rows", [(40, 768, 3), (16, 256, 16), (100, 5120, 7), (9000, 1280, 5), (33, 17408, 16), (70, 2304, 11)])
def test_three_to_sixteen_rows_as_matrix_core_operands(mod, type_name, n, k, rows):
    """3 - 16 rows of bf16 / fp16 activations of a whole number of super-blocks: one pass over the weights with the rows as
    half-precision matrix-core operands, codes exact, float32 sums.  Weight rows that do not fill a tile, many tiles of short rows
    (one tile per wave) and long rows or few tiles (two), more blocks per wave than a pass holds, random bytes in every code field."""
    rng = np.random.default_rng(500 + n + rows)
    bpr = k // 256
    blocks = rng.integers(0, 256, size=(n, bpr, O.BLOCK_BYTES[type_name]), dtype=np.uint8)
    for off in (0, 2):
        vals = rng.uniform(0.001, 0.05, size=(n, bpr)) * rng.choice([-1.0, 1.0], size=(n, bpr))
        blocks[..., off:off + 2] = vals.astype("<f2").view(np.uint8).reshape(n, bpr, 2)
    dev = torch.device("cuda:0")
    w = torch.from_numpy(blocks).to(dev)
    empty = torch.empty(0, dtype=torch.int8, device=dev)
    for dt in (torch.bfloat16, torch.float16):
        print(f"case rows as operands {type_name} n={n} k={k} rows={rows} {dt}", flush=True)
        x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(dev).to(dt)
        y = mod.gguf_quant_gemm_forward(x, w, k, O.TYPE_IDS[type_name], empty, out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks, type_name, k))
        got = y.cpu().numpy()
        assert O.rel_l2(got, want) <= 2e-6
        assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k", "q2_k", "q6_k", "iq4_xs"])
def test_single_launch_kernels_multiply_the_power_of_two_image(mod, type_name):
    """One activation row through the single-launch decode kernels: the result is the float statement of the operator applied to
    the activations rounded onto a power-of-two scale per 32 values (oracle.pow2_image: x ~= 2^(E - 13) q, |q| <= 2^14), the dots
    and the offset terms both taken from that image.  Against the image the distance is float32 summation error only (a wrong
    scale, rounding mode or sum would show at 1e-5 or more); N(0, 1) activations in bf16 lie on the image almost everywhere, so
    there the result is also close to the unrounded operator."""
    rng = np.random.default_rng(4242)
    for n, k in ((64, 5120), (48, 20480), (33, 1000)):
        bpr = (k + 255) // 256
        if type_name in ("q4_k", "q5_k", "q2_k"):
            blocks = ENCODERS[type_name](np.pad(_weights(rng, n, k), ((0, 0), (0, bpr * 256 - k))))
        else:
            blocks = C.random_blocks(rng, type_name, n, bpr)
        w = O.dequant_rows(blocks, type_name, k)
        # a wide range of magnitudes inside every group, and a group of zeros
        x_np = (rng.standard_normal((1, k)) * np.exp(rng.uniform(-6.0, 2.0, size=(1, k)))).astype(np.float32)
        x_np[0, 64:96] = 0.0
        for dt in (torch.float32, torch.bfloat16, torch.float16):
            print(f"case image {type_name} n={n} k={k} {dt}", flush=True)
            x_used, y = _run_dense(mod, type_name, blocks, x_np, dt, k)
            pad = (-k) % 32
            image = O.pow2_image(np.pad(x_used, ((0, 0), (0, pad))))[:, :k]
            want_image = O.matmul_f(image, w)
            err = O.rel_l2(y, want_image)
            assert err <= 3e-6, (type_name, n, k, dt, err)
        # N(0, 1) activations in bf16: nearly all of them lie on the image
        x_used, y = _run_dense(mod, type_name, blocks, rng.standard_normal((1, k)).astype(np.float32), torch.bfloat16, k)
        assert O.rel_l2(y, O.matmul_f(x_used, w)) <= 2e-5


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k", "q2_k", "q6_k", "iq4_xs", "iq2_xxs", "iq1_m", "iq2_xs", "iq3_xxs"])
def test_few_row_calls_equal_the_prequantized_path(mod, type_name):
    """Calls of a few rows may quantize the activations inside the matvec kernel; the result is the same bits as quantizing ahead
    for the kernels that build the pre-pass image themselves (the codebook formats).  Q4_K, Q5_K, Q2_K, Q6_K and IQ4_XS quantize a
    slice per wave on a power-of-two scale (x ~= 2^(E - 13) (256 hi + lo): exact for bf16 values within 2^-6 of their group's
    largest, error <= amax 2^-15 otherwise), another image of the same two-term form: equal to the pre-pass path within that
    bound and at least as close to the float statement of the operator."""
    rng = np.random.default_rng(78)
    dev = torch.device("cuda:0")
    tid = O.TYPE_IDS[type_name]
    for n, k, rows in ((48, 5120, 1), (130, 1002, 3), (16, 17408, 2), (20, 256, 4)):
        bpr = (k + 255) // 256
        if type_name in ("q4_k", "q5_k", "q2_k"):
            enc = {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k, "q2_k": C.quantize_q2_k}[type_name]
            blocks = enc(np.pad(_weights(rng, n, k), ((0, 0), (0, bpr * 256 - k))))
        elif type_name in ("iq2_xxs", "iq1_m"):
            blocks = (C.random_iq2_xxs if type_name == "iq2_xxs" else C.random_iq1_m)(rng, n, bpr)
        else:
            blocks = C.random_blocks(rng, type_name, n, bpr)
        blocks = torch.from_numpy(blocks).to(dev)
        for dt in (torch.bfloat16, torch.float32, torch.float16):
            x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(dev).to(dt)
            print(f"case few-row {type_name} n={n} k={k} rows={rows} {dt}", flush=True)
            y = mod.gguf_quant_gemm_forward(x, blocks, k, tid, codebooks.grid_tensor_for_type(tid).to(dev), out_dtype=torch.float32)
            y_pre = mod.gguf_quant_gemm_prequantized(mod.quantize_activations(x, bpr), blocks, tid, out_dtype=torch.float32)
            if type_name in ("q4_k", "q5_k", "q2_k", "q6_k", "iq4_xs") and not (type_name in ("q4_k", "q5_k") and rows >= 3 and dt != torch.float32 and k % 256 == 0):
                want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks.cpu().numpy(), type_name, k))
                err, err_pre = O.rel_l2(y.cpu().numpy(), want), O.rel_l2(y_pre.cpu().numpy(), want)
                assert O.rel_l2(y.cpu().numpy(), y_pre.cpu().numpy()) <= 1e-4
                assert err <= (2e-5 if dt == torch.bfloat16 else 1e-4), (err, err_pre)
            elif type_name in ("q4_k", "q5_k") and rows >= 3 and dt != torch.float32 and k % 256 == 0:
                # three rows or more of 16-bit activations go in unquantized (half-precision matrix-core operands): closer to the
                # float statement of the operator than the two-term int8 image, not the same bits
                want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks.cpu().numpy(), type_name, k))
                assert O.rel_l2(y.cpu().numpy(), want) <= 2e-6 and O.rel_l2(y.cpu().numpy(), y_pre.cpu().numpy()) <= 1e-4
            else:
                assert torch.equal(y, y_pre)


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k", "iq4_xs", "q6_k", "q2_k"])
@pytest.mark.parametrize("n,k", [(17408, 5120), (1041, 1000), (16, 256), (300, 17408), (5120, 5120)])
def test_two_to_four_rows_in_one_pass_equal_single_row_calls(mod, type_name, n, k):
    """A call of two to four rows (to eight for Q4_K, Q5_K and IQ4_XS, and for Q6_K matrices of up to 48 Mi weights) takes all its rows through every block a wave fetches and
    unpacks (one launch, one pass over the weights, whatever the matrix size): each row goes through the same slice image and the
    same products in the same order as in a call of its own, so the results are the same bits; and they meet the float statement
    like the single-row call.  (Three rows or more of 16-bit Q4_K / Q5_K activations in whole super-blocks go to the kernel that
    takes them unquantized instead: closer to the float statement, not the same bits.)"""
    rng = np.random.default_rng(n + k)
    dev = torch.device("cuda:0")
    tid = O.TYPE_IDS[type_name]
    bpr = (k + 255) // 256
    if type_name in ("iq4_xs", "q6_k"):
        blocks = C.random_blocks(rng, type_name, n, bpr)
    elif type_name == "q2_k":
        blocks = rng.integers(0, 256, size=(n, bpr, 84), dtype=np.uint8)
        blocks[..., 80:82] = np.frombuffer(np.float16(0.01).tobytes(), dtype=np.uint8)
        blocks[..., 82:84] = np.frombuffer(np.float16(0.005).tobytes(), dtype=np.uint8)
    else:
        blocks = rng.integers(0, 256, size=(n, bpr, 144 if type_name == "q4_k" else 176), dtype=np.uint8)
        blocks[..., 0:2] = np.frombuffer(np.float16(0.01).tobytes(), dtype=np.uint8)
        blocks[..., 2:4] = np.frombuffer(np.float16(0.005).tobytes(), dtype=np.uint8)
    dblocks = torch.from_numpy(blocks).to(dev)
    grid = codebooks.grid_tensor_for_type(tid).to(dev)
    rows_w = rng.choice(n, size=min(n, 48), replace=False)
    ref_w = O.dequant_rows(blocks[rows_w], type_name, k)
    most = 8 if type_name in ("q4_k", "q5_k", "iq4_xs") or (type_name == "q6_k" and n * bpr * 256 <= 48 << 20) else 4
    for rows in (2, 3, 4, 5, 8):
        if rows > most:
            continue
        for dt in (torch.bfloat16, torch.float32, torch.float16):
            x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(dev).to(dt)
            x[1] *= 37.0
            print(f"case {rows} rows {type_name} n={n} k={k} {dt}", flush=True)
            y = mod.gguf_quant_gemm_forward(x, dblocks, k, tid, grid, out_dtype=torch.float32)
            singles = [mod.gguf_quant_gemm_forward(x[r:r + 1].contiguous(), dblocks, k, tid, grid, out_dtype=torch.float32) for r in range(rows)]
            torch.cuda.synchronize()
            assert tuple(y.shape) == (rows, n)
            unquantized = type_name in ("q4_k", "q5_k") and rows >= 3 and dt != torch.float32 and k % 256 == 0
            if not unquantized:
                for r in range(rows):
                    assert torch.equal(y[r], singles[r][0]), (rows, r, dt)
            want = O.matmul_f(x.float().cpu().numpy(), ref_w)
            got = y.cpu().numpy()[:, rows_w]
            for r in range(rows):
                # (random blocks: scales and mins of every size cancel against each other, which magnifies the image's rounding)
                assert O.rel_l2(got[r], want[r]) <= (1e-4 if dt == torch.bfloat16 else 1e-3), (dt, r, O.rel_l2(got[r], want[r]))
            y16 = mod.gguf_quant_gemm_forward(x, dblocks, k, tid, grid)
            assert torch.equal(y16, y.to(y16.dtype))


@pytest.mark.parametrize("type_name", ["iq2_xxs", "iq1_m"])
@pytest.mark.parametrize("n,k", [(17408, 5120), (8192, 3072), (6144, 1536), (48, 256), (1041, 1000), (4112, 7168)])
def test_codebook_two_to_four_rows_decode_every_block_once(mod, type_name, n, k):
    """Two rows of IQ2_XXS / IQ1_M on a matrix of 24 Mi weights or more that streams through LDS (whole 16-row tiles, 16-byte
    aligned): every block is decoded once and multiplied into the images of both rows.  Same activation images and integer dots
    as in single-row calls, the scales multiplied in another order: within float rounding of them.  Other shapes and three or
    four rows run one grid row per activation row (or, IQ1_M at four rows on the largest matrix, the tile kernel, which rounds
    weights and activations to fp16).  All meet the float statement of the operator."""
    rng = np.random.default_rng(n * 3 + k)
    dev = torch.device("cuda:0")
    tid = O.TYPE_IDS[type_name]
    bpr = (k + 255) // 256
    blocks = (C.random_iq2_xxs if type_name == "iq2_xxs" else C.random_iq1_m)(rng, n, bpr)
    dblocks = torch.from_numpy(blocks).to(dev)
    grid = codebooks.grid_tensor_for_type(tid).to(dev)
    rows_w = rng.choice(n, size=min(n, 48), replace=False)
    ref_w = O.dequant_rows(blocks[rows_w], type_name, k)
    for rows in (2, 3, 4):
        for dt in (torch.float16, torch.float32, torch.bfloat16):
            x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(dev).to(dt)
            x[1] *= 37.0
            print(f"case {rows} rows {type_name} n={n} k={k} {dt}", flush=True)
            y = mod.gguf_quant_gemm_forward(x, dblocks, k, tid, grid, out_dtype=torch.float32)
            singles = torch.cat([mod.gguf_quant_gemm_forward(x[r:r + 1].contiguous(), dblocks, k, tid, grid, out_dtype=torch.float32) for r in range(rows)])
            torch.cuda.synchronize()
            assert tuple(y.shape) == (rows, n)
            tiles = type_name == "iq1_m" and rows == 4 and n * k >= 64 << 20
            for r in range(rows):
                assert O.rel_l2(y[r].cpu().numpy(), singles[r].cpu().numpy()) <= (1e-3 if tiles else 1e-6), (rows, r, dt)
            want = O.matmul_f(x.float().cpu().numpy(), ref_w)
            got = y.cpu().numpy()[:, rows_w]
            for r in range(rows):
                assert O.rel_l2(got[r], want[r]) <= (1e-3 if tiles else 1e-4), (dt, r, O.rel_l2(got[r], want[r]))
            if tiles:
                continue                     # (the residual form declines the tile kernel's row counts)
            # the residual form adds the same product into y
            y0 = torch.from_numpy(rng.standard_normal((rows, n)).astype(np.float32)).to(dev)
            acc = y0.clone()
            mod.gguf_quant_gemm_accumulate_forward(x, dblocks, k, tid, grid, acc)
            assert torch.allclose(acc, y0 + y, rtol=1e-6, atol=1e-6 * float(y.abs().max()))


@pytest.mark.parametrize("type_name", ["iq2_xs", "iq3_xxs"])
@pytest.mark.parametrize("n,k", [(17408, 5120), (8192, 3072), (8200, 1000), (8192, 8192), (4096, 3072), (8192, 8448)])
def test_two_rows_of_iq2_xs_iq3_xxs_in_one_pass_equal_single_row_calls(mod, type_name, n, k):
    """Two rows of IQ2_XS / IQ3_XXS on a matrix of 8192 rows or more and rows of up to 32 super-blocks: both activation images
    in LDS, every block's codes looked up once; per row the same image, products and float steps as a single-row call, so the
    same bits (ragged rows and a last tile that is not whole included).  Shorter or wider matrices and three rows run one grid
    row per activation row: the same bits too.  The residual form adds the same product."""
    rng = np.random.default_rng(n + 7 * k)
    dev = torch.device("cuda:0")
    tid = O.TYPE_IDS[type_name]
    bpr = (k + 255) // 256
    blocks = C.random_blocks(rng, type_name, n, bpr)
    dblocks = torch.from_numpy(blocks).to(dev)
    grid = codebooks.grid_tensor_for_type(tid).to(dev)
    rows_w = rng.choice(n, size=48, replace=False)
    rows_w[0] = n - 1
    ref_w = O.dequant_rows(blocks[rows_w], type_name, k)
    for rows in (2, 3):
        for dt in (torch.float16, torch.float32, torch.bfloat16):
            x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(dev).to(dt)
            x[1] *= 37.0
            print(f"case {rows} rows {type_name} n={n} k={k} {dt}", flush=True)
            y = mod.gguf_quant_gemm_forward(x, dblocks, k, tid, grid, out_dtype=torch.float32)
            singles = torch.cat([mod.gguf_quant_gemm_forward(x[r:r + 1].contiguous(), dblocks, k, tid, grid, out_dtype=torch.float32) for r in range(rows)])
            torch.cuda.synchronize()
            assert tuple(y.shape) == (rows, n) and torch.equal(y, singles)
            want = O.matmul_f(x.float().cpu().numpy(), ref_w)
            got = y.cpu().numpy()[:, rows_w]
            for r in range(rows):
                assert O.rel_l2(got[r], want[r]) <= 1e-4, (dt, r, O.rel_l2(got[r], want[r]))
            y0 = torch.from_numpy(rng.standard_normal((rows, n)).astype(np.float32)).to(dev)
            acc = y0.clone()
            mod.gguf_quant_gemm_accumulate_forward(x, dblocks, k, tid, grid, acc)
            assert torch.equal(acc, y0 + y)
            y16 = mod.gguf_quant_gemm_forward(x, dblocks, k, tid, grid)
            assert torch.equal(y16, y.to(y16.dtype))


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k", "q2_k", "q6_k", "iq4_xs", "iq2_xxs", "iq1_m", "iq2_xs", "iq3_xxs"])
def test_accumulate_adds_the_product_to_y(mod, type_name):
    """The residual form y += W x: equal to the plain operator's float32 product plus the old y, rounded once to y's type,
    for the in-kernel and the pre-pass activation paths, the streamed and the tile-frame kernels; rows of the tile kernel
    take the composed path of the wrapper."""
    rng = np.random.default_rng(91)
    dev = torch.device("cuda:0")
    tid = O.TYPE_IDS[type_name]
    grid = codebooks.grid_tensor_for_type(tid).to(dev)
    for n, k, rows in ((48, 5120, 1), (130, 1002, 3), (1536, 3072, 2), (64, 512, 7), (40, 768, 20)):
        bpr = (k + 255) // 256
        if type_name in ("q4_k", "q5_k", "q2_k"):
            enc = {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k, "q2_k": C.quantize_q2_k}[type_name]
            blocks = enc(np.pad(_weights(rng, n, k), ((0, 0), (0, bpr * 256 - k))))
        elif type_name in ("iq2_xxs", "iq1_m"):
            blocks = (C.random_iq2_xxs if type_name == "iq2_xxs" else C.random_iq1_m)(rng, n, bpr)
        else:
            blocks = C.random_blocks(rng, type_name, n, bpr)
        blocks = torch.from_numpy(blocks).to(dev)
        x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(dev).to(torch.bfloat16)
        prod = mod.gguf_quant_gemm_forward(x, blocks, k, tid, grid, out_dtype=torch.float32)
        for ydt in (torch.float32, torch.bfloat16, torch.float16):
            print(f"case accumulate {type_name} n={n} k={k} rows={rows} {ydt}", flush=True)
            y0 = torch.from_numpy(rng.standard_normal((rows, n)).astype(np.float32)).to(dev).to(ydt)
            y = y0.clone()
            out = mod.gguf_quant_gemm_accumulate_forward(x, blocks, k, tid, grid, y)
            torch.cuda.synchronize()
            assert out is y
            want = (y0.float() + prod).to(ydt)
            assert torch.equal(y, want), (n, k, rows, ydt, (y.float() - want.float()).abs().max().item())
    with pytest.raises(RuntimeError, match="leading shape"):
        mod.gguf_quant_gemm_accumulate_forward(x, blocks, k, tid, grid, torch.zeros(rows, n + 1, device=dev))


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k", "q6_k", "iq4_xs", "iq2_xxs", "iq1_m", "iq3_xxs", "q2_k"])
def test_multi_projection_equals_separate_calls(mod, type_name):
    """q / k / v style projections of one activation tensor in one launch (one call each for Q2_K): the results of the separate
    operators, with and without the fused RMS normalisation, heights in any order."""
    rng = np.random.default_rng(93)
    dev = torch.device("cuda:0")
    tid = O.TYPE_IDS[type_name]
    grid = codebooks.grid_tensor_for_type(tid).to(dev)
    for k, heights, rows in ((3072, (6144, 1024, 1024), 1), (1002, (40, 130, 16, 7), 3), (512, (33,), 2), (768, (64, 200), 20), (1024, (48, 200), 5)):
        bpr = (k + 255) // 256
        mats = []
        for n in heights:
            if type_name in ("q4_k", "q5_k", "q2_k"):
                enc = {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k, "q2_k": C.quantize_q2_k}[type_name]
                mats.append(torch.from_numpy(enc(np.pad(_weights(rng, n, k), ((0, 0), (0, bpr * 256 - k))))).to(dev))
            elif type_name in ("iq2_xxs", "iq1_m"):
                mats.append(torch.from_numpy((C.random_iq2_xxs if type_name == "iq2_xxs" else C.random_iq1_m)(rng, n, bpr)).to(dev))
            else:
                mats.append(torch.from_numpy(C.random_blocks(rng, type_name, n, bpr)).to(dev))
        gamma = torch.from_numpy(rng.uniform(0.5, 1.5, size=k).astype(np.float32)).to(dev)
        for dt in (torch.bfloat16, torch.float32):
            x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(dev).to(dt)
            print(f"case multi {type_name} k={k} heights={heights} rows={rows} {dt}", flush=True)
            got = mod.gguf_quant_gemm_multi_forward(x, mats, k, tid, grid, out_dtype=torch.float32)
            want = [mod.gguf_quant_gemm_forward(x, m, k, tid, grid, out_dtype=torch.float32) for m in mats]
            assert len(got) == len(want)
            # The joint launch and the single calls may split a row's blocks over different numbers of waves (and IQ2_XXS / IQ1_M
            # single calls may stream whole tiles), which sums in another order; with the normalisation the row's sum of squares
            # is summed in another order too, which can move an activation code by one step.  A wrong matrix, height or output
            # would be an error of order one.
            # (five to eight rows: the single calls of Q4_K / Q5_K / IQ4_XS / small Q6_K matrices quantize inside their kernel, on the power-of-two scale,
            # the joint call ahead of it: two images of the same rows, each within ~1e-4 of the float statement for float32 rows)
            same_image = not (5 <= rows <= 8 and type_name in ("q4_k", "q5_k", "iq4_xs", "q6_k"))
            for a, b in zip(got, want):
                assert a.shape == b.shape and O.rel_l2(a.cpu().numpy(), b.cpu().numpy()) <= (2e-6 if same_image else 2e-4)
            got = mod.gguf_quant_gemm_multi_forward(x, mats, k, tid, grid, norm_weight=gamma, eps=1e-5, out_dtype=torch.float32)
            want = [mod.gguf_quant_gemm_rmsnorm_forward(x, gamma, 1e-5, m, k, tid, grid, out_dtype=torch.float32) for m in mats]
            for a, b in zip(got, want):
                assert a.shape == b.shape and O.rel_l2(a.cpu().numpy(), b.cpu().numpy()) <= 5e-5
    bb = mats[0].size(2)
    one, two = torch.zeros(8, 1, bb, dtype=torch.uint8, device=dev), torch.zeros(8, 2, bb, dtype=torch.uint8, device=dev)
    with pytest.raises(RuntimeError, match="same number of blocks per row"):
        mod.gguf_quant_gemm_multi_forward(torch.zeros(1, 256, device=dev), [one, two], 256, tid, grid)


@pytest.mark.parametrize("type_name", ["q4_k", "q6_k", "iq2_xxs"])
def test_swiglu_image_feeds_the_down_projection(mod, type_name):
    """SiLU(gate) * up quantized in one launch, then the down projection on the image with the residual added: against the chain of
    separate operators on the same float values (image bit-equal when the product is formed identically), and against the float oracle."""
    rng = np.random.default_rng(95)
    dev = torch.device("cuda:0")
    tid = O.TYPE_IDS[type_name]
    for inter, d, rows, limit in ((1536, 96, 1, 0.0), (1002, 40, 3, 0.0), (2048, 64, 2, 1.5)):
        bpr = (inter + 255) // 256
        if type_name == "q4_k":
            wd = C.quantize_q4_k(np.pad(_weights(rng, d, inter), ((0, 0), (0, bpr * 256 - inter))))
        elif type_name == "q6_k":
            wd = C.random_blocks(rng, type_name, d, bpr)
        else:
            wd = C.random_iq2_xxs(rng, d, bpr)
        wd_dev = torch.from_numpy(wd).to(dev)
        g_np = rng.standard_normal((rows, inter)).astype(np.float32) * 2
        u_np = rng.standard_normal((rows, inter)).astype(np.float32) * 2
        for gu_dt, round_dt in ((torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.float16)):
            print(f"case swiglu image {type_name} inter={inter} d={d} rows={rows} limit={limit} {gu_dt} round {round_dt}", flush=True)
            g, u = torch.from_numpy(g_np).to(dev).to(gu_dt), torch.from_numpy(u_np).to(dev).to(gu_dt)
            image = mod.swiglu_quantize_activations(g, u, bpr, swiglu_limit=limit, round_dtype=round_dt)
            gf, uf = g.float().cpu().numpy().astype(np.float64), u.float().cpu().numpy().astype(np.float64)
            if limit > 0:
                uf, gf = np.clip(uf, -limit, limit), np.minimum(gf, limit)
            h64 = gf / (1.0 + np.exp(-gf)) * uf
            h = torch.from_numpy(h64.astype(np.float32)).to(round_dt)              # the chain's activation tensor
            y0 = torch.from_numpy(rng.standard_normal((rows, d)).astype(np.float32)).to(dev)
            y = mod.gguf_quant_gemm_prequantized(image, wd_dev, tid, accumulate_into=y0.clone())
            torch.cuda.synchronize()
            want = y0.cpu().numpy() + O.matmul_f(h.float().numpy(), O.dequant_rows(wd, type_name, inter))
            assert O.rel_l2(y.cpu().numpy(), want) <= 1e-3
            # the same through the separate operators: identical up to the last-bit differences of the device's expf
            chain = y0 + mod.gguf_quant_gemm_forward(h.to(dev), wd_dev, inter, tid, codebooks.grid_tensor_for_type(tid).to(dev), out_dtype=torch.float32)
            assert O.rel_l2(y.cpu().numpy(), chain.cpu().numpy()) <= 2e-4
            plain = mod.gguf_quant_gemm_prequantized(image, wd_dev, tid, out_dtype=torch.float32)
            assert torch.equal((y0 + plain), y)
    with pytest.raises(RuntimeError, match="agree in shape"):
        mod.swiglu_quantize_activations(g, u[:, :-1].contiguous(), bpr)
