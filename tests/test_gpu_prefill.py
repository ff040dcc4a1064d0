"""GPU parity of the prefill matmul (tile GEMM on f16 MFMA with decoded tiles) against the float oracle."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as O
from pocketllm_amd import block_codec as C, codebooks
from pocketllm_amd.cuda_loader import load_cuda_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ENC = {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k}


@pytest.fixture(scope="module")
def mod():
    m = load_cuda_kernel()
    assert m is not None and torch.cuda.is_available()
    return m


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k"])
@pytest.mark.parametrize("t,n,k", [(16, 128, 256), (64, 300, 768), (130, 129, 1000), (512, 256, 5120), (257, 64, 2048), (1100, 200, 512)])
def test_prefill_matches_float_oracle(mod, type_name, t, n, k):
    rng = np.random.default_rng(t + n + k)
    blocks = ENC[type_name]((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    x_np = rng.standard_normal((t, k)).astype(np.float32)
    x_np[3] *= 1e4                      # a token row with huge activations and one with tiny ones: the per-row power-of-two scaling must absorb both
    x_np[5] *= 1e-6
    ref_w = O.dequant_rows(blocks, type_name, k)
    grid = torch.empty(0, dtype=torch.int8, device=DEV)
    for dt, tol in ((torch.bfloat16, 4e-4), (torch.float32, 6e-4), (torch.float16, 4e-4)):
        x = torch.from_numpy(x_np).to(DEV).to(dt)
        if dt == torch.float16:
            x = torch.from_numpy(np.clip(x_np, -6e4, 6e4)).to(DEV).to(dt)
        print(f"case prefill {type_name} t={t} n={n} k={k} {dt}", flush=True)
        y = mod.gguf_quant_gemm_prefill_forward(x, torch.from_numpy(blocks).to(DEV), k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = O.matmul_f(x.float().cpu().numpy(), ref_w)
        got = y.cpu().numpy()
        assert O.rel_l2(got, want) <= 1e-3
        # row by row as well: a scaling bug in one token must not hide in the total
        row_err = np.sqrt(((got - want) ** 2).sum(axis=1) / np.maximum((want ** 2).sum(axis=1), 1e-300))
        assert row_err.max() <= tol, (dt, row_err.argmax(), row_err.max())


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k"])
@pytest.mark.parametrize("t,n,k", [(17, 100, 768), (24, 16, 256), (33, 272, 2048), (40, 129, 1000), (48, 5120, 5120), (32, 1000, 5120)])
def test_prefill_17_to_48_rows_matches_float_oracle(mod, type_name, t, n, k):
    """The token counts between decode and the large tiles: every block is decoded once in registers (sc * code as exact fp16 integers) and
    multiplied into all rows on the fp16 matrix cores.  16-bit activations are exact in the operands, so the distance to the float
    statement is float32 summation order only; float32 activations are rounded to fp16 once (<= 1e-3)."""
    rng = np.random.default_rng(7 * t + n + k)
    blocks = ENC[type_name]((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    x_np = rng.standard_normal((t, k)).astype(np.float32)
    x_np[3] *= 1e4                      # per-row power-of-two scaling has to absorb a huge and a tiny row
    x_np[5] *= 1e-6
    ref_w = O.dequant_rows(blocks, type_name, k)
    grid = torch.empty(0, dtype=torch.int8, device=DEV)
    for dt, tol in ((torch.bfloat16, 5e-6), (torch.float16, 5e-6), (torch.float32, 6e-4)):
        x = torch.from_numpy(np.clip(x_np, -6e4, 6e4) if dt == torch.float16 else x_np).to(DEV).to(dt)
        print(f"case prefill rows {type_name} t={t} n={n} k={k} {dt}", flush=True)
        y = mod.gguf_quant_gemm_prefill_forward(x, torch.from_numpy(blocks).to(DEV), k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = O.matmul_f(x.float().cpu().numpy(), ref_w)
        got = y.cpu().numpy()
        row_err = np.sqrt(((got - want) ** 2).sum(axis=1) / np.maximum((want ** 2).sum(axis=1), 1e-300))
        assert row_err.max() <= tol, (dt, row_err.argmax(), row_err.max())
        y16 = mod.gguf_quant_gemm_prefill_forward(x, torch.from_numpy(blocks).to(DEV), k, O.TYPE_IDS[type_name], grid)
        assert y16.dtype == torch.bfloat16 and torch.equal(y16, y.to(torch.bfloat16))


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k"])
@pytest.mark.parametrize("t", [20, 40, 64])
def test_prefill_17_to_64_rows_read_as_held_rescale_every_trip(mod, type_name, t):
    """bf16 / fp16 rows whose length is a whole number of super-blocks are read as the caller holds them (no staging launch); bf16
    values become fp16 inside the kernel under a power of two chosen per row and per trip of two blocks.  Magnitudes that change
    along a row by 40 orders, rows and trips of zeros and rows near the ends of the bf16 range must all come out as the float
    statement has them: the conversion is exact, so only float32 summation order is left."""
    n, k = 4352, 5120                    # 34 column groups, 7 slices of 3 blocks: two trips per workgroup, the second of one block
    rng = np.random.default_rng(100 + t)
    blocks = ENC[type_name]((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    x_np = rng.standard_normal((t, k)).astype(np.float32)
    x_np[3] *= 1e4
    x_np[5] *= 1e-6
    x_np[7, :512] *= 1e20                # the first trip of the first slice dwarfs everything else in the row ...
    x_np[7, 512:1024] *= 1e-20           # ... and its second trip and the next slice's first are tiny
    x_np[8] = 0.0
    x_np[9, 512:768] = 0.0               # a trip of zeros between ordinary ones
    x_np[10] *= 1e30
    x_np[11] *= 1e-30
    x_np[12, ::2] *= 1e-5                # neighbours five orders apart inside every group
    ref_w = O.dequant_rows(blocks, type_name, k)
    grid = torch.empty(0, dtype=torch.int8, device=DEV)
    w = torch.from_numpy(blocks).to(DEV)
    for dt in (torch.bfloat16, torch.float16):
        x = torch.from_numpy(np.clip(x_np, -6e4, 6e4) if dt == torch.float16 else x_np).to(DEV).to(dt)
        print(f"case prefill rows as held {type_name} t={t} {dt}", flush=True)
        y = mod.gguf_quant_gemm_prefill_forward(x, w, k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
        torch.cuda.synchronize()
        xs = x.float().cpu().numpy().astype(np.float64)
        want = xs @ ref_w.astype(np.float64).T
        got = y.cpu().numpy().astype(np.float64)
        assert np.isfinite(got).all()
        assert (got[8] == 0.0).all()
        # per slice of a row the error is relative to that slice's own products (each trip is scaled by itself)
        bound = (np.abs(xs) @ np.abs(ref_w.astype(np.float64)).T) * 2e-6 + 1e-44
        assert (np.abs(got - want) <= bound).all(), (dt, np.unravel_index(np.argmax(np.abs(got - want) / bound), got.shape))
        # a view that is not 16-byte aligned goes through the staging launch: same bits (both conversions are exact)
        if dt == torch.bfloat16 and t <= 48:
            pad = torch.zeros(t * k + 1, dtype=dt, device=DEV)
            pad[1:] = x.reshape(-1)
            y2 = mod.gguf_quant_gemm_prefill_forward(pad[1:].view(t, k), w, k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
            assert torch.equal(y2, y)


def test_prefill_3d_input_and_bf16_output(mod):
    rng = np.random.default_rng(0)
    blocks = torch.from_numpy(C.quantize_q4_k((rng.standard_normal((192, 512)) * 0.02).astype(np.float32))).to(DEV)
    x = torch.randn(4, 8, 512, device=DEV, dtype=torch.bfloat16)
    grid = torch.empty(0, dtype=torch.int8, device=DEV)
    y = mod.gguf_quant_gemm_prefill_forward(x, blocks, 512, 3, grid)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (4, 8, 192)
    y32 = mod.gguf_quant_gemm_prefill_forward(x, blocks, 512, 3, grid, out_dtype=torch.float32)
    assert torch.equal(y32.to(torch.bfloat16), y)
    # the tile GEMM and the decode kernels state the same operator
    yd = torch.cat([mod.gguf_quant_gemm_forward(x.view(32, 512)[i:i + 1], blocks, 512, 3, grid, out_dtype=torch.float32) for i in range(32)])
    assert O.rel_l2(y32.view(32, 192).cpu().numpy(), yd.cpu().numpy()) < 5e-4


@pytest.mark.parametrize("type_name", ["q4_k", "q5_k"])
@pytest.mark.parametrize("n", [5120, 17408])
def test_prefill_baseline_shapes_sampled(mod, type_name, n):
    """BASELINE config 3: both shapes, both formats, T = 64, 512 and 2048.  The weights are encoded once per (format, shape);
    the oracle checks 64 sampled output columns of every token row (seconds on the host)."""
    rng = np.random.default_rng(1003 + n + len(type_name))
    k = 5120
    blocks = ENC[type_name]((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))
    dblocks = torch.from_numpy(blocks).to(DEV)
    grid = codebooks.grid_tensor_for_type(O.TYPE_IDS[type_name]).to(DEV)
    cols = rng.choice(n, size=64, replace=False)
    ref_w = O.dequant_rows(blocks[cols], type_name, k)
    for t in (64, 512, 2048):
        x = torch.from_numpy(rng.standard_normal((t, k)).astype(np.float32)).to(DEV).to(torch.bfloat16)
        print(f"case prefill baseline {type_name} n={n} t={t}", flush=True)
        y = mod.gguf_quant_gemm_prefill_forward(x, dblocks, k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
        torch.cuda.synchronize()
        assert tuple(y.shape) == (t, n)
        want = O.matmul_f(x.float().cpu().numpy(), ref_w)
        got = y.cpu().numpy()[:, cols]
        assert O.rel_l2(got, want) <= 1e-3, (t, O.rel_l2(got, want))
        row_err = np.sqrt(((got - want) ** 2).sum(axis=1) / np.maximum((want ** 2).sum(axis=1), 1e-300))
        assert row_err.max() <= 2e-3, (t, row_err.argmax(), row_err.max())


@pytest.mark.parametrize("type_name,n,rows", [("q4_k", 17408, 5), ("q5_k", 17408, 7), ("q4_k", 5120, 11), ("q4_k", 5120, 12), ("q5_k", 5120, 15),
                                              ("iq1_m", 17408, 3), ("iq1_m", 17408, 4), ("q6_k", 17408, 2), ("q6_k", 17408, 3),
                                              ("iq3_xxs", 5120, 7), ("iq3_xxs", 5120, 8), ("q6_k", 5120, 5), ("iq2_xs", 5120, 9)])
def test_operator_few_rows_on_large_matrices(mod, type_name, n, rows):
    """Between 2 and 15 activation rows the operator chooses between the decode kernels and the tile
    kernel by matrix size and format; either side of that choice states the same product (64 sampled columns)."""
    rng = np.random.default_rng(n + rows)
    k = 5120
    if type_name in ENC:
        blocks = ENC[type_name]((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))
    elif type_name == "iq1_m":
        blocks = C.random_iq1_m(rng, n, k // 256)
    else:
        blocks = C.random_blocks(rng, type_name, n, k // 256)
    x_np = rng.standard_normal((rows, k)).astype(np.float32)
    x_np[1] *= 1e3
    x_np[rows - 1] *= 1e-5
    x = torch.from_numpy(x_np).to(DEV).to(torch.bfloat16)
    grid = codebooks.grid_tensor_for_type(O.TYPE_IDS[type_name]).to(DEV)
    print(f"case operator {type_name} n={n} rows={rows}", flush=True)
    y = mod.gguf_quant_gemm_forward(x, torch.from_numpy(blocks).to(DEV), k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
    torch.cuda.synchronize()
    assert tuple(y.shape) == (rows, n)
    cols = rng.choice(n, size=64, replace=False)
    want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks[cols], type_name, k))
    got = y.cpu().numpy()[:, cols]
    row_err = np.sqrt(((got - want) ** 2).sum(axis=1) / np.maximum((want ** 2).sum(axis=1), 1e-300))
    assert row_err.max() <= 6e-4, (row_err.argmax(), row_err.max())


# ---- FP8 E4M3 block-scaled weights through the same tile kernel ---------------------------------------

@pytest.mark.parametrize("t,n,k", [(16, 128, 256), (64, 300, 768), (130, 129, 1024), (257, 520, 2048)])
def test_fp8_prefill_matches_float_oracle(mod, t, n, k):
    rng = np.random.default_rng(t * 7 + n + k)
    codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x3c                       # no NaN codes
    scale = rng.uniform(0.001, 0.01, size=((n + 127) // 128, k // 128)).astype(np.float32)
    x_np = rng.standard_normal((t, k)).astype(np.float32)
    x_np[1] *= 300.0
    for dt in (torch.bfloat16, torch.float32):
        print(f"case fp8 prefill t={t} n={n} k={k} {dt}", flush=True)
        x = torch.from_numpy(x_np).to(DEV).to(dt)
        y = mod.fp8_block_gemm_forward(x, torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV))
        torch.cuda.synchronize()
        want = O.matmul_f(x.float().cpu().numpy(), O.dequant_fp8_block(codes, scale))
        # rows compared one by one: the huge row must not hide errors in the others
        got = y.cpu().numpy()
        for r in (0, 1, t - 1):
            assert O.rel_l2(got[r], want[r]) <= 1e-3, (t, n, k, dt, r)
        assert O.rel_l2(got, want) <= 1e-3


def test_fp8_float32_activations_precision_step_at_16_rows(mod):
    """float32 activations stay on the float32 matvec (<= 1e-5 against the float statement of soft_fp8_blockfp8_gemm,
    src/kernels/ops.py:641-648) up to 15 rows and take the fp16 tile kernel from 16 rows on (operands rounded to fp16, <= 1e-3):
    both sides of the switch are pinned here."""
    rng = np.random.default_rng(16)
    n, k = 384, 2048
    codes, scale = C.quantize_fp8_block((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    ref_w = O.dequant_fp8_block(codes, scale)
    dc, ds = torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV)
    errs = {}
    for rows in (15, 16):
        x_np = rng.standard_normal((rows, k)).astype(np.float32)
        print(f"case fp8 float32 activations rows={rows}", flush=True)
        y = mod.fp8_block_gemm_forward(torch.from_numpy(x_np).to(DEV), dc, ds, out_dtype=torch.float32)
        torch.cuda.synchronize()
        errs[rows] = O.rel_l2(y.cpu().numpy(), O.matmul_f(x_np, ref_w))
    assert errs[15] <= 1e-5, errs
    assert errs[16] <= 1e-3, errs


def test_fp8_prefill_baseline_shape_sampled(mod):
    """BASELINE config 4 at T = 512 (N = 17408, K = 5120, weights N(0, 0.02) with blockmax/448 scales); 64 sampled columns."""
    rng = np.random.default_rng(1004)
    n, k, t = 17408, 5120, 512
    codes, scale = C.quantize_fp8_block(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    x = torch.from_numpy(rng.standard_normal((t, k)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    y = mod.fp8_block_gemm_forward(x, torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV))
    torch.cuda.synchronize()
    cols = rng.choice(n, size=64, replace=False)
    w = O.dequant_fp8_block(codes, scale)[cols]
    want = O.matmul_f(x.float().cpu().numpy(), w)
    assert O.rel_l2(y.cpu().numpy()[:, cols], want) <= 1e-3


@pytest.mark.parametrize("n,rows", [(17408, 2), (17408, 3), (5120, 4), (5120, 5)])
def test_fp8_operator_few_rows_on_large_matrices(mod, n, rows):
    """FP8 with a few activation rows: one matvec per row below the crossover, the tile kernel from it on."""
    rng = np.random.default_rng(n + rows)
    k = 5120
    codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x3c
    scale = rng.uniform(0.001, 0.01, size=((n + 127) // 128, k // 128)).astype(np.float32)
    x_np = rng.standard_normal((rows, k)).astype(np.float32)
    x_np[1] *= 300.0
    x = torch.from_numpy(x_np).to(DEV).to(torch.bfloat16)
    print(f"case fp8 operator n={n} rows={rows}", flush=True)
    y = mod.fp8_block_gemm_forward(x, torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV))
    torch.cuda.synchronize()
    cols = rng.choice(n, size=64, replace=False)
    w = O.dequant_fp8_block(codes, scale)[cols]
    want = O.matmul_f(x.float().cpu().numpy(), w)
    got = y.cpu().numpy()[:, cols]
    for r in range(rows):
        assert O.rel_l2(got[r], want[r]) <= 1e-3, (n, rows, r)


# ---- the other super-block formats through the same tile kernel --------------------------------------

@pytest.mark.parametrize("type_name", ["q2_k", "iq2_xxs", "iq1_m"])
@pytest.mark.parametrize("t,n,k", [(16, 128, 256), (64, 300, 768), (130, 129, 1024), (300, 520, 3072)])
def test_prefill_other_formats_match_float_oracle(mod, type_name, t, n, k):
    from pocketllm_amd import codebooks
    rng = np.random.default_rng(t + 3 * n + k)
    if type_name == "q2_k":
        blocks = C.quantize_q2_k((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
        grid = torch.empty(0, dtype=torch.int8, device=DEV)
    elif type_name == "iq2_xxs":
        blocks = C.random_iq2_xxs(rng, n, k // 256)
        grid = codebooks.get_iq2xxs_signed_grid_tensor().to(DEV)
    else:
        blocks = C.random_iq1_m(rng, n, k // 256)
        grid = codebooks.get_iq1_grid_tensor().to(DEV)
    x = torch.from_numpy(rng.standard_normal((t, k)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    print(f"case {type_name} prefill t={t} n={n} k={k}", flush=True)
    y = mod.gguf_quant_gemm_prefill_forward(x, torch.from_numpy(blocks).to(DEV), k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
    torch.cuda.synchronize()
    want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks, type_name, k))
    assert O.rel_l2(y.cpu().numpy(), want) <= 1e-3, (type_name, t, n, k)


@pytest.mark.parametrize("type_name", ["q6_k", "iq4_xs", "iq2_xs", "iq3_xxs"])
@pytest.mark.parametrize("t,n,k", [(16, 128, 256), (40, 96, 768), (130, 33, 1000), (300, 520, 5120), (1100, 200, 512)])
def test_prefill_operator_serves_q6_k_and_iq4_xs(mod, type_name, t, n, k):
    """Q6_K (2-byte aligned blocks, signed scales), IQ4_XS (code table through byte permutes), IQ2_XS and IQ3_XXS (grid and sign
    tables in LDS) in the tile kernel."""
    rng = np.random.default_rng(t + n + k)
    if type_name in ("q6_k", "iq4_xs"):
        enc = C.quantize_q6_k if type_name == "q6_k" else C.quantize_iq4_xs
        blocks = enc((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    else:
        blocks = C.random_blocks(rng, type_name, n, (k + 255) // 256)
    x = torch.from_numpy(rng.standard_normal((t, k)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    print(f"case {type_name} prefill t={t} n={n} k={k}", flush=True)
    y = mod.gguf_quant_gemm_prefill_forward(x, torch.from_numpy(blocks).to(DEV), k, O.TYPE_IDS[type_name],
                                            codebooks.grid_tensor_for_type(O.TYPE_IDS[type_name]).to(DEV), out_dtype=torch.float32)
    torch.cuda.synchronize()
    want = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks, type_name, k))
    assert O.rel_l2(y.cpu().numpy(), want) <= 1e-3, (type_name, t, n, k)


# ---- FP8 activations x FP8 weights on the native FP8 matrix path -----------------------------------

@pytest.mark.parametrize("t,n,k", [(1, 128, 128), (16, 130, 256), (77, 300, 1024), (200, 512, 5120), (129, 130, 128), (300, 1100, 1024),
                                   (513, 2050, 384)])
def test_fp8_gemm_native_matches_act_quant_semantics(mod, t, n, k):
    """act_quant + fp8_gemm (ops.py:982-1051) against the oracle, which dequantizes both sides and multiplies in
    float64.  The only differences are the matrix core's own summation of 64 products per instruction (full-range
    random codes make that visible at a few 1e-5) and float32 accumulation across the K blocks."""
    rng = np.random.default_rng(5 * t + n + k)
    codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x3c
    scale = rng.uniform(0.001, 0.01, size=((n + 127) // 128, k // 128)).astype(np.float32)
    x_np = rng.standard_normal((t, k)).astype(np.float32)
    x_np[0] *= 50.0
    x = torch.from_numpy(x_np).to(DEV)
    a, a_s = mod.fp8_act_quant_forward(x)
    print(f"case fp8 native t={t} n={n} k={k}", flush=True)
    y = mod.fp8_gemm_forward(a, a_s, torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV))
    torch.cuda.synchronize()
    want = O.fp8_gemm_q(x_np, codes, scale)
    assert O.rel_l2(y.cpu().numpy(), want) <= 2e-4
    # the ops-layer name takes the same route
    from pocketllm_amd import ops
    y2 = ops.fp8_gemm(a, a_s, torch.from_numpy(codes).to(DEV).view(torch.float8_e4m3fn), torch.from_numpy(scale).to(DEV))
    assert O.rel_l2(y2.float().cpu().numpy(), want) <= 1e-2       # default dtype may be 16-bit


@pytest.mark.parametrize("t,n,k", [(300, 1102, 512), (260, 257, 1024)])
def test_fp8_gemm_native_output_forms_above_128_tokens(mod, t, n, k):
    """The kernel for more than 128 tokens stores four neighbouring outputs of a token at once where the row length allows it and
    element by element otherwise; bf16 / fp16 outputs are the float32 ones rounded once; activation scales that do not start on a
    16-byte boundary take the other kernel (same sums up to the grouping of float32 additions)."""
    rng = np.random.default_rng(t * n + k)
    codes, scale = C.quantize_fp8_block(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    x_np = rng.standard_normal((t, k)).astype(np.float32)
    a, a_s = mod.fp8_act_quant_forward(torch.from_numpy(x_np).to(DEV))
    w, sc = torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV)
    print(f"case fp8 native outputs t={t} n={n} k={k}", flush=True)
    y32 = mod.fp8_gemm_forward(a, a_s, w, sc)
    torch.cuda.synchronize()
    want = O.fp8_gemm_q(x_np, codes, scale)
    assert O.rel_l2(y32.cpu().numpy(), want) <= 2e-4
    for dt in (torch.bfloat16, torch.float16):
        y16 = mod.fp8_gemm_forward(a, a_s, w, sc, out_dtype=dt)
        assert torch.equal(y16, y32.to(dt)), dt
    # the same scales four bytes off a 16-byte boundary
    shifted = torch.empty(a_s.numel() + 1, dtype=torch.float32, device=DEV)[1:].view_as(a_s)
    shifted.copy_(a_s)
    assert shifted.data_ptr() % 16 != 0
    y_other = mod.fp8_gemm_forward(a, shifted, w, sc)
    torch.cuda.synchronize()
    assert O.rel_l2(y_other.cpu().numpy(), y32.cpu().numpy()) <= 1e-6


def test_fp8_gemm_native_baseline_shape_sampled(mod):
    """BASELINE config 4 at T = 512 with the reference's FP8-activation semantics; 64 sampled columns."""
    rng = np.random.default_rng(1005)
    n, k, t = 17408, 5120, 512
    codes, scale = C.quantize_fp8_block(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    x_np = rng.standard_normal((t, k)).astype(np.float32)
    a, a_s = mod.fp8_act_quant_forward(torch.from_numpy(x_np).to(DEV))
    y = mod.fp8_gemm_forward(a, a_s, torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV))
    torch.cuda.synchronize()
    cols = np.sort(rng.choice(n, size=64, replace=False))
    xa_codes, xs = O.fp8_act_quant(x_np)
    xa = O.fp8_e4m3_decode(xa_codes).reshape(t, k // 128, 128) * xs[..., None]
    want = O.matmul_f(xa.reshape(t, k), O.dequant_fp8_block(codes, scale)[cols])
    assert O.rel_l2(y.cpu().numpy()[:, cols], want) <= 2e-4


@pytest.mark.parametrize("t,n,k", [(512, 17408, 5120), (640, 1024, 2048), (100, 3000, 1280)])
def test_fp8_gemm_native_split_tiles_equal_whole_tiles(mod, t, n, k):
    """With a workspace the left-over output tiles are cut along K and their partial sums added in slice order; without one
    every tile runs whole.  Same operands, every output element: the two differ only by the grouping of float32 additions."""
    from pocketllm_amd import _ffi
    lib = _ffi.load_library()
    rng = np.random.default_rng(t + n + k)
    codes, scale = C.quantize_fp8_block(rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02))
    a, a_s = mod.fp8_act_quant_forward(torch.from_numpy(rng.standard_normal((t, k)).astype(np.float32)).to(DEV))
    w, sc = torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV)
    a8 = a.view(torch.uint8)
    need = int(lib.pllm_fp8_gemm_workspace_bytes(t, k, n))
    assert need > 0, "shape no longer splits any tile"
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    y_split = torch.empty(t, n, dtype=torch.float32, device=DEV)
    y_whole = torch.empty(t, n, dtype=torch.float32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    print(f"case fp8 native split t={t} n={n} k={k} workspace={need}", flush=True)
    assert lib.pllm_fp8_gemm_ws(a8.data_ptr(), a_s.data_ptr(), w.data_ptr(), sc.data_ptr(), y_split.data_ptr(), 0, t, k, n, ws.data_ptr(), need, stream) == 0
    assert lib.pllm_fp8_gemm(a8.data_ptr(), a_s.data_ptr(), w.data_ptr(), sc.data_ptr(), y_whole.data_ptr(), 0, t, k, n, stream) == 0
    torch.cuda.synchronize()
    got, ref = y_split.cpu().numpy(), y_whole.cpu().numpy()
    assert np.isfinite(got).all()
    assert O.rel_l2(got, ref) <= 1e-6
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()
    # a short workspace falls back to whole tiles: bit-identical to the entry point without one
    y_short = torch.empty(t, n, dtype=torch.float32, device=DEV)
    assert lib.pllm_fp8_gemm_ws(a8.data_ptr(), a_s.data_ptr(), w.data_ptr(), sc.data_ptr(), y_short.data_ptr(), 0, t, k, n, ws.data_ptr(), 16, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(y_short, y_whole)


# ---- Q4_K / Q5_K on the int8 matrix cores: int8 activation semantics ------------------------------------

@pytest.mark.parametrize("type_name", ["q4_k", "q5_k"])
@pytest.mark.parametrize("t,n,k", [(16, 128, 256), (64, 300, 768), (130, 129, 1000), (257, 64, 2048), (1, 40, 512), (700, 200, 512)])
def test_int8_prefill_matches_the_int8_activation_oracle(mod, type_name, t, n, k):
    """pllm_gguf_quant_gemm_q8 against oracle.kquant_gemm_q (activations quantized per 32 values, integer group dots, float32
    scales): the integer part is exact, so the two differ by the order of the float32 sums only.  The distance to the
    float-activation oracle is the quantization error of the activations (about 5e-3) and is reported, not bounded tightly."""
    rng = np.random.default_rng(t + n + k)
    kp = (k + 255) // 256 * 256
    w = np.zeros((n, kp), dtype=np.float32)
    w[:, :k] = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    blocks = ENC[type_name](w)
    x_np = rng.standard_normal((t, k)).astype(np.float32)
    if t > 5:
        x_np[3] *= 1e4
        x_np[5] *= 1e-6
        x_np[2, 64:96] = 0.0                                   # an all-zero activation group
    grid = torch.empty(0, dtype=torch.int8, device=DEV)
    for dt in (torch.bfloat16, torch.float32):
        x = torch.from_numpy(x_np).to(DEV).to(dt)
        print(f"case int8 prefill {type_name} t={t} n={n} k={k} {dt}", flush=True)
        y = mod.gguf_quant_gemm_q8_forward(x, torch.from_numpy(blocks).to(DEV), k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
        torch.cuda.synchronize()
        xp = np.zeros((t, kp), dtype=np.float32)
        xp[:, :k] = x.float().cpu().numpy()
        want = O.kquant_gemm_q(xp, blocks, type_name)
        got = y.cpu().numpy()
        row_err = np.sqrt(((got - want) ** 2).sum(axis=1) / np.maximum((want ** 2).sum(axis=1), 1e-300))
        assert row_err.max() <= 2e-5, (dt, row_err.argmax(), row_err.max())
        far = O.rel_l2(got, O.matmul_f(xp, O.dequant_rows(blocks, type_name, kp)))
        assert far <= 2e-2, far


@pytest.mark.parametrize("type_name,n", [("q4_k", 5120), ("q5_k", 17408)])
def test_int8_prefill_baseline_shapes_sampled(mod, type_name, n):
    """BASELINE config 3 with its own semantics (int8 activation blocks): T = 64 and 2048, 48 sampled columns against the int8 oracle."""
    rng = np.random.default_rng(1013 + n)
    k = 5120
    blocks = ENC[type_name]((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))
    dblocks = torch.from_numpy(blocks).to(DEV)
    grid = torch.empty(0, dtype=torch.int8, device=DEV)
    cols = rng.choice(n, size=48, replace=False)
    for t in (64, 2048):
        x = torch.from_numpy(rng.standard_normal((t, k)).astype(np.float32)).to(DEV).to(torch.bfloat16)
        print(f"case int8 prefill baseline {type_name} n={n} t={t}", flush=True)
        y = mod.gguf_quant_gemm_q8_forward(x, dblocks, k, O.TYPE_IDS[type_name], grid, out_dtype=torch.float32)
        torch.cuda.synchronize()
        want = O.kquant_gemm_q(x.float().cpu().numpy(), blocks[cols], type_name)
        assert O.rel_l2(y.cpu().numpy()[:, cols], want) <= 2e-5
