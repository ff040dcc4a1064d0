"""GPU: bit-exact block dequantization for every format, FP8 quantizer and FP8 matvec parity."""
import json

import numpy as np
import pytest
import torch

from oracle import gguf_oracle as O
from pocketllm_amd import _ffi, block_codec as C, ops
from pocketllm_amd.cuda_loader import load_cuda_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def mod():
    m = load_cuda_kernel()
    assert m is not None and torch.cuda.is_available()
    return m


def _random_blocks(rng, type_name, n, bpr):
    bb = O.BLOCK_BYTES[type_name]
    if type_name == "iq1_m":
        return C.random_iq1_m(rng, n, bpr, d_range=(0.001, 0.08))
    blocks = rng.integers(0, 256, size=(n, bpr, bb), dtype=np.uint8)
    for off in {"q8_0": [0], "q4_k": [0, 2], "q5_k": [0, 2], "q2_k": [80, 82], "iq2_xxs": [0], "q6_k": [208], "iq4_xs": [0], "iq2_xs": [0], "iq3_xxs": [0], "q3_k": [108]}[type_name]:
        vals = rng.uniform(0.001, 0.05, size=(n, bpr)) * rng.choice([-1.0, 1.0], size=(n, bpr))
        blocks[..., off:off + 2] = vals.astype("<f2").view(np.uint8).reshape(n, bpr, 2)
    return blocks


def _tid(type_name):
    return {"q8_0": _ffi.TYPE_Q8_0, "q3_k": _ffi.TYPE_Q3_K}.get(type_name) or O.TYPE_IDS[type_name]


@pytest.mark.parametrize("type_name", ["q8_0", "q4_k", "q5_k", "q2_k", "iq2_xxs", "iq1_m", "q6_k", "iq4_xs", "iq2_xs", "iq3_xxs", "q3_k"])
def test_dequant_is_bit_exact_on_random_bytes(mod, type_name):
    rng = np.random.default_rng(31)
    n, bpr = 37, (24 if type_name == "q8_0" else 3)
    k = bpr * O.BLOCK_ELEMS[type_name]
    blocks = _random_blocks(rng, type_name, n, bpr)
    got = mod.gguf_dequantize_rows(torch.from_numpy(blocks).to(DEV), _tid(type_name), k).cpu().numpy()
    np.testing.assert_array_equal(got, O.dequant_rows(blocks, type_name, k))
    # ragged K and selected rows (with a repeat and an out-of-range id that must come back as zeros)
    ids = np.array([5, 0, 36, 5, 99, -1], dtype=np.int64)
    kk = k - 19
    got = mod.gguf_dequantize_rows(torch.from_numpy(blocks).to(DEV), _tid(type_name), kk, torch.from_numpy(ids).to(DEV)).cpu().numpy()
    want = O.dequant_rows(blocks, type_name, kk)
    np.testing.assert_array_equal(got[:4], want[ids[:4]])
    assert (got[4:] == 0).all()


@pytest.mark.parametrize("name", ["iq1m_oracle.json", "q8_0_reference_decode.json", "q4_k_reference_decode.json",
                                  "q5_k_reference_decode.json", "iq2_xxs_reference_decode.json", "q6_k_reference_decode.json",
                                  "iq4_xs_reference_decode.json", "iq2_xs_reference_decode.json", "iq3_xxs_reference_decode.json",
                                  "q3_k_reference_decode.json"])
def test_dequant_matches_golden_vectors(mod, golden_dir, name):
    raw = json.loads((golden_dir / name).read_text())
    blocks = np.frombuffer(bytes.fromhex(raw["blocks_u8"]), dtype=np.uint8)
    values = np.frombuffer(bytes.fromhex(raw["values_f32"]), dtype="<f4")
    if name.startswith("iq1m"):
        type_name, blocks = "iq1_m", blocks.reshape(raw["n_blocks"], 1, 56)
    else:
        type_name = raw["type"]
        blocks = blocks.reshape(raw["rows"], raw["blocks_per_row"], raw["block_bytes"])
    k = blocks.shape[1] * O.BLOCK_ELEMS[type_name]
    got = mod.gguf_dequantize_rows(torch.from_numpy(blocks.copy()).to(DEV), _tid(type_name), k).cpu().numpy()
    np.testing.assert_array_equal(got, values.reshape(blocks.shape[0], k))


def test_embedding_operator(mod):
    rng = np.random.default_rng(8)
    w = (rng.standard_normal((50, 512)) * 0.02).astype(np.float32)
    for type_name, enc in (("q4_k", C.quantize_q4_k), ("q5_k", C.quantize_q5_k), ("q6_k", C.quantize_q6_k), ("iq4_xs", C.quantize_iq4_xs)):
        blocks = enc(w)
        ids = torch.tensor([[3, 49, 0], [7, 7, 21]], device=DEV)
        grid = torch.empty(0, dtype=torch.int8, device=DEV)
        y = mod.gguf_quant_embedding_forward(ids, torch.from_numpy(blocks).to(DEV), 512, O.TYPE_IDS[type_name], grid)
        assert y.dtype == torch.bfloat16 and tuple(y.shape) == (2, 3, 512)
        want = torch.from_numpy(O.dequant_rows(blocks, type_name)[ids.cpu().numpy()]).to(torch.bfloat16)
        assert torch.equal(y.cpu(), want)
    with pytest.raises(RuntimeError, match="token_ids must be int64"):
        mod.gguf_quant_embedding_forward(ids.int(), torch.from_numpy(blocks).to(DEV), 512, O.TYPE_IDS[type_name], grid)


def test_q8_0_ops_surface(mod):
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((96, 64)) * 0.5).astype(np.float32)
    blocks_np = C.pack_q8_0(w)
    blocks = torch.from_numpy(blocks_np).to(DEV)
    np.testing.assert_array_equal(ops.q8_0_weight_dequantize(blocks, 64).cpu().numpy(), O.dequant_rows(blocks_np, "q8_0", 64))
    x = torch.randn(2, 64, device=DEV, dtype=torch.bfloat16)
    ref = O.matmul_f(x.float().cpu().numpy(), O.dequant_rows(blocks_np, "q8_0", 64))
    got = ops.q8_0_weight_gemm(x, blocks, row_elems=64, out_dtype=torch.float32)
    assert O.rel_l2(got.cpu().numpy(), ref) < 1e-4
    # the reference's own test bound (tests/test_q8_0_cuda.py:39)
    got_bf = ops.q8_0_weight_gemm_cuda_ext(x, blocks, row_elems=64, out_dtype=torch.bfloat16)
    assert torch.allclose(got_bf.float().cpu(), torch.from_numpy(ref).float(), atol=0.05, rtol=0.02)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.q8_0_weight_gemm(x.cpu(), blocks.cpu(), row_elems=64)


# ---- FP8 -----------------------------------------------------------------------------------------

def test_fp8_dequant_all_codes_and_block_scales(mod):
    rng = np.random.default_rng(1)
    n, k = 130, 300
    codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x3c                       # no NaN codes, as the reference's tests
    codes[0, :256] = np.where((np.arange(256) & 0x7f) == 0x7f, 0, np.arange(256)).astype(np.uint8)
    scale = rng.uniform(0.25, 4.0, size=(2, 3)).astype(np.float32)
    got = mod.fp8_block_dequantize(torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV)).cpu().numpy()
    np.testing.assert_array_equal(got, O.dequant_fp8_block(codes, scale))
    # float8 tensor input and the ops-layer name
    w8 = torch.from_numpy(codes).to(DEV).view(torch.float8_e4m3fn)
    got2 = ops.soft_fp8_blockfp8_weight_dequant(w8, torch.from_numpy(scale).to(DEV))
    np.testing.assert_array_equal(got2.cpu().numpy(), got)


@pytest.mark.parametrize("n,k,rows", [(130, 304, 1), (256, 1024, 1), (17408, 5120, 1), (64, 5120, 3), (33, 300, 2), (16, 40960, 1), (4500, 8192, 1), (17408, 5120, 6)])
def test_fp8_matvec_matches_oracle(mod, n, k, rows):
    rng = np.random.default_rng(40 + n)
    if n * k <= 4_000_000:
        codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
        codes[(codes & 0x7f) == 0x7f] = 0x3c
        scale = rng.uniform(0.001, 0.01, size=((n + 127) // 128, (k + 127) // 128)).astype(np.float32)
    else:
        codes, scale = C.quantize_fp8_block((rng.standard_normal((n, k), dtype=np.float32) * np.float32(0.02)))
    x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(DEV)
    for dt in (torch.bfloat16, torch.float32):
        print(f"case fp8 n={n} k={k} rows={rows} {dt}", flush=True)
        xd = x.to(dt)
        y = mod.fp8_block_gemm_forward(xd, torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV))
        torch.cuda.synchronize()
        want = O.matmul_f(xd.float().cpu().numpy(), O.dequant_fp8_block(codes, scale))
        # float32 activations stay on the float32 matvec below 16 rows whatever the matrix size; 16-bit activations take the
        # matrix-core matvec (exact products) up to 16 rows and may take the fp16 tile kernel beyond (operands rounded to fp16)
        tol = 1e-3 if (dt != torch.float32 and rows > 16 and n * k >= (64 << 20)) else 1e-5
        assert O.rel_l2(y.cpu().numpy(), want) <= tol, (n, k, rows, dt)


@pytest.mark.parametrize("n,k,rows", [(33, 384, 2), (16, 128, 5), (130, 1024, 16), (64, 5120, 17), (48, 6144, 9), (5, 256, 40), (33, 384, 40)])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_fp8_few_rows_on_the_matrix_cores(mod, n, k, rows, dt):
    """Two or more rows of 16-bit activations with k a multiple of 128: one pass over the weights for every 16 rows, codes and
    activations exact in the matrix-core operands.  Row counts around 16, weight rows that do not fill a tile, rows of more
    scale blocks than a wave holds at once; every code value occurs."""
    rng = np.random.default_rng(90 + n + rows)
    codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x3c
    scale = rng.uniform(0.001, 0.01, size=((n + 127) // 128, (k + 127) // 128)).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(DEV).to(dt)
    print(f"case fp8 few rows n={n} k={k} rows={rows} {dt}", flush=True)
    y = mod.fp8_block_gemm_forward(x, torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV))
    torch.cuda.synchronize()
    want = O.matmul_f(x.float().cpu().numpy(), O.dequant_fp8_block(codes, scale))
    got = y.cpu().numpy()
    assert y.dtype == torch.float32 and got.shape == want.shape
    # more than 16 rows of a multiple of 256 columns run the fp16 tile kernel (operands rounded to fp16); other column counts
    # stay here, 16 rows per pass over the weights
    exact = rows <= 16 or k % 256 != 0
    assert O.rel_l2(got, want) <= (1e-5 if exact else 1e-3)
    assert np.abs(got - want).max() <= (1e-4 if exact else 1e-2) * np.abs(want).max()


def test_fp8_act_quant_matches_reference_recipe(mod):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((5, 640)).astype(np.float32) * 3
    x[2, 128:256] = 0.0
    x[3, :128] *= 1e-6
    codes, scales = mod.fp8_act_quant_forward(torch.from_numpy(x).to(DEV))
    want_codes, want_scales = O.fp8_act_quant(x)
    np.testing.assert_array_equal(scales.cpu().numpy(), want_scales)
    got = codes.view(torch.uint8).cpu().numpy()
    nz = x != 0
    np.testing.assert_array_equal(got[nz], want_codes[nz])
    assert ((got[~nz] & 0x7f) == 0).all()
    # power-of-two scales: every scale is 2^e and not below the plain scale
    _, s2 = mod.fp8_act_quant_forward(torch.from_numpy(x).to(DEV), round_scale_pow2=True)
    s2 = s2.cpu().numpy()
    assert (np.log2(s2) == np.round(np.log2(s2))).all() and (s2 >= want_scales).all() and (s2 < 2 * want_scales).all()
    # ops layer: quantize, then the FP8 x FP8 gemm equals the oracle's statement of act_quant + fp8_gemm
    w_codes, w_scale = C.quantize_fp8_block((rng.standard_normal((96, 640)) * 0.02).astype(np.float32))
    xt = torch.from_numpy(x).to(DEV).to(torch.bfloat16)
    q, s = ops.act_quant(xt)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float32)
    try:
        y = ops.fp8_gemm(q, s, torch.from_numpy(w_codes).to(DEV).view(torch.float8_e4m3fn), torch.from_numpy(w_scale).to(DEV))
    finally:
        torch.set_default_dtype(old)
    want = O.fp8_gemm_q(xt.float().cpu().numpy(), w_codes, w_scale)
    # the native FP8 matrix-core path sums each 128-wide block in the hardware's own order and width
    assert O.rel_l2(y.cpu().numpy(), want) <= 2e-4


@pytest.mark.parametrize("n,k,rows", [(130, 304, 1), (256, 1024, 3), (4500, 8192, 1), (64, 512, 20)])
def test_fp8_accumulate_adds_the_product_to_y(mod, n, k, rows):
    """y += W x for FP8 weights: the plain operator's float32 product plus the old y, rounded once to y's type."""
    rng = np.random.default_rng(60 + n)
    codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x3c
    scale = rng.uniform(0.001, 0.01, size=((n + 127) // 128, (k + 127) // 128)).astype(np.float32)
    w, sc = torch.from_numpy(codes).to(DEV), torch.from_numpy(scale).to(DEV)
    x = torch.from_numpy(rng.standard_normal((rows, k)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    prod = mod.fp8_block_gemm_forward(x, w, sc)
    for ydt in (torch.float32, torch.bfloat16, torch.float16):
        print(f"case fp8 accumulate n={n} k={k} rows={rows} {ydt}", flush=True)
        y0 = torch.from_numpy(rng.standard_normal((rows, n)).astype(np.float32)).to(DEV).to(ydt)
        y = y0.clone()
        assert mod.fp8_block_gemm_accumulate_forward(x, w, sc, y) is y
        torch.cuda.synchronize()
        assert torch.equal(y, (y0.float() + prod).to(ydt))
