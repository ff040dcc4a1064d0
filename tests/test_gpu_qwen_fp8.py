"""FP8 E4M3 weights with fp16 block scales through the C ABI: the cases of the reference's own test of its C++ engine
operators (cpp_engine/tests/test_qwen_fp8_online.cpp:405-427, 228-300), same value ranges, same bound (max error over
max(1, |want|) below 2e-4 against a float64 sum), plus pitched layouts, fp16 activations and the error contract."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as O
from pocketllm_amd import qwen_fp8_ops as Q

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _case(rng, batch, rows, cols, wstride=None, sstride=None, nan_free=True):
    wstride = cols if wstride is None else wstride
    sstride = (cols + 127) // 128 if sstride is None else sstride
    weight = rng.integers(0, 256, size=rows * wstride, dtype=np.uint8)
    if nan_free:
        weight[(weight & 0x7F) == 0x7F] = 0x70               # 0x7f / 0xff are NaN; checkpoints never store them (reference test: 141-146)
    scale = rng.uniform(0.01, 0.4, size=((rows + 127) // 128) * sstride).astype(np.float32).astype(np.float16)
    x = rng.uniform(-1.5, 1.5, size=(batch, cols)).astype(np.float32)
    return x, weight, scale.view(np.uint16), wstride, sstride


def _max_rel(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want) / np.maximum(1.0, np.abs(want))))


CASES = [(1, 384, 640), (1, 130, 300), (4, 256, 512), (9, 128, 256), (64, 130, 300), (130, 130, 300), (256, 256, 512)]


@pytest.mark.parametrize("batch,rows,cols", CASES)
def test_reference_test_cases(batch, rows, cols):
    rng = np.random.default_rng(0x5EED1234 + rows)
    x, weight, scale, wstride, sstride = _case(rng, batch, rows, cols)
    want = O.fp8_fp16scale_matmul(x, weight, scale, rows, cols, wstride, sstride)
    xd, wd, sd = torch.from_numpy(x).to(DEV), torch.from_numpy(weight).to(DEV), torch.from_numpy(scale.view(np.int16)).to(DEV)
    y = torch.full((batch, rows), float("nan"), device=DEV)
    print(f"case fp16scale batch={batch} rows={rows} cols={cols}", flush=True)
    if batch == 1:
        assert Q.qwen_fp8_e4m3_fp16scale_matvec(xd, wd, sd, y, rows, cols, wstride, sstride)
    else:
        assert Q.qwen_fp8_e4m3_fp16scale_matmul_rows(xd, wd, sd, y, batch, rows, cols, cols, rows, wstride, sstride)
    torch.cuda.synchronize()
    assert _max_rel(y.cpu().numpy(), want) < 2.0e-4


@pytest.mark.parametrize("batch,rows,cols,wstride,sstride,xstride,ystride", [
    (1, 130, 300, 304, 5, 300, 130), (3, 200, 640, 768, 7, 700, 256), (20, 130, 512, 512, 4, 520, 130), (32, 384, 512, 512, 4, 512, 384),
    (2, 64, 17408, 17408, 136, 17408, 64)])
def test_pitched_layouts_and_wide_rows(batch, rows, cols, wstride, sstride, xstride, ystride):
    rng = np.random.default_rng(rows + cols + batch)
    x, weight, scale, _, _ = _case(rng, batch, rows, cols, wstride, sstride)
    want = O.fp8_fp16scale_matmul(x, weight, scale, rows, cols, wstride, sstride)
    xp = np.zeros((batch, xstride), dtype=np.float32)
    xp[:, :cols] = x
    xd, wd, sd = torch.from_numpy(xp).to(DEV), torch.from_numpy(weight).to(DEV), torch.from_numpy(scale.view(np.int16)).to(DEV)
    y = torch.full((batch, ystride), -7.0, device=DEV)
    print(f"case pitched batch={batch} rows={rows} cols={cols}", flush=True)
    assert Q.qwen_fp8_e4m3_fp16scale_matmul_rows(xd, wd, sd, y, batch, rows, cols, xstride, ystride, wstride, sstride)
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    assert _max_rel(got[:, :rows], want) < 2.0e-4
    assert np.all(got[:, rows:] == -7.0)                     # nothing written past the row


def test_fused_swiglu_matches_two_matvecs_and_the_float64_statement():
    """The reference's fused case (4352 x 5120, scales 0.5 and 0.75, x in [-1, 1]): fused against the two matvecs followed
    by silu(g) * u, and against float64."""
    rows, cols = 4352, 5120
    rng = np.random.default_rng(0x1234ABCD)
    x = rng.uniform(-1.0, 1.0, size=(1, cols)).astype(np.float32)
    gate = rng.integers(0, 256, size=rows * cols, dtype=np.uint8)
    up = rng.integers(0, 256, size=rows * cols, dtype=np.uint8)
    for w in (gate, up):
        w[(w & 0x7F) == 0x7F] = 0x70
    sc = (cols // 128) * (rows // 128)
    gs, us = np.full(sc, 0x3800, dtype=np.uint16), np.full(sc, 0x3A00, dtype=np.uint16)
    xd = torch.from_numpy(x).to(DEV)
    gd, ud = torch.from_numpy(gate).to(DEV), torch.from_numpy(up).to(DEV)
    gsd, usd = torch.from_numpy(gs.view(np.int16)).to(DEV), torch.from_numpy(us.view(np.int16)).to(DEV)
    g, u, fused = (torch.empty(1, rows, device=DEV) for _ in range(3))
    assert Q.qwen_fp8_e4m3_fp16scale_matvec(xd, gd, gsd, g, rows, cols, cols, cols // 128)
    assert Q.qwen_fp8_e4m3_fp16scale_matvec(xd, ud, usd, u, rows, cols, cols, cols // 128)
    assert Q.qwen_fp8_e4m3_fp16scale_swiglu_matvec(xd, gd, gsd, ud, usd, fused, rows, cols, cols, cols // 128)
    torch.cuda.synchronize()
    two_step = (torch.nn.functional.silu(g) * u).cpu().numpy().astype(np.float64)
    assert _max_rel(fused.cpu().numpy(), two_step) <= 2.0e-4
    want = O.silu_mul(O.fp8_fp16scale_matmul(x, gate, gs, rows, cols, cols, cols // 128), O.fp8_fp16scale_matmul(x, up, us, rows, cols, cols, cols // 128))
    assert O.rel_l2(fused.cpu().numpy(), want) < 1.0e-5       # outputs are products of two sums of ~1e3: judged on the whole vector


@pytest.mark.parametrize("batch,rows,cols", [(1, 130, 300), (4, 100, 512), (3, 37, 17408), (1, 2100, 8192)])
def test_fused_swiglu_small_batch_and_fp16_storage(batch, rows, cols):
    rng = np.random.default_rng(rows * 3 + cols)
    x, gate, gscale, wstride, sstride = _case(rng, batch, rows, cols)
    _, up, uscale, _, _ = _case(rng, batch, rows, cols)
    shrink = np.float16(0.05 if cols <= 1024 else 0.005)      # keeps silu(g) * u inside fp16's range for the fp16-storage pass
    gscale = (gscale.view(np.float16) * shrink).view(np.uint16)
    uscale = (uscale.view(np.float16) * shrink).view(np.uint16)
    dev = lambda a: torch.from_numpy(a.view(np.int16) if a.dtype == np.uint16 else a).to(DEV)
    for dt, tol in ((torch.float32, 2.0e-4), (torch.float16, 2.0e-3)):
        xd = dev(x).to(dt)
        xf = xd.float().cpu().numpy()
        want = O.silu_mul(O.fp8_fp16scale_matmul(xf, gate, gscale, rows, cols, wstride, sstride),
                          O.fp8_fp16scale_matmul(xf, up, uscale, rows, cols, wstride, sstride))
        y = torch.empty(batch, rows, device=DEV, dtype=dt)
        print(f"case swiglu batch={batch} rows={rows} cols={cols} {dt}", flush=True)
        assert Q.qwen_fp8_e4m3_fp16scale_swiglu_matvec(xd, dev(gate), dev(gscale), dev(up), dev(uscale), y, rows, cols, wstride, sstride, batch=batch)
        torch.cuda.synchronize()
        assert _max_rel(y.float().cpu().numpy(), want) < tol


@pytest.mark.parametrize("batch,rows,cols", [(64, 256, 512), (200, 130, 768), (16, 384, 5120)])
def test_fp16_storage_rows_take_the_tile_kernel(batch, rows, cols):
    """fp16 activations and outputs (the reference's _f16 variants, bound 3e-2 in cpp_engine/tests/test_qwen_half_ops.cpp:651-730;
    here 2e-3 of the output scale): 16 rows or more run on the matrix cores."""
    rng = np.random.default_rng(batch + rows)
    x, weight, scale, wstride, sstride = _case(rng, batch, rows, cols)
    scale = (scale.view(np.float16) * np.float16(0.05)).view(np.uint16)
    xd = torch.from_numpy(x).to(DEV).half()
    want = O.fp8_fp16scale_matmul(xd.float().cpu().numpy(), weight, scale, rows, cols, wstride, sstride)
    y = torch.empty(batch, rows, device=DEV, dtype=torch.float16)
    print(f"case fp16 rows batch={batch} rows={rows} cols={cols}", flush=True)
    assert Q.qwen_fp8_e4m3_fp16scale_matmul_rows(xd, torch.from_numpy(weight).to(DEV), torch.from_numpy(scale.view(np.int16)).to(DEV), y,
                                                 batch, rows, cols, cols, rows, wstride, sstride)
    torch.cuda.synchronize()
    assert O.rel_l2(y.float().cpu().numpy(), want) < 2.0e-3


@pytest.mark.parametrize("batch,rows,cols", [(1, 384, 640), (1, 130, 300), (9, 128, 256)])
def test_bf16_scale_compatibility_forms(batch, rows, cols):
    """Scale table as bf16 bits (the checkpoint's storage, cpp_engine/tests/test_qwen_fp8_online.cpp:150-156): the expectation is the
    fp16-scale statement evaluated on the same scale values, which are chosen exactly representable in both formats."""
    rng = np.random.default_rng(rows + batch)
    x, weight, _, wstride, sstride = _case(rng, batch, rows, cols)
    sc = (rng.integers(3, 100, size=((rows + 127) // 128) * sstride).astype(np.float32) / np.float32(256.0))   # 7 significant bits
    bf16_bits = (sc.view(np.uint32) >> 16).astype(np.uint16)
    want = O.fp8_fp16scale_matmul(x, weight, sc.astype(np.float16).view(np.uint16), rows, cols, wstride, sstride)
    y = torch.empty(batch, rows, device=DEV)
    dev = lambda a: torch.from_numpy(a.view(np.int16) if a.dtype == np.uint16 else a).to(DEV)
    if batch == 1:
        assert Q.qwen_fp8_e4m3_bf16_matvec(dev(x), dev(weight), dev(bf16_bits), y, rows, cols, wstride, sstride)
    else:
        assert Q.qwen_fp8_e4m3_bf16_matmul_rows(dev(x), dev(weight), dev(bf16_bits), y, batch, rows, cols, cols, rows, wstride, sstride)
    torch.cuda.synchronize()
    assert _max_rel(y.cpu().numpy(), want) < 2.0e-4


def test_bad_arguments_return_false_and_write_nothing():
    """cpp_engine/cuda/qwen_fp8_ops.cu:951-955, 969-970, 1087-1088: null pointers, non-positive sizes, pitches below the
    extent: false, no launch."""
    rng = np.random.default_rng(3)
    x, weight, scale, wstride, sstride = _case(rng, 2, 130, 300)
    xd, wd, sd = torch.from_numpy(x).to(DEV), torch.from_numpy(weight).to(DEV), torch.from_numpy(scale.view(np.int16)).to(DEV)
    y = torch.full((2, 130), 5.0, device=DEV)
    assert not Q.qwen_fp8_e4m3_fp16scale_matvec(xd, wd, sd, y, 0, 300, 300, 3)
    assert not Q.qwen_fp8_e4m3_fp16scale_matvec(xd, wd, sd, y, 130, 300, 299, 3)          # weight pitch below cols
    assert not Q.qwen_fp8_e4m3_fp16scale_matvec(xd, wd, sd, y, 130, 300, 300, 2)          # scale pitch below ceil(cols / 128)
    assert not Q.qwen_fp8_e4m3_fp16scale_matvec(xd, wd, None, y, 130, 300, 300, 3)
    assert not Q.qwen_fp8_e4m3_fp16scale_matmul_rows(xd, wd, sd, y, 0, 130, 300, 300, 130, 300, 3)
    assert not Q.qwen_fp8_e4m3_fp16scale_matmul_rows(xd, wd, sd, y, 2, 130, 300, 299, 130, 300, 3)
    assert not Q.qwen_fp8_e4m3_fp16scale_matmul_rows(xd, wd, sd, y, 2, 130, 300, 300, 129, 300, 3)
    assert not Q.qwen_fp8_e4m3_fp16scale_swiglu_matvec(xd, wd, sd, None, sd, y, 130, 300, 300, 3)
    assert not Q.qwen_fp8_e4m3_fp16scale_matvec(xd.cpu(), wd, sd, y, 130, 300, 300, 3)
    torch.cuda.synchronize()
    assert bool((y == 5.0).all())
