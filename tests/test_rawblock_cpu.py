"""The plain-C restatement of the raw-block matvec (oracle/rawblock_cpu.c, the benchmark's OpenMP CPU baseline) against the
numpy oracle, which the reference-written vectors pin.  CPU only."""
import numpy as np
import pytest

from oracle import gguf_oracle as O
from oracle import rawblock_cpu as R
from pocketllm_amd import block_codec as C

pytestmark = pytest.mark.skipif(not R.available(), reason="oracle/_build not built (make -C oracle cpu)")


@pytest.mark.parametrize("type_name,k", [("q4_k", 256), ("q4_k", 1000), ("q5_k", 768), ("q5_k", 2050)])
def test_superblock_matvec_matches_the_numpy_oracle(type_name, k):
    rng = np.random.default_rng(k)
    kp = (k + 255) // 256 * 256
    enc = {"q4_k": C.quantize_q4_k, "q5_k": C.quantize_q5_k}[type_name]
    blocks = enc((rng.standard_normal((41, kp)) * 0.02).astype(np.float32))
    # random bytes too: every scale / min index branch and every fifth-bit plane is live
    raw = rng.integers(0, 256, size=blocks.shape, dtype=np.uint8)
    raw[..., 0:4] = blocks[..., 0:4]
    x = rng.standard_normal((3, k)).astype(np.float32)
    for b in (blocks, raw):
        want = O.matmul_f(x, O.dequant_rows(b, type_name, k))
        assert O.rel_l2(R.matvec(b, type_name, x), want) <= 2e-6


def test_q8_0_matvec_and_dequantize():
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((37, 160)) * 0.02).astype(np.float32)
    blocks = C.pack_q8_0(w)
    np.testing.assert_array_equal(R.q8_0_dequantize(blocks), O.dequant_rows(blocks, "q8_0", 160))
    for k in (160, 150):
        x = rng.standard_normal((2, k)).astype(np.float32)
        want = O.matmul_f(x, O.dequant_rows(blocks, "q8_0", 160)[:, :k])
        assert O.rel_l2(R.matvec(blocks, "q8_0", x), want) <= 2e-6
    # subnormal and negative fp16 scales decode as IEEE half
    blocks[0, 0, 0:2] = np.array([0x01, 0x80], dtype=np.uint8)       # -2^-24
    blocks[0, 1, 0:2] = np.array([0xff, 0x03], dtype=np.uint8)       # largest subnormal
    np.testing.assert_array_equal(R.q8_0_dequantize(blocks), O.dequant_rows(blocks, "q8_0", 160))
