"""Host-side proofs of the arithmetic identities the device activation quantizer relies on (CPU only)."""
import shutil
import subprocess
from pathlib import Path

import numpy as np
import pytest

from oracle import gguf_oracle as O

HERE = Path(__file__).resolve().parent


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_division_by_127_through_two_fused_multiply_adds_is_correctly_rounded(tmp_path):
    """scale = amax / 127 is formed on the device as q0 = amax * c, fma(fma(-q0, 127, amax), c, q0): exhaustive over every
    finite positive float32 (about ten seconds on eight cores)."""
    exe = tmp_path / "div127"
    subprocess.run(["gcc", "-O2", "-mfma", "-ffp-contract=off", "-fopenmp", str(HERE / "quantizer_div127.c"), "-o", str(exe), "-lm"], check=True)
    out = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True, timeout=600)
    assert out.returncode == 0 and out.stdout.strip() == "0"


def test_residual_test_certifies_the_fast_code():
    """The device takes q = rint(v * y), y ~ 1 / scale, and keeps it when |fl(v - q * scale)| < scale * (0.5 - 1e-4); otherwise it
    divides.  Restated in numpy (float64 stands in for the fused multiply-add's single rounding) on rows that sit on and next to
    rounding ties: every code the residual test lets through equals the oracle's, and the ties themselves are sent to the divider."""
    rng = np.random.default_rng(3)
    k = 1 << 16
    amax = rng.uniform(0.01, 50.0, size=k // 32).astype(np.float32)
    scale = (amax / np.float32(127.0)).astype(np.float32)
    x = (rng.integers(-126, 126, size=(k // 32, 32)).astype(np.float32) + np.float32(0.5)) * scale[:, None]
    nudge = rng.integers(-2, 3, size=x.shape)
    for step in (1, 2):
        x = np.where(nudge >= step, np.nextafter(x, np.float32(np.inf)), np.where(nudge <= -step, np.nextafter(x, np.float32(-np.inf)), x))
    x[:, 0] = amax
    x = np.concatenate([x, rng.standard_normal(x.shape).astype(np.float32) * amax[:, None] / 4]).astype(np.float32)
    x[k // 32:, 0] = amax
    want_q, want_s = O.q8_1_quantize(x.reshape(1, -1), 32)
    want_q = want_q.reshape(x.shape)
    s = want_s.reshape(-1)[:, None].astype(np.float32)
    for rel_err in (0.0, 2.0 ** -23, -(2.0 ** -23)):                      # y anywhere within an ulp of 1 / scale
        y = (np.float32(1.0) / s * np.float32(1.0 + rel_err)).astype(np.float32)
        q = np.rint(x.astype(np.float64) * y.astype(np.float64))
        r = (x.astype(np.float64) - q * s.astype(np.float64)).astype(np.float32)
        sure = np.abs(r) < (s * np.float32(0.5 - 1e-4)).astype(np.float32)
        assert sure.mean() > 0.45                                        # the random half passes, the tie half mostly does not
        np.testing.assert_array_equal(q[sure].astype(np.int8), want_q[sure])
    assert (~sure[: k // 32, 1:]).mean() > 0.9
