"""CPU restatement (numpy) of the reference's raw-block decoders and of its dequantize-then-matmul path.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the benchmark's CPU-baseline
leg, never by the shipped package.

Every function cites the reference lines it follows (paths relative to the reference checkout).
All decoder arithmetic is float32, in the reference's operand order; every product in the GGUF
decoders is exactly representable in float32, so only the final subtraction of the K-quants rounds.

How each function is pinned (what a wrong sign / index / transposed operand would trip over):
  dequant_iq1_m      reference-held golden vector tests/data/iq1m_oracle.json (bit-exact).
  dequant_q2_k,
  dequant_iq2_xxs    the reference's own C++ CPU kernels (deepseek_cpu_moe_ext.cpp) compiled into
                     oracle/_ref and probed with unit vectors, which returns single weights exactly.
  dequant_q8_0       closed form d*q on hand-built blocks; fixtures written by the reference reader.
  dequant_q4_k,
  dequant_q5_k       hand-built blocks that isolate every field (scale index j<4 / j>=4, nibble
                     halves, qh bit planes) plus fixtures written by the reference's numpy reader.
  dequant_iq2_xs,
  dequant_iq3_xxs    fixtures written by the reference's numpy reader, hand-built blocks with one live
                     entry (grid id, sign index and parity bit, both scale nibbles / the 4-bit scale).
  dequant_q6_k,
  dequant_iq4_xs     fixtures written by the reference's numpy reader, hand-built blocks with one
                     live field (every scale index, both nibble halves, every qh bit pair / high
                     scale bit pair), and a per-weight scalar restatement of the ggml layout.
  fp8_e4m3_decode    torch's float8_e4m3fn cast over all 256 codes.
  q8_1_quantize,
  fp8_act_quant      invariants (|q*d - x| <= d/2, clamp range) and torch's e4m3 cast.
  swiglu_route       closed form on hand values, both with and without the clamp.
  group_routes       invariants (monotone segment starts, multiset of routes preserved).
  fp8_fp16scale_matmul  the decode against the C++ engine's bit-trick decoder restated from its description (all 254
                     non-NaN codes), the pitched indexing against a plain loop on an unaligned case.
  silu_mul, rms_norm closed forms on hand values (constant rows, scale invariance at eps = 0, zero row).
  route_topk         hand-computed cases: a bias that changes the selection but not the weights, softmax routing
                     against softmax -> top-k -> renormalise, equal scores in expert order.
  matmul_f, moe_forward, fp8_gemm_q   float64 compositions of the pinned pieces above (no arithmetic of their own
                     beyond a matrix product).
"""
from __future__ import annotations

import math
import re
from functools import lru_cache
from pathlib import Path

import numpy as np

_CODEBOOK_FILE = Path(__file__).resolve().parents[1] / "pocketllm_amd" / "csrc" / "ggml_codebooks.inc"

# type_id map of the reference: src/loader/gguf/quant_types.py:3-13, src/csrc/cuda_kernel.cpp:401-412
TYPE_IDS = {"iq2_xxs": 0, "q2_k": 1, "iq1_m": 2, "q4_k": 3, "q5_k": 4, "iq2_xs": 5, "iq3_xxs": 6, "iq4_xs": 7, "q6_k": 8}
TYPE_NAMES = {v: k for k, v in TYPE_IDS.items()}
BLOCK_BYTES = {"q8_0": 34, "iq2_xxs": 66, "q2_k": 84, "iq1_m": 56, "q4_k": 144, "q5_k": 176, "iq4_xs": 136, "q6_k": 210, "iq2_xs": 74, "iq3_xxs": 98, "q3_k": 110}
BLOCK_ELEMS = {"q8_0": 32, "iq2_xxs": 256, "q2_k": 256, "iq1_m": 256, "q4_k": 256, "q5_k": 256, "iq4_xs": 256, "q6_k": 256, "iq2_xs": 256, "iq3_xxs": 256, "q3_k": 256}


# --------------------------------------------------------------------------------------------
# codebooks
# --------------------------------------------------------------------------------------------

def _parse_table(name: str) -> list[int]:
    text = _CODEBOOK_FILE.read_text(encoding="utf-8")
    m = re.search(r"PLLM_TABLE_U\d+\(%s,\s*\d+\)(.*?)PLLM_TABLE_END" % re.escape(name), text, flags=re.S)
    if m is None:
        raise RuntimeError(f"table {name} not found in {_CODEBOOK_FILE}")
    return [int(v, 16) for v in re.findall(r"0x[0-9a-fA-F]+", m.group(1))]


@lru_cache(maxsize=1)
def iq2xxs_grid_u8() -> np.ndarray:
    """(256, 8) uint8 magnitudes. Reference: src/loader/gguf/tensor_reader.py:23-88."""
    vals = np.asarray(_parse_table("PLLM_IQ2XXS_GRID"), dtype="<u8")
    return vals.view(np.uint8).reshape(256, 8).copy()


@lru_cache(maxsize=1)
def ksigns_u8() -> np.ndarray:
    """(128,) sign bytes: idx | parity(idx) << 7. Reference: tensor_reader.py:205-215."""
    return np.asarray([i | ((bin(i).count("1") & 1) << 7) for i in range(128)], dtype=np.uint8)


@lru_cache(maxsize=1)
def iq2xxs_signed_grid() -> np.ndarray:
    """(256, 128, 8) int8 sign-expanded grid. Reference: tensor_reader.py:205-215."""
    base = iq2xxs_grid_u8().astype(np.int16)
    bits = (ksigns_u8()[:, None] >> np.arange(8)[None, :]) & 1
    signs = np.where(bits != 0, -1, 1).astype(np.int16)
    return (base[:, None, :] * signs[None, :, :]).astype(np.int8)


@lru_cache(maxsize=1)
def iq1_grid_i8() -> np.ndarray:
    """(2048, 8) int8 in {-1, 0, 1}. Reference: src/loader/gguf/iq1_grid.py:313-321."""
    packed = np.asarray(_parse_table("PLLM_IQ1_GRID_PACKED"), dtype=np.uint16)
    vals = (packed[:, None] >> (2 * np.arange(8, dtype=np.uint16))[None, :]) & 3
    return (vals.astype(np.int8) - 1).astype(np.int8)


# --------------------------------------------------------------------------------------------
# block decoders: uint8 [..., block_bytes] -> float32 [..., block_elems]
# --------------------------------------------------------------------------------------------

def _f16(b: np.ndarray) -> np.ndarray:
    """Two little-endian bytes -> float32. Reference: tensor_reader.py:131-132."""
    return np.ascontiguousarray(b).view("<f2").astype(np.float32).reshape(b.shape[:-1])


def dequant_q8_0(blocks: np.ndarray) -> np.ndarray:
    """w[i] = d * qs[i]. Reference: tensor_reader.py:543-550, src/kernels/ops.py:734-741."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 34
    d = _f16(blocks[..., 0:2])
    qs = np.ascontiguousarray(blocks[..., 2:34]).view(np.int8).astype(np.float32)
    return qs * d[..., None]


def scale_min_k4(scales: np.ndarray, j: int):
    """6-bit (scale, min) pair j of a 12-byte K-quant scales field. Reference: tensor_reader.py:135-146."""
    if j < 4:
        return scales[..., j] & 63, scales[..., j + 4] & 63
    sc = (scales[..., j + 4] & 0x0F) | ((scales[..., j - 4] >> 6) << 4)
    mn = (scales[..., j + 4] >> 4) | ((scales[..., j] >> 6) << 4)
    return sc, mn


def dequant_q4_k(blocks: np.ndarray) -> np.ndarray:
    """Reference: tensor_reader.py:786-812 (also cuda_kernel_impl.cu:6039-6054)."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 144
    d = _f16(blocks[..., 0:2])[..., None]
    dmin = _f16(blocks[..., 2:4])[..., None]
    scales = blocks[..., 4:16]
    qs = blocks[..., 16:144]
    out = np.empty(blocks.shape[:-1] + (256,), dtype=np.float32)
    for pair in range(4):
        q = qs[..., 32 * pair:32 * pair + 32]
        sc, mn = scale_min_k4(scales, 2 * pair)
        out[..., 64 * pair:64 * pair + 32] = (
            d * sc.astype(np.float32)[..., None] * (q & 0x0F).astype(np.float32)
            - dmin * mn.astype(np.float32)[..., None])
        sc, mn = scale_min_k4(scales, 2 * pair + 1)
        out[..., 64 * pair + 32:64 * pair + 64] = (
            d * sc.astype(np.float32)[..., None] * (q >> 4).astype(np.float32)
            - dmin * mn.astype(np.float32)[..., None])
    return out


def dequant_q5_k(blocks: np.ndarray) -> np.ndarray:
    """Reference: tensor_reader.py:823-857 (also cuda_kernel_impl.cu:6056-6077)."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 176
    d = _f16(blocks[..., 0:2])[..., None]
    dmin = _f16(blocks[..., 2:4])[..., None]
    scales = blocks[..., 4:16]
    qh = blocks[..., 16:48]
    qs = blocks[..., 48:176]
    out = np.empty(blocks.shape[:-1] + (256,), dtype=np.float32)
    for pair in range(4):
        q = qs[..., 32 * pair:32 * pair + 32]
        hi0 = ((qh >> (2 * pair)) & 1).astype(np.float32) * np.float32(16.0)
        hi1 = ((qh >> (2 * pair + 1)) & 1).astype(np.float32) * np.float32(16.0)
        sc, mn = scale_min_k4(scales, 2 * pair)
        out[..., 64 * pair:64 * pair + 32] = (
            d * sc.astype(np.float32)[..., None] * ((q & 0x0F).astype(np.float32) + hi0)
            - dmin * mn.astype(np.float32)[..., None])
        sc, mn = scale_min_k4(scales, 2 * pair + 1)
        out[..., 64 * pair + 32:64 * pair + 64] = (
            d * sc.astype(np.float32)[..., None] * ((q >> 4).astype(np.float32) + hi1)
            - dmin * mn.astype(np.float32)[..., None])
    return out


def dequant_q2_k(blocks: np.ndarray) -> np.ndarray:
    """Reference: tensor_reader.py:592-614 (also deepseek_cpu_moe_ext.cpp:280-302)."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 84
    scales = blocks[..., 0:16]
    qs = blocks[..., 16:80]
    d = _f16(blocks[..., 80:82])[..., None]
    dmin = _f16(blocks[..., 82:84])[..., None]
    out = np.empty(blocks.shape[:-1] + (256,), dtype=np.float32)
    for group in range(16):
        half, gi = divmod(group, 8)
        shift = 2 * (gi // 2)
        start = 32 * half + 16 * (gi % 2)
        q = ((qs[..., start:start + 16] >> shift) & 3).astype(np.float32)
        sc = (scales[..., group] & 0x0F).astype(np.float32)[..., None]
        mn = (scales[..., group] >> 4).astype(np.float32)[..., None]
        out[..., 16 * group:16 * group + 16] = d * sc * q - dmin * mn
    return out


def dequant_iq2_xxs(blocks: np.ndarray) -> np.ndarray:
    """Reference: tensor_reader.py:625-652."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 66
    d = _f16(blocks[..., 0:2])[..., None]
    qs = blocks[..., 2:66]
    grid = iq2xxs_signed_grid()
    out = np.empty(blocks.shape[:-1] + (256,), dtype=np.float32)
    for sub in range(8):
        chunk = qs[..., 8 * sub:8 * sub + 8]
        aux = (chunk[..., 4].astype(np.uint32) | (chunk[..., 5].astype(np.uint32) << 8)
               | (chunk[..., 6].astype(np.uint32) << 16) | (chunk[..., 7].astype(np.uint32) << 24))
        ls = (2 * (aux >> 28) + 1).astype(np.float32)[..., None]
        for part in range(4):
            ids = chunk[..., part].astype(np.int64)
            sidx = ((aux >> (7 * part)) & 127).astype(np.int64)
            vals = grid[ids, sidx].astype(np.float32)
            start = 32 * sub + 8 * part
            out[..., start:start + 8] = np.float32(0.125) * d * ls * vals
    return out


def dequant_iq1_m(blocks: np.ndarray) -> np.ndarray:
    """Reference: tensor_reader.py:957-1000 (also cuda_kernel_impl.cu:6224-6263)."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 56
    lead = blocks.shape[:-1]
    b = np.ascontiguousarray(blocks).reshape(-1, 56)
    n = b.shape[0]
    qs = b[:, 0:32]
    qh = b[:, 32:48]
    sc = np.ascontiguousarray(b[:, 48:56]).view("<u2").reshape(n, 4)
    dbits = ((sc[:, 0] >> 12) | ((sc[:, 1] >> 12) << 4) | ((sc[:, 2] >> 12) << 8) | (sc[:, 3] & 0xF000)).astype(np.uint16)
    d = dbits.view(np.float16).astype(np.float32)
    grid = iq1_grid_i8().astype(np.float32)
    out = np.empty((n, 256), dtype=np.float32)
    for j in range(32):                     # one codebook index per 8 weights
        s = j >> 1                          # 16-weight scale group
        ls = (sc[:, s >> 2] >> (3 * (s & 3))) & 7
        dl = d * (2 * ls + 1).astype(np.float32)
        h = (qh[:, j >> 1] >> (4 * (j & 1))) & 15
        idx = qs[:, j].astype(np.int64) | ((h & 7).astype(np.int64) << 8)
        delta = np.where((h & 8) != 0, np.float32(-0.125), np.float32(0.125)).astype(np.float32)
        out[:, 8 * j:8 * j + 8] = dl[:, None] * (grid[idx] + delta[:, None])
    return out.reshape(lead + (256,))


@lru_cache(maxsize=1)
def iq2xs_grid_u8() -> np.ndarray:
    """(512, 8) uint8 magnitudes. Reference: tensor_reader.py:167-169 (parsed there from ggml-common.h)."""
    return np.asarray(_parse_table("PLLM_IQ2XS_GRID"), dtype="<u8").view(np.uint8).reshape(512, 8).copy()


@lru_cache(maxsize=1)
def iq3xxs_grid_u8() -> np.ndarray:
    """(256, 4) uint8 magnitudes. Reference: tensor_reader.py:172-174."""
    return np.asarray(_parse_table("PLLM_IQ3XXS_GRID"), dtype="<u4").view(np.uint8).reshape(256, 4).copy()


def _sign_table() -> np.ndarray:
    """(128, 8) float32 of +-1: bit j of the 7-bit index, bit 7 = parity of the others (tensor_reader.py:183-187)."""
    idx = np.arange(128)
    parity = np.zeros(128, dtype=np.int64)
    for b in range(7):
        parity ^= (idx >> b) & 1
    full = idx | (parity << 7)
    return np.where((full[:, None] >> np.arange(8)) & 1, np.float32(-1.0), np.float32(1.0)).astype(np.float32)


def dequant_iq2_xs(blocks: np.ndarray) -> np.ndarray:
    """IQ2_XS: d(f16) qs u16[32] scales(8).  Entry e (8 weights): grid id = low 9 bits, sign index = high 7 bits of qs[e];
    sub-block s = e // 4 (32 weights) has two 4-bit scales, the low nibble for its first 16 weights, the high nibble for the
    others; w = 0.25 * d * (ls + 0.5) * grid * sign.  Reference: tensor_reader.py:663-690."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 74
    lead = blocks.shape[:-1]
    b = blocks.reshape(-1, 74)
    d = _f16(b[:, 0:2])
    qs = b[:, 2:66].astype(np.uint16)
    q = qs[:, 0::2] | (qs[:, 1::2] << 8)                                    # [n, 32]
    scales = b[:, 66:74]
    grid = iq2xs_grid_u8().astype(np.float32)
    signs = _sign_table()
    out = np.empty((b.shape[0], 256), dtype=np.float32)
    for e in range(32):
        sub, part = divmod(e, 4)
        ls = ((scales[:, sub] & 0x0F) if part < 2 else (scales[:, sub] >> 4)).astype(np.float32)
        values = grid[q[:, e] & 0x1FF] * signs[q[:, e] >> 9]
        out[:, 8 * e:8 * e + 8] = np.float32(0.25) * d[:, None] * (ls + np.float32(0.5))[:, None] * values
    return out.reshape(lead + (256,))


def dequant_iq3_xxs(blocks: np.ndarray) -> np.ndarray:
    """IQ3_XXS: d(f16) grid ids(64) aux u32[8].  Sub-block s (32 weights): ids qs[8 s + k] give four weights each from the
    256-entry grid; aux_s holds four 7-bit sign indices (one per 8 weights) and a 4-bit scale; w = 0.5 * d * (ls + 0.5) * grid * sign.
    Reference: tensor_reader.py:700-735."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 98
    lead = blocks.shape[:-1]
    b = blocks.reshape(-1, 98)
    d = _f16(b[:, 0:2])
    ids = b[:, 2:66]
    aux = b[:, 66:98].astype(np.uint32)
    aux = aux[:, 0::4] | (aux[:, 1::4] << 8) | (aux[:, 2::4] << 16) | (aux[:, 3::4] << 24)      # [n, 8]
    grid = iq3xxs_grid_u8().astype(np.float32)
    signs = _sign_table()
    out = np.empty((b.shape[0], 256), dtype=np.float32)
    for sub in range(8):
        ls = (aux[:, sub] >> 28).astype(np.float32)
        for part in range(8):
            sg = signs[(aux[:, sub] >> (7 * (part // 2))) & 127][:, 4 * (part % 2):4 * (part % 2) + 4]
            values = grid[ids[:, 8 * sub + part]] * sg
            start = 32 * sub + 4 * part
            out[:, start:start + 4] = np.float32(0.5) * d[:, None] * (ls + np.float32(0.5))[:, None] * values
    return out.reshape(lead + (256,))


def dequant_q6_k(blocks: np.ndarray) -> np.ndarray:
    """Q6_K: ql(128) qh(64) scales int8(16) d(f16); w = d * scales[i // 16] * (q - 32), q = 4 low bits from ql and 2
    high bits from qh.  Reference: tensor_reader.py:868-908."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 210
    ql = blocks[..., 0:128]
    qh = blocks[..., 128:192]
    scales = blocks[..., 192:208].view(np.int8).astype(np.float32)
    d = _f16(blocks[..., 208:210])[..., None]
    out = np.empty(blocks.shape[:-1] + (256,), dtype=np.float32)
    for half in range(2):
        ql_a = ql[..., 64 * half:64 * half + 32]
        ql_b = ql[..., 64 * half + 32:64 * half + 64]
        qh_h = qh[..., 32 * half:32 * half + 32]
        sc = scales[..., 8 * half:8 * half + 8]
        quads = (
            (ql_a & 0x0F) | (((qh_h >> 0) & 3) << 4),
            (ql_b & 0x0F) | (((qh_h >> 2) & 3) << 4),
            (ql_a >> 4) | (((qh_h >> 4) & 3) << 4),
            (ql_b >> 4) | (((qh_h >> 6) & 3) << 4),
        )
        for j, q in enumerate(quads):
            # weights 128 half + 32 j + l, l < 32: scale index 2 j + l // 16 of the half
            scale = np.repeat(sc[..., 2 * j:2 * j + 2], 16, axis=-1)
            out[..., 128 * half + 32 * j:128 * half + 32 * j + 32] = d * scale * (q.astype(np.int16) - 32).astype(np.float32)
    return out


def dequant_q3_k(blocks: np.ndarray) -> np.ndarray:
    """Q3_K as the reference's reader decodes it: hmask(32) qs(64) scales(12) d(f16), sixteen groups of 16 weights.
    Group g: scale = nibble g of the first eight scale bytes (low nibbles for g < 8, high nibbles of byte g - 8 else) minus 8;
    weight j of the group: two low bits (qs[4 g + j % 4] >> 2 (j // 4)) & 3, minus 4 when bit j % 8 of hmask[2 g + j // 8] is
    clear; w = (d * scale) * q in float32.  Reference: tensor_reader.py:746-776 (its own layout: the last four scale bytes
    are not read).  The reference gives this type no type id and no device kernel; only the decoder exists."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 110
    hmask = blocks[..., 0:32]
    qs = blocks[..., 32:96]
    scales = blocks[..., 96:108]
    d = _f16(blocks[..., 108:110])
    out = np.empty(blocks.shape[:-1] + (256,), dtype=np.float32)
    j = np.arange(16)
    for g in range(16):
        nib = (scales[..., g] & 0x0F) if g < 8 else (scales[..., g - 8] >> 4)
        scale = (nib.astype(np.int16) - 8).astype(np.float32)
        low = (qs[..., 4 * g + (j & 3)] >> (2 * (j >> 2)).astype(np.uint8)) & 3
        bit = (hmask[..., 2 * g + (j >> 3)] >> (j & 7).astype(np.uint8)) & 1
        q = low.astype(np.int16) - np.where(bit == 0, 4, 0).astype(np.int16)
        out[..., 16 * g:16 * g + 16] = (d * scale)[..., None] * q.astype(np.float32)
    return out


IQ4_KVALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)


def dequant_iq4_xs(blocks: np.ndarray) -> np.ndarray:
    """IQ4_XS: d(f16) scales_h(u16) scales_l(4) qs(128); per 32 weights a 6-bit scale (4 low bits from scales_l, 2 high
    bits from scales_h) minus 32; 16 bytes per group, low nibbles = weights 0..15, high nibbles = weights 16..31, codes
    through the 16-entry non-linear table.  Reference: tensor_reader.py:918-948."""
    assert blocks.dtype == np.uint8 and blocks.shape[-1] == 136
    d = _f16(blocks[..., 0:2])[..., None]
    scales_h = (blocks[..., 2].astype(np.uint16) | (blocks[..., 3].astype(np.uint16) << 8))
    scales_l = blocks[..., 4:8]
    qs = blocks[..., 8:136]
    out = np.empty(blocks.shape[:-1] + (256,), dtype=np.float32)
    for g in range(8):
        lo4 = (scales_l[..., g // 2] >> (4 if g & 1 else 0)) & 0x0F
        hi2 = (scales_h >> (2 * g)) & 3
        scale = ((lo4.astype(np.int16) | (hi2.astype(np.int16) << 4)) - 32).astype(np.float32)[..., None]
        q = qs[..., 16 * g:16 * g + 16]
        out[..., 32 * g:32 * g + 16] = d * scale * IQ4_KVALUES[q & 0x0F]
        out[..., 32 * g + 16:32 * g + 32] = d * scale * IQ4_KVALUES[q >> 4]
    return out


_DECODERS = {
    "q3_k": dequant_q3_k,
    "q8_0": dequant_q8_0, "q4_k": dequant_q4_k, "q5_k": dequant_q5_k,
    "q2_k": dequant_q2_k, "iq2_xxs": dequant_iq2_xxs, "iq1_m": dequant_iq1_m,
    "q6_k": dequant_q6_k, "iq4_xs": dequant_iq4_xs, "iq2_xs": dequant_iq2_xs, "iq3_xxs": dequant_iq3_xxs,
}


def dequant_rows(blocks: np.ndarray, type_name: str, row_elems: int | None = None) -> np.ndarray:
    """uint8 [..., blocks_per_row, block_bytes] -> float32 [..., row_elems].

    Reference: tensor_reader.py:566-590 (`_read_quantized_matrix`: decode, reshape, cut the K tail).
    """
    vals = _DECODERS[type_name](blocks)
    vals = vals.reshape(blocks.shape[:-2] + (blocks.shape[-2] * BLOCK_ELEMS[type_name],))
    if row_elems is not None:
        vals = vals[..., :row_elems]
    return np.ascontiguousarray(vals)


# --------------------------------------------------------------------------------------------
# FP8 E4M3FN with 128x128 block scales
# --------------------------------------------------------------------------------------------

def fp8_e4m3_decode(codes: np.ndarray) -> np.ndarray:
    """OCP E4M3FN byte -> float32 (0x7f / 0xff are NaN).

    Closed form as in cpp_engine/tests/test_fp8_matvec.cpp:59-67; the Python reference relies on
    torch's cast (src/kernels/ops.py:144-147).
    """
    c = codes.astype(np.int32)
    sign = np.where((c & 0x80) != 0, np.float32(-1.0), np.float32(1.0))
    e = (c >> 3) & 15
    m = (c & 7).astype(np.float32)
    sub = m / np.float32(8.0) * np.float32(2.0 ** -6)
    nor = (np.float32(1.0) + m / np.float32(8.0)) * np.exp2((e - 7).astype(np.float32)).astype(np.float32)
    val = np.where(e == 0, sub, nor).astype(np.float32)
    val = np.where((c & 0x7F) == 0x7F, np.float32(np.nan), val)
    return (sign * val).astype(np.float32)


def dequant_fp8_block(weight: np.ndarray, scale: np.ndarray, block: int = 128) -> np.ndarray:
    """W[r, c] = f32(code[r, c]) * scale[r // 128, c // 128]. Reference: ops.py:104-107, 144-147."""
    n, k = weight.shape
    s = np.repeat(np.repeat(scale.astype(np.float32), block, axis=0)[:n], block, axis=1)[:, :k]
    return fp8_e4m3_decode(weight) * s


def fp8_fp16scale_matmul(x: np.ndarray, weight: np.ndarray, scale_bits: np.ndarray, rows: int, cols: int,
                          weight_stride: int, scale_stride: int) -> np.ndarray:
    """y[b, r] = sum_c x[b, c] * f32(code[r, c]) * f32(f16 scale[r // 128, c // 128]) in float64: the expectation the
    reference's own test builds for its C++ engine operators (cpp_engine/tests/test_qwen_fp8_online.cpp:159-171), with
    their pitches: weight is a flat byte array read at r * weight_stride + c, scale_bits a flat uint16 array read at
    (r // 128) * scale_stride + c // 128.  Pinned by: the decode (torch's cast, all codes), the fp16 bits (numpy's
    float16 view), the indexing (brute-force loop on a small unaligned case in tests/test_oracle_pinning.py)."""
    w = np.lib.stride_tricks.as_strided(weight, shape=(rows, cols), strides=(weight_stride, 1))
    tr, tc = (rows + 127) // 128, (cols + 127) // 128
    sc = np.lib.stride_tricks.as_strided(scale_bits, shape=(tr, tc), strides=(2 * scale_stride, 2)).view(np.float16).astype(np.float64)
    wf = fp8_e4m3_decode(np.ascontiguousarray(w)).astype(np.float64) * np.repeat(np.repeat(sc, 128, axis=0)[:rows], 128, axis=1)[:, :cols]
    return x.astype(np.float64) @ wf.T


def silu_mul(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """silu(g) * u, the epilogue of the fused gate/up matvec (cpp_engine/cuda/qwen_fp8_ops.cu:41-43, 815-896)."""
    g = gate.astype(np.float64)
    with np.errstate(over="ignore"):                         # exp(-g) = inf for very negative g: silu -> -0, as in float arithmetic
        return g / (1.0 + np.exp(-g)) * up.astype(np.float64)


def fp8_e4m3_encode_rne(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest E4M3FN code, ties to even, saturating at +-448 (test helper)."""
    table = fp8_e4m3_decode(np.arange(256, dtype=np.uint8))
    pos = table[:127].astype(np.float64)                       # codes 0..126 are monotone, 126 -> 448
    a = np.minimum(np.abs(x.astype(np.float64)), 448.0)
    hi = np.searchsorted(pos, a, side="left").clip(0, 126)
    lo = (hi - 1).clip(0, 126)
    dlo = a - pos[lo]
    dhi = pos[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((hi & 1) == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    return np.where(np.signbit(x), code | 0x80, code).astype(np.uint8)


def fp8_act_quant(x: np.ndarray, block: int = 128, eps: float = 1e-4):
    """Per-(row, 128) activation quantizer: s = max(amax, eps) / 448, q = clamp(x / s) -> e4m3 (RNE).

    Reference: src/kernels/ops.py:501-516.  Returns (codes uint8 [T, K], scales f32 [T, K / 128]).
    """
    t, k = x.shape
    assert k % block == 0
    xf = x.astype(np.float32).reshape(t, k // block, block)
    s = (np.maximum(np.abs(xf).max(axis=-1), np.float32(eps)) / np.float32(448.0)).astype(np.float32)
    q = np.clip(xf / s[..., None], np.float32(-448.0), np.float32(448.0)).astype(np.float32)
    return fp8_e4m3_encode_rne(q).reshape(t, k), s


# --------------------------------------------------------------------------------------------
# int8 activation quantizers (q8_1 style)
# --------------------------------------------------------------------------------------------

def q8_1_quantize(x: np.ndarray, group: int = 32):
    """scale = amax / 127 (1e-8 for an all-zero group); q = clamp(rint(x / scale), -127, 127).

    Reference: src/csrc/cuda_kernel_impl.cu:7090-7117 (group 32) and 6339-6364 (group 16).
    x [T, K] with K a multiple of `group`.  Returns (q int8 [T, K], scale f32 [T, K / group]).
    """
    t, k = x.shape
    assert k % group == 0
    xf = x.astype(np.float32).reshape(t, k // group, group)
    amax = np.abs(xf).max(axis=-1)
    scale = np.where(amax > 0, amax / np.float32(127.0), np.float32(1e-8)).astype(np.float32)
    q = np.clip(np.rint(xf / scale[..., None]), -127, 127).astype(np.int8)
    return q.reshape(t, k), scale


def pow2_image(x: np.ndarray, group: int = 32) -> np.ndarray:
    """The activations as the single-launch decode kernels of this package carry them (no counterpart in the reference, whose
    decode matvec multiplies float activations, src/csrc/cuda_kernel_impl.cu:6082-6137): per `group` values one power-of-two
    scale xs = 2^(E - 13), E the exponent of the group's largest magnitude (groups below 2^-113: E clamped, values round to
    zero), and q = rint(x / xs) with |q| <= 2^14, which the kernels split into two int8 terms q = 256 hi + lo.  Returns the
    rounded activations xs * q as float64 [T, K]: the kernels' results are the float statement of the operator applied to these.
    """
    t, k = x.shape
    assert k % group == 0
    xf = x.astype(np.float32).reshape(t, k // group, group)
    amax = np.abs(xf).max(axis=-1)
    e = np.maximum(amax.view(np.uint32) >> np.uint32(23), np.uint32(14)).astype(np.int64)      # biased exponent
    xs = np.ldexp(1.0, (e - 140).astype(np.int64))                                             # 2^(e - 127 - 13), float64
    q = np.rint(xf.astype(np.float64) / xs[..., None])                                         # exact quotient, ties to even
    assert np.abs(q).max() <= 16384
    return (q * xs[..., None]).reshape(t, k)


# --------------------------------------------------------------------------------------------
# matvec / matmul semantics
# --------------------------------------------------------------------------------------------

def matmul_f(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """Float-activation semantics: y = x @ W^T with float64 accumulation, returned as float64.

    Reference: the dequantize-then-matmul path (ops.py:782-792, tests/bench_gguf_raw_matmul.py:44-49)
    and the float block-dot kernels (cuda_kernel_impl.cu:6544-6583).
    """
    return x.astype(np.float64) @ w.astype(np.float64).T


def kquant_gemm_q(x: np.ndarray, blocks: np.ndarray, type_name: str, ds4_pair: bool = False) -> np.ndarray:
    """Int8-activation semantics for Q4_K / Q5_K (the prefill path of BASELINE config 3).

    acts -> int8 per 32 (q8_1_quantize); per 32-group g:
        y += (d * sc_g) * xs_g * sum_i(q_i * xq_i)  -  (dmin * m_g) * xs_g * sum_i(xq_i)
    with d*sc and dmin*m kept in float32 (the reference's MMQ rounds them to fp16:
    llama_mmq/mmq.cuh:2160-2165, 1374-1378; that loss is not reproduced).  Returns float64 [T, N].

    ds4_pair=True restates the activation side the way the reference's MMA path stores it (llama_mmq/gguf_mma_wrapper.cu:90-126,
    layout DS4): per 32 values the pair {fp16(amax / 127), fp16(sum of the float activations)}, codes rint(x * (1 / d)) with d the
    float32 quotient; the min term then uses the stored float sum, y -= (dmin * m_g) * fp16(sum_i x_i), and the dot term the fp16
    scale.  The library's operator is the default statement; the two are compared in tests/test_oracle_pinning.py.
    """
    assert type_name in ("q4_k", "q5_k")
    n, bpr, _ = blocks.shape
    t, k = x.shape
    assert k == bpr * 256
    if ds4_pair:
        xg = x.astype(np.float32).reshape(t, bpr * 8, 32)
        dq = (np.abs(xg).max(axis=-1) / np.float32(127.0)).astype(np.float32)
        inv = np.where(dq > 0, np.float32(1.0) / np.where(dq > 0, dq, np.float32(1.0)), np.float32(0.0)).astype(np.float32)
        xq = np.rint(xg * inv[..., None]).astype(np.int64)
        xs = dq.astype(np.float16).astype(np.float32)
        fsum = xg.sum(axis=-1, dtype=np.float32).astype(np.float16).astype(np.float64)       # [T, G]
    else:
        xq, xs = q8_1_quantize(x, 32)
        xq = xq.astype(np.int64).reshape(t, bpr * 8, 32)
        fsum = None
    xsum = xq.sum(axis=-1)                                           # [T, G]
    if type_name == "q4_k":
        d = _f16(blocks[..., 0:2]); dmin = _f16(blocks[..., 2:4]); scales = blocks[..., 4:16]
        qs = blocks[..., 16:144]; qh = None
    else:
        d = _f16(blocks[..., 0:2]); dmin = _f16(blocks[..., 2:4]); scales = blocks[..., 4:16]
        qh = blocks[..., 16:48]; qs = blocks[..., 48:176]
    q = np.empty((n, bpr, 8, 32), dtype=np.int64)
    sc = np.empty((n, bpr, 8), dtype=np.float32)
    mn = np.empty((n, bpr, 8), dtype=np.float32)
    for pair in range(4):
        qb = qs[..., 32 * pair:32 * pair + 32]
        lo = (qb & 0x0F).astype(np.int64)
        hi = (qb >> 4).astype(np.int64)
        if qh is not None:
            lo = lo + 16 * ((qh >> (2 * pair)) & 1).astype(np.int64)
            hi = hi + 16 * ((qh >> (2 * pair + 1)) & 1).astype(np.int64)
        q[:, :, 2 * pair] = lo
        q[:, :, 2 * pair + 1] = hi
        for j in (2 * pair, 2 * pair + 1):
            s, m = scale_min_k4(scales, j)
            sc[:, :, j] = d * s.astype(np.float32)
            mn[:, :, j] = dmin * m.astype(np.float32)
    q = q.reshape(n, bpr * 8, 32)
    sc = sc.reshape(n, bpr * 8).astype(np.float64)
    mn = mn.reshape(n, bpr * 8).astype(np.float64)
    out = np.zeros((t, n), dtype=np.float64)
    xs64 = xs.astype(np.float64)
    for g in range(bpr * 8):
        dots = xq[:, g, :] @ q[:, g, :].T                             # exact integers [T, N]
        if fsum is None:
            out += xs64[:, g:g + 1] * (dots * sc[None, :, g] - xsum[:, g:g + 1] * mn[None, :, g])
        else:
            out += xs64[:, g:g + 1] * dots * sc[None, :, g] - fsum[:, g:g + 1] * mn[None, :, g]
    return out


def fp8_gemm_q(x: np.ndarray, weight: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """FP8-activation semantics of the reference's act_quant + fp8_gemm pair (ops.py:982-1001,
    1043-1051): acts are quantized per (row, 128) to E4M3, dequantized, then multiplied by the
    dequantized weight.  Returns float64 [T, N]."""
    codes, s = fp8_act_quant(x)
    t, k = x.shape
    xa = fp8_e4m3_decode(codes).reshape(t, k // 128, 128) * s[..., None]
    return matmul_f(xa.reshape(t, k), dequant_fp8_block(weight, scale))


# --------------------------------------------------------------------------------------------
# routed experts
# --------------------------------------------------------------------------------------------

def swiglu_route(gate: np.ndarray, up: np.ndarray, route_w: np.ndarray, limit: float) -> np.ndarray:
    """h = silu(min(g, L)) * clamp(u, -L, L) * w, the clamp only when L > 0.

    Reference: cuda_kernel_impl.cu:241-262, deepseek_cpu_moe_ext.cpp:2826-2830.
    gate/up [R, I] float, route_w [R]."""
    g = gate.astype(np.float64)
    u = up.astype(np.float64)
    if limit > 0:
        u = np.clip(u, -limit, limit)
        g = np.minimum(g, limit)
    return g / (1.0 + np.exp(-g)) * u * route_w.astype(np.float64)[:, None]


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """x * rsqrt(mean(x^2) + eps) * weight per row, in float64 (no output rounding).

    Reference: fused_rms_norm_kernel, src/csrc/cuda_kernel_impl.cu:9639-9697 (float32 there, output rounded to fp16), and the
    framework fallback src/models/minimax_m2/architecture.py:77-85.  Pinned by closed forms in tests/test_oracle_pinning.py."""
    xf = x.astype(np.float64)
    inv = 1.0 / np.sqrt((xf * xf).mean(axis=-1, keepdims=True) + float(eps))
    return xf * inv * weight.astype(np.float64)


def route_topk(logits: np.ndarray, bias, top_k: int, softmax: bool = False):
    """Scores, top-k and renormalised weights from gate logits [T, E] (float64 arithmetic on the given logits).

    Reference: MiniMaxMoE.route, src/models/minimax_m2/architecture.py:291-298 (sigmoid, optional bias added for the
    selection only, weights = picked probabilities / max(their sum, 1e-20)); softmax=True is softmax -> top-k ->
    renormalise, which equals the softmax over the picked logits.  Picks come in descending score order, the lower expert id
    first on equal scores (the reference's topk leaves ties unspecified).  Pinned by closed-form cases in
    tests/test_oracle_pinning.py."""
    l = logits.astype(np.float64)
    if softmax:
        score, prob = l, l
    else:
        prob = 1.0 / (1.0 + np.exp(-l))
        score = prob if bias is None else prob + bias.astype(np.float64)[None, :]
    order = np.argsort(-score, axis=1, kind="stable")[:, :top_k]
    picked = np.take_along_axis(prob, order, axis=1)
    if softmax:
        ex = np.exp(picked - picked.max(axis=1, keepdims=True))
        w = ex / ex.sum(axis=1, keepdims=True)
    else:
        w = picked / np.maximum(picked.sum(axis=1, keepdims=True), 1.0e-20)
    return order.astype(np.int64), w


def group_routes(indices: np.ndarray, weights: np.ndarray, experts_start: int, n_local: int):
    """Counting sort of (token, k) routes by local expert.

    Reference: cuda_kernel_impl.cu:295-351, 4306-4377.  Returns (local_ids, route_tokens,
    route_weights, seg_starts[E + 1]); inside a segment the reference's order is unspecified
    (atomic fill), here it is ascending (token, k)."""
    t, topk = indices.shape
    local = indices.astype(np.int64) - experts_start
    toks = np.repeat(np.arange(t, dtype=np.int64), topk)
    flat_local = local.reshape(-1)
    flat_w = weights.astype(np.float32).reshape(-1)
    keep = (flat_local >= 0) & (flat_local < n_local)
    order = np.argsort(flat_local[keep], kind="stable")
    route_tokens = toks[keep][order]
    route_weights = flat_w[keep][order]
    counts = np.bincount(flat_local[keep], minlength=n_local)
    seg = np.zeros(n_local + 1, dtype=np.int32)
    seg[1:] = np.cumsum(counts)
    local_ids = np.nonzero(counts)[0].astype(np.int64)
    return local_ids, route_tokens, route_weights, seg


def moe_forward(x: np.ndarray, route_tokens: np.ndarray, route_weights: np.ndarray, route_experts: np.ndarray,
                w1: np.ndarray, w3: np.ndarray, w2: np.ndarray, t1: str, t3: str, t2: str,
                swiglu_limit: float = 0.0) -> np.ndarray:
    """y[t] = sum over routes r of token t:  W2_e · ( silu(W1_e x_t) * (W3_e x_t) * w_r ).

    Reference: cuda_kernel_impl.cu:8688-9138 (grouped) and 9140-9385 (single token);
    CPU twin deepseek_cpu_moe_ext.cpp:2759-2872.  w1/w3 uint8 [E, I, D/256, bb], w2 uint8
    [E, D, I/256, bb].  Float64 accumulation, fixed route order.  Returns float64 [T, D]."""
    t, dim = x.shape
    y = np.zeros((t, dim), dtype=np.float64)
    cache: dict[int, tuple[np.ndarray, np.ndarray, np.ndarray]] = {}
    for r in range(len(route_tokens)):
        e = int(route_experts[r])
        if e not in cache:
            cache[e] = (dequant_rows(w1[e], t1, dim).astype(np.float64),
                        dequant_rows(w3[e], t3, dim).astype(np.float64),
                        dequant_rows(w2[e], t2, w1.shape[1]).astype(np.float64))
        a, b, c = cache[e]
        xt = x[int(route_tokens[r])].astype(np.float64)
        h = swiglu_route((a @ xt)[None, :], (b @ xt)[None, :], route_weights[r:r + 1], swiglu_limit)[0]
        y[int(route_tokens[r])] += c @ h
    return y


def rel_l2(got: np.ndarray, want: np.ndarray) -> float:
    w = want.astype(np.float64)
    den = math.sqrt(float((w * w).sum()))
    num = math.sqrt(float(((got.astype(np.float64) - w) ** 2).sum()))
    return num / den if den > 0 else num
