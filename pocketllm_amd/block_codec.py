"""Encoders and generators for raw weight blocks (host side, numpy).

The reference ships no K-quant or IQ encoder: its checkpoints come from external llama.cpp tools, and
the only quantizers in its tree are the Q8_0 test packer (tests/test_q8_0_cuda.py:12-24) and the
activation quantizers.  Synthetic benchmarks and tests still need valid blocks, so this module holds
simple encoders of this library's own.  Every correctness statement elsewhere is about
blocks -> values, never about how good an encoder is.

Layouts are the GGUF ones: Q8_0 34 B / 32 weights; Q2_K 84 B, Q4_K 144 B, Q5_K 176 B, Q6_K 210 B, IQ4_XS 136 B, IQ2_XXS 66 B,
IQ1_M 56 B per 256 weights; FP8 is one OCP E4M3FN byte per weight plus a float32 scale per 128x128.
"""
from __future__ import annotations

import numpy as np
import torch


def _f16_bytes(v: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(v.astype("<f2")).view(np.uint8).reshape(v.shape + (2,))


def _pad_rows(w: np.ndarray, multiple: int) -> np.ndarray:
    n, k = w.shape
    kp = (k + multiple - 1) // multiple * multiple
    if kp == k:
        return np.ascontiguousarray(w, dtype=np.float32)
    out = np.zeros((n, kp), dtype=np.float32)
    out[:, :k] = w
    return out


def pack_q8_0(weight: np.ndarray) -> np.ndarray:
    """float [N, K] -> uint8 [N, ceil(K/32), 34].

    scale = max(absmax, 1e-6) / 127, q = clamp(round(w / scale), +-127), scale stored as fp16:
    the recipe of the reference's test packer (tests/test_q8_0_cuda.py:12-24).
    """
    w = _pad_rows(np.asarray(weight, dtype=np.float32), 32)
    n = w.shape[0]
    v = w.reshape(n, -1, 32)
    scale = (np.maximum(np.abs(v).max(axis=-1), np.float32(1e-6)) / np.float32(127.0)).astype(np.float32)
    q = np.clip(np.rint(v / scale[..., None]), -127, 127).astype(np.int8)
    blocks = np.empty((n, v.shape[1], 34), dtype=np.uint8)
    blocks[..., 0:2] = _f16_bytes(scale)
    blocks[..., 2:34] = q.view(np.uint8)
    return blocks


def _pack_scales_k4(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """Inverse of the 6-bit (scale, min) unpacker: sc, mn uint8 [..., 8] in 0..63 -> uint8 [..., 12]."""
    out = np.zeros(sc.shape[:-1] + (12,), dtype=np.uint8)
    for j in range(4):
        out[..., j] = (sc[..., j] & 63) | ((sc[..., j + 4] >> 4) << 6)
        out[..., j + 4] = (mn[..., j] & 63) | ((mn[..., j + 4] >> 4) << 6)
        out[..., j + 8] = (sc[..., j + 4] & 0x0F) | ((mn[..., j + 4] & 0x0F) << 4)
    return out


def _kquant_scales(v: np.ndarray, qmax: int, smax: int):
    """Shared affine fit for the K-quants.

    v: float32 [N, B, G, L] (G groups of L weights).  Each group is modelled as
    w ~ d*sc*q - dmin*m with q in 0..qmax, sc and m in 0..smax, d and dmin fp16 per super-block.
    Returns (d16, dmin16, sc, m, q) with the integer fields as uint8.
    """
    lo = np.minimum(v.min(axis=-1), 0.0)
    hi = v.max(axis=-1)
    m_f = -lo                                               # >= 0
    s_f = np.maximum(hi + m_f, 0.0) / np.float32(qmax)      # >= 0
    d = (s_f.max(axis=-1) / np.float32(smax)).astype(np.float16)
    dmin = (m_f.max(axis=-1) / np.float32(smax)).astype(np.float16)
    d32 = d.astype(np.float32)[..., None]
    dmin32 = dmin.astype(np.float32)[..., None]
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d32 > 0, np.rint(s_f / d32), 0.0)
        mn = np.where(dmin32 > 0, np.rint(m_f / dmin32), 0.0)
    sc = np.clip(sc, 0, smax).astype(np.uint8)
    mn = np.clip(mn, 0, smax).astype(np.uint8)
    step = d32 * sc.astype(np.float32)
    off = dmin32 * mn.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(step[..., None] > 0, np.rint((v + off[..., None]) / step[..., None]), 0.0)
    q = np.clip(q, 0, qmax).astype(np.uint8)
    return d, dmin, sc, mn, q


def quantize_q4_k(weight: np.ndarray) -> np.ndarray:
    """float [N, K] -> uint8 [N, ceil(K/256), 144] (d, dmin, 12 scale bytes, 128 nibble bytes)."""
    w = _pad_rows(np.asarray(weight, dtype=np.float32), 256)
    n = w.shape[0]
    v = w.reshape(n, -1, 8, 32)
    d, dmin, sc, mn, q = _kquant_scales(v, 15, 63)
    blocks = np.empty((n, v.shape[1], 144), dtype=np.uint8)
    blocks[..., 0:2] = _f16_bytes(d)
    blocks[..., 2:4] = _f16_bytes(dmin)
    blocks[..., 4:16] = _pack_scales_k4(sc, mn)
    for pair in range(4):
        blocks[..., 16 + 32 * pair:48 + 32 * pair] = q[:, :, 2 * pair] | (q[:, :, 2 * pair + 1] << 4)
    return blocks


def quantize_q5_k(weight: np.ndarray) -> np.ndarray:
    """float [N, K] -> uint8 [N, ceil(K/256), 176] (d, dmin, scales[12], qh[32], qs[128])."""
    w = _pad_rows(np.asarray(weight, dtype=np.float32), 256)
    n = w.shape[0]
    v = w.reshape(n, -1, 8, 32)
    d, dmin, sc, mn, q = _kquant_scales(v, 31, 63)
    blocks = np.empty((n, v.shape[1], 176), dtype=np.uint8)
    blocks[..., 0:2] = _f16_bytes(d)
    blocks[..., 2:4] = _f16_bytes(dmin)
    blocks[..., 4:16] = _pack_scales_k4(sc, mn)
    qh = np.zeros((n, v.shape[1], 32), dtype=np.uint8)
    for pair in range(4):
        lo = q[:, :, 2 * pair]
        hi = q[:, :, 2 * pair + 1]
        blocks[..., 48 + 32 * pair:80 + 32 * pair] = (lo & 15) | ((hi & 15) << 4)
        qh |= ((lo >> 4) & 1) << (2 * pair)
        qh |= ((hi >> 4) & 1) << (2 * pair + 1)
    blocks[..., 16:48] = qh
    return blocks


def quantize_q2_k(weight: np.ndarray) -> np.ndarray:
    """float [N, K] -> uint8 [N, ceil(K/256), 84] (scales[16], qs[64], d, dmin)."""
    w = _pad_rows(np.asarray(weight, dtype=np.float32), 256)
    n = w.shape[0]
    v = w.reshape(n, -1, 16, 16)
    d, dmin, sc, mn, q = _kquant_scales(v, 3, 15)
    blocks = np.zeros((n, v.shape[1], 84), dtype=np.uint8)
    blocks[..., 0:16] = sc | (mn << 4)
    for group in range(16):
        half, gi = divmod(group, 8)
        shift = 2 * (gi // 2)
        start = 16 + 32 * half + 16 * (gi % 2)
        blocks[..., start:start + 16] |= q[:, :, group] << shift
    blocks[..., 80:82] = _f16_bytes(d)
    blocks[..., 82:84] = _f16_bytes(dmin)
    return blocks


def quantize_q6_k(weight: np.ndarray) -> np.ndarray:
    """float [N, K] -> uint8 [N, ceil(K/256), 210] (ql[128], qh[64], scales int8[16], d): w ~= d * scale[i // 16] * (q - 32)."""
    w = _pad_rows(np.asarray(weight, dtype=np.float32), 256)
    n = w.shape[0]
    v = w.reshape(n, -1, 16, 16)
    amax = np.abs(v).max(axis=-1)
    gscale = amax / np.float32(31.0)                                         # per 16 weights
    d = np.maximum(gscale.max(axis=-1), np.float32(1e-12)) / np.float32(127.0)
    d = d.astype(np.float16).astype(np.float32)
    sc = np.clip(np.rint(gscale / d[..., None]), 1, 127).astype(np.int8)
    q = np.clip(np.rint(v / (d[..., None, None] * sc.astype(np.float32)[..., None])) + 32, 0, 63).astype(np.uint8)
    q = q.reshape(n, -1, 2, 4, 32)                                           # [half][j][l]: weight 128 half + 32 j + l
    blocks = np.zeros((n, v.shape[1], 210), dtype=np.uint8)
    for half in range(2):
        blocks[..., 64 * half:64 * half + 32] = (q[:, :, half, 0] & 15) | ((q[:, :, half, 2] & 15) << 4)
        blocks[..., 64 * half + 32:64 * half + 64] = (q[:, :, half, 1] & 15) | ((q[:, :, half, 3] & 15) << 4)
        blocks[..., 128 + 32 * half:160 + 32 * half] = ((q[:, :, half, 0] >> 4) | ((q[:, :, half, 1] >> 4) << 2) |
                                                        ((q[:, :, half, 2] >> 4) << 4) | ((q[:, :, half, 3] >> 4) << 6))
    blocks[..., 192:208] = sc.view(np.uint8)
    blocks[..., 208:210] = _f16_bytes(d)
    return blocks


IQ4_KVALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)


def quantize_iq4_xs(weight: np.ndarray) -> np.ndarray:
    """float [N, K] -> uint8 [N, ceil(K/256), 136] (d, scales_h u16, scales_l[4], qs[128]): w ~= d * (ls - 32) * kvalues[code],
    16 bytes per 32 weights with weights 0..15 in the low and 16..31 in the high nibbles."""
    w = _pad_rows(np.asarray(weight, dtype=np.float32), 256)
    n = w.shape[0]
    v = w.reshape(n, -1, 8, 32)
    gscale = np.abs(v).max(axis=-1) / np.float32(127.0)                      # per 32 weights
    d = np.maximum(gscale.max(axis=-1), np.float32(1e-12)) / np.float32(31.0)
    d = d.astype(np.float16).astype(np.float32)
    ls = np.clip(np.rint(gscale / d[..., None]), 1, 31).astype(np.int16)      # scale - 32 in [1, 31]
    target = v / (d[..., None, None] * ls.astype(np.float32)[..., None])
    code = np.abs(target[..., None] - IQ4_KVALUES).argmin(axis=-1).astype(np.uint8)
    blocks = np.zeros((n, v.shape[1], 136), dtype=np.uint8)
    blocks[..., 0:2] = _f16_bytes(d)
    stored = (ls + 32).astype(np.uint16)
    sh = np.zeros(stored.shape[:-1], dtype=np.uint16)
    for g in range(8):
        sh |= ((stored[..., g] >> 4) & 3) << (2 * g)
        blocks[..., 4 + g // 2] |= ((stored[..., g] & 15) << (4 if g & 1 else 0)).astype(np.uint8)
        blocks[..., 8 + 16 * g:24 + 16 * g] = code[:, :, g, 0:16] | (code[:, :, g, 16:32] << 4)
    blocks[..., 2] = (sh & 0xFF).astype(np.uint8)
    blocks[..., 3] = (sh >> 8).astype(np.uint8)
    return blocks


def random_blocks(rng: np.random.Generator, type_name: str, *lead: int, d_range=(0.001, 0.02)) -> np.ndarray:
    """Every byte random except the fp16 scale field (finite, drawn from d_range): q6_k, iq4_xs, iq2_xs or iq3_xxs."""
    nbytes, off = {"q6_k": (210, 208), "iq4_xs": (136, 0), "iq2_xs": (74, 0), "iq3_xxs": (98, 0)}[type_name]
    blocks = rng.integers(0, 256, size=tuple(lead) + (nbytes,), dtype=np.uint8)
    d = rng.uniform(d_range[0], d_range[1], size=tuple(lead)).astype(np.float32)
    blocks[..., off:off + 2] = _f16_bytes(d)
    return blocks


def random_iq2_xxs(rng: np.random.Generator, *lead: int, d_range=(0.01, 0.04)) -> np.ndarray:
    """Random valid IQ2_XXS blocks, uint8 [*lead, 66]: uniform grid ids, sign bits and 4-bit scales,
    fp16 super-block scale drawn uniformly from d_range."""
    blocks = rng.integers(0, 256, size=tuple(lead) + (66,), dtype=np.uint8)
    d = rng.uniform(d_range[0], d_range[1], size=tuple(lead)).astype(np.float32)
    blocks[..., 0:2] = _f16_bytes(d)
    return blocks


def random_iq1_m(rng: np.random.Generator, *lead: int, d_range=(0.01, 0.04)) -> np.ndarray:
    """Random valid IQ1_M blocks, uint8 [*lead, 56]: uniform qs/qh bytes and 3-bit local scales; the
    fp16 super-block scale is scattered over the top nibbles of the four scale words (the layout
    cpp_engine/tests/test_moe_grouped_iq1.cpp:30-56 builds)."""
    lead = tuple(lead)
    blocks = rng.integers(0, 256, size=lead + (56,), dtype=np.uint8)
    d = rng.uniform(d_range[0], d_range[1], size=lead).astype(np.float16)
    bits = d.view(np.uint16)
    sc = np.ascontiguousarray(blocks[..., 48:56]).view("<u2").reshape(lead + (4,)).copy()
    sc &= np.uint16(0x0FFF)
    sc[..., 0] |= (bits & 0x000F) << 12
    sc[..., 1] |= (bits & 0x00F0) << 8
    sc[..., 2] |= (bits & 0x0F00) << 4
    sc[..., 3] |= bits & 0xF000
    blocks[..., 48:56] = sc.view(np.uint8).reshape(lead + (8,))
    return blocks


def quantize_fp8_block(weight: np.ndarray, block: int = 128):
    """float [N, K] -> (uint8 codes [N, K], float32 scales [ceil(N/128), ceil(K/128)]).

    scale = blockmax / 448 (1.0 for an all-zero block), code = RNE cast of w / scale to E4M3FN.
    """
    w = np.asarray(weight, dtype=np.float32)
    n, k = w.shape
    nb, kb = (n + block - 1) // block, (k + block - 1) // block
    pad = np.zeros((nb * block, kb * block), dtype=np.float32)
    pad[:n, :k] = w
    tiles = pad.reshape(nb, block, kb, block)
    amax = np.abs(tiles).max(axis=(1, 3))
    scale = np.where(amax > 0, amax / np.float32(448.0), np.float32(1.0)).astype(np.float32)
    scaled = (tiles / scale[:, None, :, None]).reshape(nb * block, kb * block)[:n, :k]
    codes = torch.from_numpy(np.ascontiguousarray(scaled)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    return codes, scale
