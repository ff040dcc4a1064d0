"""The attention core between the quantized projections of a decoder block: rotary position phases, the key/value store and
grouped-query softmax attention.  None of it is on the quantized matmul path; it is plain framework arithmetic kept here so
that a block can be run and timed end to end (what the reference does at src/models/minimax_m2/architecture.py:158-266 with
its own cache layout and PyTorch's fused attention).  Written for one GPU and for HIP-graph capture: no host round trips, no
data-dependent shapes, all state preallocated.

Conventions: activations are [batch, steps, heads, head_dim]; positions are absolute token indices.
"""
from __future__ import annotations

import torch


class RotaryTable:
    """Half-split rotary embedding over the first `rope_dim` values of every head: value j (j < rope_dim / 2) and value
    j + rope_dim / 2 form a pair that is turned by the angle position * base ** (-2 j / rope_dim).  Kept per position as two
    float32 rows of head_dim values, so that a turn is two multiplications and an addition on whole heads:
        out = x * cos_row + swap(x) * sin_row
    with swap exchanging the two halves of the rotary part; cos_row is 1 and sin_row 0 on the values behind rope_dim, sin_row
    carries the minus sign of the first half.  The tables grow by doubling."""

    def __init__(self, rope_dim: int, base: float, device: torch.device, head_dim: int | None = None, positions: int = 256):
        self.rope_dim = int(rope_dim)
        self.half = self.rope_dim // 2
        self.head_dim = int(head_dim) if head_dim is not None else self.rope_dim
        self.base = float(base)
        self.device = device
        self._cos: torch.Tensor | None = None
        self._sin: torch.Tensor | None = None
        tail = torch.arange(2 * self.half, self.head_dim, device=device)
        self._swap = torch.cat((torch.arange(self.half, 2 * self.half, device=device), torch.arange(0, self.half, device=device), tail))
        if self.half > 0:
            self.reserve(positions)

    def reserve(self, positions: int) -> None:
        have = 0 if self._cos is None else self._cos.size(0)
        if positions <= have or self.half == 0:
            return
        count = max(int(positions), 2 * have)
        exponent = torch.arange(0, 2 * self.half, 2, device=self.device, dtype=torch.float64) / float(self.rope_dim)
        rate = torch.exp(-exponent * torch.log(torch.tensor(self.base, dtype=torch.float64, device=self.device)))
        angle = torch.outer(torch.arange(count, device=self.device, dtype=torch.float64), rate)
        rest = self.head_dim - 2 * self.half
        self._cos = torch.cat((angle.cos(), angle.cos(), torch.ones(count, rest, device=self.device, dtype=torch.float64)), dim=1).float()
        self._sin = torch.cat((-angle.sin(), angle.sin(), torch.zeros(count, rest, device=self.device, dtype=torch.float64)), dim=1).float()

    def rows(self, pos: int) -> tuple[torch.Tensor, torch.Tensor]:
        """The cos and sin rows (float32, head_dim values each) of one position; all ones / zeros without a rotary part."""
        if self.half == 0:
            if self._cos is None:
                self._cos = torch.ones(1, self.head_dim, device=self.device)
                self._sin = torch.zeros(1, self.head_dim, device=self.device)
            return self._cos[0], self._sin[0]
        self.reserve(pos + 1)
        return self._cos[pos], self._sin[pos]

    def rotate(self, x: torch.Tensor, first_pos: int) -> torch.Tensor:
        """x [batch, steps, heads, head_dim] at positions first_pos .. first_pos + steps - 1; returns a new tensor of x's dtype
        (float32 arithmetic, one rounding)."""
        if self.half == 0:
            return x
        steps = x.size(1)
        self.reserve(first_pos + steps)
        cos = self._cos[first_pos:first_pos + steps].view(1, steps, 1, self.head_dim)
        sin = self._sin[first_pos:first_pos + steps].view(1, steps, 1, self.head_dim)
        return torch.addcmul(x * cos, x.index_select(-1, self._swap), sin).to(x.dtype)


class KeyValueCache:
    """Keys and values of one layer, head-major: [batch, kv_heads, capacity, head_dim].  A query head then reads its keys as one
    contiguous [length, head_dim] matrix and nothing is transposed or repeated per step."""

    def __init__(self, kv_heads: int, head_dim: int, device: torch.device, dtype: torch.dtype):
        self.kv_heads, self.head_dim, self.device, self.dtype = int(kv_heads), int(head_dim), device, dtype
        self.keys: torch.Tensor | None = None
        self.values: torch.Tensor | None = None

    def allocate(self, batch: int, capacity: int) -> None:
        shape = (int(batch), self.kv_heads, int(capacity), self.head_dim)
        self.keys = torch.zeros(shape, device=self.device, dtype=self.dtype)
        self.values = torch.zeros(shape, device=self.device, dtype=self.dtype)

    def ensure(self, batch: int, length: int) -> None:
        """Room for `length` positions of `batch` sequences; what is stored survives a growth."""
        if self.keys is not None and self.keys.size(0) >= batch and self.keys.size(2) >= length:
            return
        old_k, old_v = self.keys, self.values
        self.allocate(max(batch, 0 if old_k is None else old_k.size(0)), max(256, length, 0 if old_k is None else 2 * old_k.size(2)))
        if old_k is not None:
            self.keys[: old_k.size(0), :, : old_k.size(2)] = old_k
            self.values[: old_v.size(0), :, : old_v.size(2)] = old_v

    def write(self, k: torch.Tensor, v: torch.Tensor, first_pos: int) -> None:
        """k, v [batch, steps, kv_heads, head_dim] go to positions first_pos .. first_pos + steps - 1."""
        batch, steps = k.size(0), k.size(1)
        self.ensure(batch, first_pos + steps)
        self.keys[:batch, :, first_pos:first_pos + steps] = k.permute(0, 2, 1, 3)
        self.values[:batch, :, first_pos:first_pos + steps] = v.permute(0, 2, 1, 3)

    def read(self, batch: int, length: int) -> tuple[torch.Tensor, torch.Tensor]:
        return self.keys[:batch, :, :length], self.values[:batch, :, :length]


def grouped_query_attention(q: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, first_pos: int) -> torch.Tensor:
    """softmax(q k^T / sqrt(head_dim)) v with every key/value head shared by heads / kv_heads query heads.

    q [batch, steps, heads, head_dim] at positions first_pos ..; keys, values [batch, kv_heads, length, head_dim] hold positions
    0 .. length - 1 (length = first_pos + steps).  A query sees the keys at positions up to its own.  The query heads of one
    group are folded into the row dimension of one matrix product per key/value head.  The products run in the cache's dtype
    (float32 accumulation inside the matrix multiply), the softmax in float32.  Returns [batch, steps, heads * head_dim] in q's dtype."""
    batch, steps, heads, dim = q.shape
    kv_heads, length = keys.size(1), keys.size(2)
    group = heads // kv_heads
    if steps > 1 and first_pos == 0 and length == steps and q.is_cuda and q.dtype == keys.dtype and q.dtype in (torch.float16, torch.bfloat16):
        # a whole prompt at once: the framework's fused causal attention (the routine the reference calls), key/value heads shared
        out = torch.nn.functional.scaled_dot_product_attention(q.permute(0, 2, 1, 3), keys, values, is_causal=True, enable_gqa=group > 1)
        return out.permute(0, 2, 1, 3).reshape(batch, steps, heads * dim)
    # [batch, kv_heads, group * steps, head_dim]: row g * steps + s is query head (kv * group + g) at step s
    rows = (q * (float(dim) ** -0.5)).view(batch, steps, kv_heads, group, dim).permute(0, 2, 3, 1, 4).reshape(batch, kv_heads, group * steps, dim)
    scores = torch.matmul(rows.to(keys.dtype), keys.transpose(2, 3))
    if steps > 1:                            # a single new token sees everything stored; several need the triangle
        q_pos = first_pos + torch.arange(steps, device=q.device).repeat(group)
        hidden = torch.arange(length, device=q.device).view(1, length) > q_pos.view(-1, 1)
        scores = scores.masked_fill(hidden.view(1, 1, group * steps, length), float("-inf"))
    weights = torch.softmax(scores, dim=-1, dtype=torch.float32).to(values.dtype)
    context = torch.matmul(weights, values)                                    # [batch, kv_heads, group * steps, head_dim]
    context = context.view(batch, kv_heads, group, steps, dim).permute(0, 3, 1, 2, 4)
    return context.reshape(batch, steps, heads * dim).to(q.dtype)
