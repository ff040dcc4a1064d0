"""The attention core of the decoder block (pocketllm_amd/attention_core.py) against a plain numpy statement of half-split rotary
embedding and causal grouped-query attention (what src/models/minimax_m2/architecture.py:197-266 computes).  CPU only."""
import numpy as np
import torch

from pocketllm_amd.attention_core import KeyValueCache, RotaryTable, grouped_query_attention


def _rope_np(x, first, rope_dim, base):
    half = rope_dim // 2
    f = np.arange(first, first + x.shape[1])[:, None] * (base ** (-(2.0 * np.arange(half)) / rope_dim))[None, :]
    s, c = np.sin(f)[None, :, None, :], np.cos(f)[None, :, None, :]
    x1, x2 = x[..., :half], x[..., half:rope_dim]
    return np.concatenate([x1 * c - x2 * s, x1 * s + x2 * c, x[..., rope_dim:]], axis=-1)


def test_rotary_table_matches_the_pairwise_rotation_and_grows():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 5, 4, 16))
    table = RotaryTable(8, 10000.0, torch.device("cpu"), head_dim=16, positions=4)
    for first in (0, 3, 700):                # 700 lies beyond the first table: it has to grow
        got = table.rotate(torch.from_numpy(x).float(), first).numpy()
        assert np.abs(got - _rope_np(x, first, 8, 10000.0)).max() < 2e-5
    whole = RotaryTable(16, 5.0e6, torch.device("cpu"))                        # rope_dim == head_dim, no tail
    assert np.abs(whole.rotate(torch.from_numpy(x).float(), 11).numpy() - _rope_np(x, 11, 16, 5.0e6)).max() < 2e-5
    none = RotaryTable(0, 10000.0, torch.device("cpu"), head_dim=16)
    assert none.rotate(torch.from_numpy(x), 5) is not None and torch.equal(none.rotate(torch.from_numpy(x), 5), torch.from_numpy(x))


def test_grouped_query_attention_is_causal_softmax_attention_over_the_store():
    rng = np.random.default_rng(1)
    batch, heads, kv_heads, dim = 2, 4, 2, 16
    cache = KeyValueCache(kv_heads, dim, torch.device("cpu"), torch.float32)
    ks, vs = [], []
    first = 0
    for steps in (3, 5, 1):                  # a prefill, a second chunk at a non-zero position, one decode step (the store grows on the way)
        k, v = rng.standard_normal((batch, steps, kv_heads, dim)), rng.standard_normal((batch, steps, kv_heads, dim))
        q = rng.standard_normal((batch, steps, heads, dim))
        ks.append(k)
        vs.append(v)
        cache.write(torch.from_numpy(k).float(), torch.from_numpy(v).float(), first)
        keys, values = cache.read(batch, first + steps)
        got = grouped_query_attention(torch.from_numpy(q).float(), keys, values, first).numpy()
        all_k, all_v = np.concatenate(ks, axis=1), np.concatenate(vs, axis=1)
        want = np.zeros((batch, steps, heads, dim))
        for b in range(batch):
            for t in range(steps):
                for h in range(heads):
                    kk, vv = all_k[b, :first + t + 1, h // (heads // kv_heads)], all_v[b, :first + t + 1, h // (heads // kv_heads)]
                    s = kk @ q[b, t, h] / np.sqrt(dim)
                    p = np.exp(s - s.max())
                    want[b, t, h] = (p / p.sum()) @ vv
        assert np.abs(got - want.reshape(batch, steps, heads * dim)).max() < 1e-5
        first += steps
    assert cache.keys.size(2) >= first
