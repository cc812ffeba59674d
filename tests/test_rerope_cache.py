"""Host logic of the ReRoPE key/value cache (CPU): appended keys outside the window advance by one rotary position per
generation step.  Checked against the composition law RoPE(RoPE(k, a), 1) == RoPE(k, a + 1) in float64."""
import torch

from vqtree_amd.ops.attn_rerope import ReRoPECache
from vqtree_amd.ops.attn_vq import rope_tables, rotate_half


def _rope(x, cos, sin, p):
    return x * cos[p] + rotate_half(x) * sin[p]


def test_far_keys_advance_one_position_per_step():
    B, H, D, W, n0, steps = 1, 2, 16, 4, 9, 3
    g = torch.Generator().manual_seed(0)
    raw = torch.randn(B, H, n0 + steps, D, generator=g, dtype=torch.float64)
    vals = torch.randn(B, H, n0 + steps, D, generator=g, dtype=torch.float64)
    cos, sin = rope_tables(D, 64, dtype=torch.float64)
    pos = torch.arange(n0 + steps)
    rotated = raw * cos[pos] + rotate_half(raw) * sin[pos]  # every key at its true position
    cache = ReRoPECache(W)
    keys, values = cache.update(rotated[:, :, :n0].clone(), vals[:, :, :n0], 0, {"cos": cos, "sin": sin})
    assert cache.get_seq_length() == n0 and cache.seen_tokens == n0
    assert torch.equal(keys, rotated[:, :, :n0])  # the first update stores the keys untouched
    # position each cached key is expected to sit at; a key outside the last W entries advances once per update
    expect_pos = list(range(n0))
    for t in range(steps):
        n = n0 + t
        keys, values = cache.update(rotated[:, :, n:n + 1].clone(), vals[:, :, n:n + 1], 0, {"cos": cos, "sin": sin})
        expect_pos.append(n)
        for j in range(n + 1 - W):
            expect_pos[j] += 1
        want = torch.stack([_rope(raw[:, :, j], cos, sin, expect_pos[j]) for j in range(n + 1)], dim=2)
        assert keys.shape[2] == n + 1 and cache.get_seq_length() == n + 1
        torch.testing.assert_close(keys, want, rtol=0, atol=1e-5)  # tables are built in fp32
        assert torch.equal(values, vals[:, :, :n + 1])
    assert cache.seen_tokens == n0 + steps


def test_reorder_and_layers():
    cache = ReRoPECache(8)
    cos, sin = rope_tables(4, 8)
    k = torch.arange(2 * 1 * 3 * 4, dtype=torch.float32).reshape(2, 1, 3, 4)
    cache.update(k, k + 100, 0, {"cos": cos, "sin": sin})
    cache.update(k + 1, k + 101, 1, {"cos": cos, "sin": sin})
    assert cache.get_seq_length(1) == 3 and cache.get_seq_length(2) == 0 and cache.seen_tokens == 3
    cache.reorder_cache(torch.tensor([1, 0]))
    assert torch.equal(cache.key_cache[0], k[[1, 0]]) and torch.equal(cache.value_cache[1], (k + 101)[[1, 0]])
