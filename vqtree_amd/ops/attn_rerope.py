"""Caller of the full-context ReRoPE kernel: the key/value cache with decode-time re-rotation and the attention
routing of the reference's ReRoPE module (ops/attn_rerope.py:19-288) on [B,H,N,D] states.  The transformers module
around it (projections, o_proj, `use_rerope`) is `hf_llama.LlamaFlashAttention2ReRoPE`, reachable from here by name.
"""
import math

import torch

from .attn_vq import apply_rope, attn_exact_decode, rope_tables, rotate_half
from .triton_fused_attn_rerope import attention
from .triton_fused_local_attn import flash_attn_func as causal_window_attention


class ReRoPECache:
    """Growing per-layer key/value cache of ops/attn_rerope.py:19-115.  Keys are stored already rotated; whenever the
    cache is longer than `window_length` after an append, every key outside the last `window_length` positions is
    rotated forward by one position (cos[1], sin[1]), so far keys keep a fixed distance to the newest query."""

    def __init__(self, window_length):
        self.key_cache = []
        self.value_cache = []
        self.window_length = window_length
        self.cos_1 = {}
        self.sin_1 = {}
        self.seen_tokens = 0

    def get_seq_length(self, layer_idx=0):
        return 0 if len(self.key_cache) <= layer_idx else self.key_cache[layer_idx].shape[-2]

    def get_usable_length(self, new_seq_length, layer_idx=0):
        return self.get_seq_length(layer_idx)

    # what a transformers (5.x) model asks of a cache while it builds its (unused) causal mask
    def get_query_offset(self, layer_idx=0):
        return self.get_seq_length(layer_idx)

    def get_mask_sizes(self, query_length, layer_idx=0):
        return self.get_seq_length(layer_idx) + query_length, 0

    def get_max_length(self):
        return int(1e8)

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        """Append [B,H,n,D] states; `cache_kwargs` carries the model's cos / sin tables [n_pos, D]."""
        cos = (cache_kwargs or {}).get("cos")
        sin = (cache_kwargs or {}).get("sin")
        assert cos is not None and sin is not None, "This is useless for models without RoPE."
        assert (cache_kwargs or {}).get("partial_rotation_size") is None, "partial rotation is not supported"
        if layer_idx == 0:
            self.seen_tokens += key_states.shape[-2]
        if len(self.key_cache) <= layer_idx:
            self.key_cache.append(key_states)
            self.value_cache.append(value_states)
        else:
            self.key_cache[layer_idx] = torch.cat([self.key_cache[layer_idx], key_states], dim=-2)
            self.value_cache[layer_idx] = torch.cat([self.value_cache[layer_idx], value_states], dim=-2)
            if self.get_seq_length(layer_idx) > self.window_length:
                far = self.key_cache[layer_idx][:, :, : -self.window_length]
                dev = far.device
                if dev not in self.cos_1:
                    self.cos_1[dev], self.sin_1[dev] = cos[1].to(dev), sin[1].to(dev)
                far.copy_(far * self.cos_1[dev] + rotate_half(far) * self.sin_1[dev])
        return self.key_cache[layer_idx], self.value_cache[layer_idx]

    def reorder_cache(self, beam_idx):
        for layer_idx in range(len(self.key_cache)):
            self.key_cache[layer_idx] = self.key_cache[layer_idx].index_select(
                0, beam_idx.to(self.key_cache[layer_idx].device))
            self.value_cache[layer_idx] = self.value_cache[layer_idx].index_select(
                0, beam_idx.to(self.value_cache[layer_idx].device))


def _rope_at(x, cos, sin, positions):
    """x [B,H,N,D]; positions: LongTensor [B,N] or a single int."""
    return apply_rope(x, cos, sin, positions)


def rerope_attn_forward(query_states, key_states, value_states, position_ids, cache, layer_idx=0, rope_base=10000.0):
    """Attention core of `LlamaFlashAttention2ReRoPE.forward` (ops/attn_rerope.py:119-253).  Un-rotated states
    [B,H,q_len,D], position_ids [B,q_len]; returns [B, q_len, H*D] (before o_proj).

    * prefill longer than the window: q1/k1 rotated at the true positions, q2 at position `window_length`, k2 = keys
      at position 0 (unrotated); the cache receives far keys rotated to `q_len - window_length` and the last
      `window_length` keys at their true positions; the full ReRoPE kernel computes the output;
    * short prefill: plain causal attention on the rotated operands (window kernel with the window covering
      everything);
    * generation (q_len == 1): the new key is appended (far keys re-rotated by the cache) and the query attends over
      all cached keys with the exact-key streaming decode kernel (a third-party flash attention call in the
      reference, ops/attn_rerope.py:279-286).
    """
    assert isinstance(cache, ReRoPECache), "ReRoPECache is required"
    B, H, q_len, D = query_states.shape
    W = cache.window_length
    past = cache.get_seq_length(layer_idx)
    assert past == 0 or q_len == 1, "Only support prefilling or generation"
    scale = 1.0 / math.sqrt(D)
    # sized on the host (no device-to-host copy of the largest position): a model's positions are past .. past + q_len - 1
    n_pos = max(past + q_len, W + 1, 2)
    cos, sin = rope_tables(D, n_pos, rope_base, query_states.dtype, query_states.device)
    kwargs = {"cos": cos, "sin": sin}
    if past == 0 and q_len > W:
        q1 = _rope_at(query_states, cos, sin, position_ids)
        k1 = _rope_at(key_states, cos, sin, position_ids)
        q2 = _rope_at(query_states, cos, sin, W)
        k2 = _rope_at(key_states, cos, sin, 0)
        k3 = _rope_at(key_states, cos, sin, q_len - W)
        merged = torch.cat([k3[:, :, :-W], k1[:, :, -W:]], dim=2)
        cache.update(merged, value_states, layer_idx, kwargs)
        out = attention(q1, q2, k1, k2, value_states, True, scale, W)
        return out.transpose(1, 2).reshape(B, q_len, H * D).contiguous()
    q = _rope_at(query_states, cos, sin, position_ids)
    k = _rope_at(key_states, cos, sin, position_ids)
    keys, values = cache.update(k, value_states, layer_idx, kwargs)
    if past == 0:
        out = causal_window_attention(q.transpose(1, 2), keys.transpose(1, 2), values.transpose(1, 2), q_len,
                                      softmax_scale=scale)
        return out.reshape(B, q_len, H * D).contiguous()
    out = attn_exact_decode(q, keys, values, softmax_scale=scale)
    return out.transpose(1, 2).reshape(B, q_len, H * D).contiguous()


def __getattr__(name):
    # `LlamaFlashAttention2ReRoPE` and `use_rerope` (ops/attn_rerope.py:116, 291) live in hf_llama and are imported on
    # first use, so that the operators do not pay for importing transformers.
    if name in ("LlamaFlashAttention2ReRoPE", "use_rerope"):
        from . import hf_llama

        return getattr(hf_llama, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
