"""Llama attention modules on the HIP attention paths: counterparts of the reference's
`LlamaFlashAttention2VectorQuantizedReRoPE` (ops/attn_vq.py:176-276) and `LlamaFlashAttention2ReRoPE`
(ops/attn_rerope.py:116-253) and of their `use_rerope()` context managers (ops/attn_vq.py:482-486,
ops/attn_rerope.py:291-295), written against the `LlamaAttention` of the transformers release that is installed
(5.x: one attention class, `forward(hidden_states, position_embeddings, attention_mask, past_key_values, **kwargs)`
returning `(attn_output, attn_weights)`; there is no `LLAMA_ATTENTION_CLASSES` table any more).

Both modules project q / k / v with the layer's own weights, hand [B,H,N,D] states to the attention core
(`attn_vq.dispatch_attn` / `attn_rerope.rerope_attn_forward`, which rotate at the positions they need -- the
`position_embeddings` the model passes in are not used, as the reference's modules call their own rotary embedding),
and apply `o_proj`.  The reference's VQ module returns before `o_proj` (the call is commented out, ops/attn_vq.py:224),
which no decoder layer can consume; here both modules are drop-in `LlamaAttention`s.

The caches are the ones of `attn_vq` / `attn_rerope`; they answer the two questions the model's mask construction asks
of a cache (`get_query_offset`, `get_mask_sizes`), the mask itself is ignored (the kernels are causal by
construction).
"""
import logging
from contextlib import contextmanager

import torch
from transformers.models.llama import modeling_llama
from transformers.models.llama.modeling_llama import LlamaAttention as _LlamaAttention

from . import attn_rerope as _rerope
from . import attn_vq as _vq

logger = logging.getLogger(__name__)
_warned = set()


def _rope_base(config):
    params = getattr(config, "rope_parameters", None)
    if isinstance(params, dict) and "rope_theta" in params:
        return float(params["rope_theta"])
    return float(getattr(config, "rope_theta", 10000.0))


class _HipAttentionBase(_LlamaAttention):
    cache_type = None
    cache_name = ""

    def _type_guard(self, vectors):
        """fp32 states (upcast layer norms / embeddings) are cast back to the model dtype, with one warning
        (ops/attn_vq.py:250-276, ops/attn_rerope.py:213-233)."""
        single = isinstance(vectors, torch.Tensor)
        vectors = [vectors] if single else list(vectors)
        if vectors[0].dtype == torch.float32:
            if torch.is_autocast_enabled():
                target = torch.get_autocast_gpu_dtype()
            elif hasattr(self.config, "_pre_quantization_dtype"):
                target = self.config._pre_quantization_dtype
            else:
                target = self.q_proj.weight.dtype
            if target != torch.float32:
                if "cast" not in _warned:
                    _warned.add("cast")
                    logger.warning(
                        "The input hidden states seems to be silently casted in float32, this might be related to the "
                        "fact you have upcasted embedding or layer norm layers in float32. We will cast back the input "
                        f"in {target}.")
                vectors = [x.to(target) for x in vectors]
        return vectors[0] if single else vectors

    def _states(self, hidden_states, cache, output_attentions):
        bsz, q_len, _ = hidden_states.size()
        assert isinstance(cache, self.cache_type), f"{self.cache_name} is required"
        assert cache.get_seq_length(self.layer_idx) == 0 or q_len == 1, "Only support prefilling or generation"
        assert not output_attentions, "Not implemented"
        assert not self.training, "Not implemented"
        assert self.num_key_value_groups == 1, "grouped-query attention is not supported (one key head per query head)"
        shape = (bsz, q_len, -1, self.head_dim)
        q = self.q_proj(hidden_states).view(shape).transpose(1, 2)
        k = self.k_proj(hidden_states).view(shape).transpose(1, 2)
        v = self.v_proj(hidden_states).view(shape).transpose(1, 2)
        return self._type_guard([q, k, v])

    def _positions(self, position_ids, cache, bsz, q_len, device):
        if position_ids is None:
            past = cache.get_seq_length(self.layer_idx)
            position_ids = torch.arange(past, past + q_len, device=device).unsqueeze(0)
        if position_ids.shape[0] != bsz:
            position_ids = position_ids.expand(bsz, -1)
        return position_ids


class LlamaFlashAttention2VectorQuantizedReRoPE(_HipAttentionBase):
    """Attention with a VQ far-context memory (ops/attn_vq.py:176-248): long prefills through the linear-time VQ route,
    short ones exact, generation steps on the cache's count state."""
    cache_type = _vq.VectorQuantizedReRoPECache
    cache_name = "VQReRoPECache"

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None,
                position_ids=None, output_attentions=False, **kwargs):
        bsz, q_len, _ = hidden_states.size()
        cache = past_key_values
        q, k, v = self._states(hidden_states, cache, output_attentions)
        assert not cache.sphere, "Not implemented"
        position_ids = self._positions(position_ids, cache, bsz, q_len, hidden_states.device)
        out = _vq.dispatch_attn(q, k, v, position_ids, cache, self.layer_idx, _rope_base(self.config))
        return self.o_proj(out.to(self.o_proj.weight.dtype)), None


class LlamaFlashAttention2ReRoPE(_HipAttentionBase):
    """Full-context ReRoPE attention (ops/attn_rerope.py:116-253)."""
    cache_type = _rerope.ReRoPECache
    cache_name = "ReRoPECache"

    def forward(self, hidden_states, position_embeddings=None, attention_mask=None, past_key_values=None,
                position_ids=None, output_attentions=False, **kwargs):
        bsz, q_len, _ = hidden_states.size()
        cache = past_key_values
        q, k, v = self._states(hidden_states, cache, output_attentions)
        assert bsz == 1, "Not implemented"  # as the reference, ops/attn_rerope.py:139
        position_ids = self._positions(position_ids, cache, bsz, q_len, hidden_states.device)
        out = _rerope.rerope_attn_forward(q, k, v, position_ids, cache, self.layer_idx, _rope_base(self.config))
        return self.o_proj(out.to(self.o_proj.weight.dtype)), None


@contextmanager
def _swap_llama_attention(cls):
    """Models built inside the context get `cls` as their attention module (the role of the reference's swap of the
    `flash_attention_2` entry of `LLAMA_ATTENTION_CLASSES`); the original class is restored on exit, also when the
    body raises."""
    saved = modeling_llama.LlamaAttention
    modeling_llama.LlamaAttention = cls
    try:
        yield
    finally:
        modeling_llama.LlamaAttention = saved


def use_vq_rerope():
    return _swap_llama_attention(LlamaFlashAttention2VectorQuantizedReRoPE)


def use_rerope():
    return _swap_llama_attention(LlamaFlashAttention2ReRoPE)
