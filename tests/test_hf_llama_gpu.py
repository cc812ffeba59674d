"""GPU tests of the Llama attention modules (`hf_llama`): a tiny random-init LlamaConfig, no download.  The module
output must equal the oracle attention fed through the same projections (q/k/v projections of the module, oracle
attention in fp32, the module's o_proj)."""
import logging
import math

import pytest
import torch

import oracle
from tests.util import assert_close_16
from vqtree_amd.ops import attn_rerope as R
from vqtree_amd.ops import attn_vq as A

pytestmark = pytest.mark.gpu

HIDDEN, HEADS, D = 256, 2, 128


def _config(layers=2):
    from transformers import LlamaConfig

    return LlamaConfig(hidden_size=HIDDEN, num_attention_heads=HEADS, num_key_value_heads=HEADS, head_dim=D,
                       num_hidden_layers=layers, intermediate_size=512, vocab_size=1000, max_position_embeddings=4096)


def _module(cls, seed):
    torch.manual_seed(seed)
    mod = cls(_config(), layer_idx=0)
    for lin in (mod.q_proj, mod.k_proj, mod.v_proj, mod.o_proj):  # O(1) activations, so the tolerance means something
        torch.nn.init.normal_(lin.weight, std=1.0 / math.sqrt(lin.in_features))
    return mod.to(torch.bfloat16).cuda().eval()


def _project(mod, hidden):
    B, N, _ = hidden.shape
    shape = (B, N, HEADS, D)
    return tuple(lin(hidden).view(shape).transpose(1, 2) for lin in (mod.q_proj, mod.k_proj, mod.v_proj))


def _through_o_proj(mod, attn):  # attn [B,H,N,D] fp32 from the oracle
    B, H, N, _ = attn.shape
    x = attn.transpose(1, 2).reshape(B, N, H * D).to(torch.bfloat16).cuda()
    return mod.o_proj(x)


def test_vq_module_prefill_and_generation_equal_oracle_through_the_same_projections():
    print("hf: VQ ReRoPE attention module, N=700 W=256 C=256", flush=True)
    from vqtree_amd.ops.hf_llama import LlamaFlashAttention2VectorQuantizedReRoPE

    B, N, W, C = 2, 700, 256, 256
    mod = _module(LlamaFlashAttention2VectorQuantizedReRoPE, 1)
    g = torch.Generator("cpu").manual_seed(2)
    hidden = torch.randn(B, N, HIDDEN, generator=g).bfloat16().cuda()
    cb = (torch.randn(HEADS, C, D, generator=g)).bfloat16().cuda()
    cache = A.VectorQuantizedReRoPECache(W, cb)
    pos = torch.arange(N, device="cuda").unsqueeze(0).expand(B, -1)
    with torch.no_grad():
        out, weights = mod(hidden, position_embeddings=None, attention_mask=None, past_key_values=cache, position_ids=pos)
        assert weights is None and out.shape == (B, N, HIDDEN) and cache.get_seq_length(0) == N
        q, k, v = _project(mod, hidden)
        q1, k1, q2 = A.rerope_operands(q, k, pos, W)
        attn, _ = oracle.attn_vq_prefill(q1.cpu(), cache.key_codes[0].cpu(), cb.unsqueeze(1).cpu(), v.cpu(),
                                         k_exact=k1.cpu(), window_size=W, q2=q2.cpu(), k2=k.cpu())
        # o_proj (weights ~ N(0, 1/256)) sums 256 products of attention outputs that are each within 2e-2 + 1e-2 |x|:
        # the sum of their errors stays within a few times 2e-2
        want = _through_o_proj(mod, attn)
        err = (out.float() - want.float()).abs().max().item()
        print(f"hf: prefill max abs err {err:.4g}", flush=True)
        assert err <= 6e-2, err

        # generation step through the module: all keys through their codewords, clamped query, then o_proj
        h1 = torch.randn(B, 1, HIDDEN, generator=g).bfloat16().cuda()
        step, _ = mod(h1, past_key_values=cache)  # positions default to the cache length
        assert cache.get_seq_length(0) == N + 1
        qs, ks, vs = _project(mod, h1)
        ids = torch.cat([cache.key_codes[0].long(), A.quantize_ids(ks, cb).unsqueeze(-1)], dim=2)
        cos, sin = A.rope_tables(D, W + 2, dtype=torch.bfloat16, device="cuda")
        q2s = qs * cos[W + 1] + A.rotate_half(qs) * sin[W + 1]
        attn1, _ = oracle.attn_vq_decode(q2s.cpu(), ids.cpu(), cb.unsqueeze(1).cpu(), torch.cat([v, vs], 2).cpu(),
                                         1 / math.sqrt(D))
        want1 = _through_o_proj(mod, attn1)
        assert (step.float() - want1.float()).abs().max().item() <= 6e-2


def test_rerope_module_equals_oracle_through_the_same_projections():
    print("hf: full ReRoPE attention module, N=300 W=128", flush=True)
    from vqtree_amd.ops.hf_llama import LlamaFlashAttention2ReRoPE

    B, N, W = 1, 300, 128
    mod = _module(LlamaFlashAttention2ReRoPE, 3)
    hidden = torch.randn(B, N, HIDDEN, generator=torch.Generator("cpu").manual_seed(4)).bfloat16().cuda()
    cache = R.ReRoPECache(W)
    pos = torch.arange(N, device="cuda").unsqueeze(0)
    with torch.no_grad():
        out, _ = mod(hidden, past_key_values=cache, position_ids=pos)
        q, k, v = _project(mod, hidden)
        cos, sin = A.rope_tables(D, N + 1, dtype=torch.bfloat16, device="cuda")
        rope = lambda x, p: x * cos[p] + A.rotate_half(x) * sin[p]
        attn, _ = oracle.rerope_full(rope(q, pos[0]).cpu(), rope(q, W).cpu(), rope(k, pos[0]).cpu(), k.cpu(), v.cpu(),
                                     True, 1 / math.sqrt(D), W)
        want = _through_o_proj(mod, attn)
    assert out.shape == (B, N, HIDDEN) and cache.get_seq_length(0) == N
    assert (out.float() - want.float()).abs().max().item() <= 6e-2
    with pytest.raises(AssertionError):  # batch > 1 is refused, as in the reference
        mod(torch.cat([hidden, hidden]), past_key_values=R.ReRoPECache(W))


def test_use_rerope_swaps_the_attention_class_and_a_tiny_model_runs():
    print("hf: use_rerope() + 2-layer LlamaModel", flush=True)
    from transformers.models.llama import modeling_llama as m

    original = m.LlamaAttention
    with A.use_rerope():
        assert m.LlamaAttention.__name__ == "LlamaFlashAttention2VectorQuantizedReRoPE"
        torch.manual_seed(5)
        model = m.LlamaModel(_config()).to(torch.bfloat16).cuda().eval()
    assert m.LlamaAttention is original
    with pytest.raises(RuntimeError):  # restored on an exception too
        with R.use_rerope():
            assert m.LlamaAttention.__name__ == "LlamaFlashAttention2ReRoPE"
            raise RuntimeError("x")
    assert m.LlamaAttention is original
    assert all(type(l.self_attn).__name__ == "LlamaFlashAttention2VectorQuantizedReRoPE" for l in model.layers)

    B, N, W, C = 1, 600, 256, 128
    g = torch.Generator("cpu").manual_seed(6)
    cache = A.VectorQuantizedReRoPECache(W, torch.randn(HEADS, C, D, generator=g).bfloat16().cuda())
    ids = torch.randint(0, 1000, (B, N), generator=g).cuda()
    with torch.no_grad():
        h = model(ids, past_key_values=cache, use_cache=True).last_hidden_state
        assert h.shape == (B, N, HIDDEN) and torch.isfinite(h.float()).all()
        assert cache.get_seq_length(0) == N and cache.get_seq_length(1) == N and cache.seen_tokens == N
        h1 = model(ids[:, :1], past_key_values=cache, use_cache=True).last_hidden_state  # one generation step
        assert h1.shape == (B, 1, HIDDEN) and torch.isfinite(h1.float()).all()
        assert cache.get_seq_length(0) == N + 1 and cache.get_seq_length(1) == N + 1 and cache.seen_tokens == N + 1


def test_type_guard_casts_fp32_states_to_the_model_dtype_with_a_warning(caplog):
    from vqtree_amd.ops import hf_llama

    mod = _module(hf_llama.LlamaFlashAttention2VectorQuantizedReRoPE, 7)
    hf_llama._warned.clear()
    x = torch.randn(1, HEADS, 4, D, device="cuda")
    with caplog.at_level(logging.WARNING, logger=hf_llama.logger.name):
        a, b = mod._type_guard([x, x])
        c = mod._type_guard(x)
    assert a.dtype == b.dtype == c.dtype == torch.bfloat16
    assert sum("cast back the input" in r.message for r in caplog.records) == 1  # warned once
    y = x.to(torch.float16)
    assert mod._type_guard(y) is y  # 16-bit states pass through
    cache = A.VectorQuantizedReRoPECache(256, torch.zeros(HEADS, 128, D, dtype=torch.bfloat16, device="cuda"), sphere=True)
    with pytest.raises(AssertionError):
        mod(torch.zeros(1, 8, HIDDEN, dtype=torch.bfloat16, device="cuda"), past_key_values=cache)
