"""CPU-only checks of host-side logic that needs no kernel: the far-boundary rule of the generation window, and the
attention-class swap of `use_rerope()` (class substitution and restoration only; running the modules needs a GPU)."""
import pytest


def test_far_boundary_of_the_generation_window_follows_the_prefill_rule():
    """boundary(i) = max(0, floor((i - W) / 128) * 128), ops/attn_vq.py:283, 311 -- the same values as the oracle's
    prefill boundary, row by row."""
    import oracle
    from vqtree_amd.ops.count_state import far_boundary

    for W in (0, 128, 256, 1000):
        want = oracle.far_boundary(900, W, "block")
        assert [far_boundary(i, W) for i in range(900)] == [int(x) for x in want]
    assert far_boundary(5, 256) == 0 and far_boundary(256 + 127, 256) == 0 and far_boundary(256 + 128, 256) == 128


def test_use_rerope_swaps_and_restores_the_attention_class():
    from transformers.models.llama import modeling_llama as m

    from vqtree_amd.ops import attn_rerope as R
    from vqtree_amd.ops import attn_vq as A

    original = m.LlamaAttention
    with A.use_rerope():
        assert m.LlamaAttention is A.LlamaFlashAttention2VectorQuantizedReRoPE
        assert issubclass(m.LlamaAttention, original)
    assert m.LlamaAttention is original
    with pytest.raises(KeyError):
        with R.use_rerope():
            assert m.LlamaAttention is R.LlamaFlashAttention2ReRoPE
            raise KeyError("body failed")
    assert m.LlamaAttention is original
    with pytest.raises(AttributeError):
        A.no_such_name
