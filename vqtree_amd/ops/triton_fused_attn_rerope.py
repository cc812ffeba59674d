"""Full-context ReRoPE attention.  Counterpart of ops/triton_fused_attn_rerope.py:185-233 (module name kept for
drop-in imports; the kernel is hand-written HIP)."""
from ._common import last_dim_contiguous, local_attention_bhnd


def attention(q1, q2, k1, k2, v, causal, sm_scale, window):
    """q1, k1: local pair; q2, k2: distant pair; all [Z, H, N_CTX, D_HEAD].

    score(i, j) = q1_i.k1_j if |i - j| < window else q2_i.k2_j; causal mask j <= i when `causal`.  Returns o like q1.
    """
    assert q1.shape[-1] == k1.shape[-1] == v.shape[-1]
    q1, q2, k1, k2, v = last_dim_contiguous(q1, q2, k1, k2, v)
    out, _ = local_attention_bhnd(q1, q2, k1, k2, v, window, None, sm_scale, False, full_causal=bool(causal))
    return out
