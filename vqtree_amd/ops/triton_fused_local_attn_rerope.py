"""Block-local sliding-window attention with the ReRoPE boundary rule and optional base-2 LSE output.
Counterpart of ops/triton_fused_local_attn_rerope.py:287-294 (module name kept for drop-in imports)."""
from ._common import LOCAL_REROPE, last_dim_contiguous, local_attention_bhnd


def flash_attn_func(q1, q2, k1, k2, v, window_size, softmax_scale=None, return_lse=False):
    """
    q: (batch_size, seqlen_q, nheads, headdim)
    k, v: (batch_size, seqlen_k, nheads, headdim)
    Keys [floor(i/128)*128 - window_size, i] are visible; score = q1.k1 when i - j <= window_size, else q2.k2.
    Returns o, or (o, lse [batch, nheads, seqlen] fp32 base 2) with return_lse.
    """
    q1, q2, k1, k2, v = last_dim_contiguous(q1, q2, k1, k2, v)
    out, lse = local_attention_bhnd(q1.transpose(1, 2), q2.transpose(1, 2), k1.transpose(1, 2), k2.transpose(1, 2),
                                    v.transpose(1, 2), window_size, LOCAL_REROPE, softmax_scale, return_lse, out_bnhd=True)
    out = out.transpose(1, 2)
    return (out, lse) if return_lse else out
