"""Strict sliding-window causal attention (module name kept from the reference for drop-in imports; the kernel is
hand-written HIP, not Triton).  Counterpart of ops/triton_fused_local_attn.py:254-262."""
from ._common import LOCAL_STRICT, last_dim_contiguous, local_attention_bhnd


def flash_attn_func(q, k, v, window_size, softmax_scale=None):
    """
    q: (batch_size, seqlen_q, nheads, headdim)
    k, v: (batch_size, seqlen_k, nheads, headdim)
    Key j is visible to query i iff j <= i and i - j <= window_size.  Returns o (batch, seqlen, nheads, headdim).
    """
    q, k, v = last_dim_contiguous(q, k, v)
    out, _ = local_attention_bhnd(q.transpose(1, 2), None, k.transpose(1, 2), None, v.transpose(1, 2), window_size,
                                  LOCAL_STRICT, softmax_scale, False, out_bnhd=True)
    return out.transpose(1, 2)
