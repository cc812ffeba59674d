"""Block-granular ("loose") sliding-window causal attention with optional base-2 LSE output.
Counterpart of ops/triton_fused_local_attn2.py:249-275 (module name kept for drop-in imports)."""
import torch

from ._common import LOCAL_LOOSE, last_dim_contiguous, local_attention_bhnd


def flash_attn_func(q, k, v, window_size, softmax_scale=None, return_lse=False):
    """
    q: (batch_size, seqlen_q, nheads, headdim)
    k, v: (batch_size, seqlen_k, nheads, headdim)
    Query tile t (128 rows) sees the whole key blocks [t*128 - window_size, t*128) plus the causal diagonal block.
    Returns o, or (o, lse [batch, nheads, seqlen] fp32 base 2) with return_lse.
    """
    q, k, v = last_dim_contiguous(q, k, v)
    out, lse = local_attention_bhnd(q.transpose(1, 2), None, k.transpose(1, 2), None, v.transpose(1, 2), window_size,
                                    LOCAL_LOOSE, softmax_scale, return_lse, out_bnhd=True)
    out = out.transpose(1, 2)
    return (out, lse) if return_lse else out


def local_attn2_ref_impl(q, k, v, window_size, softmax_scale=None, return_lse=False):
    """Dense PyTorch statement of the same mask (ops/triton_fused_local_attn2.py:259-275), on q's device."""
    n_ctx = q.shape[1]
    q_position = torch.arange(n_ctx, device=q.device)
    k_position = (torch.arange((n_ctx + 127) // 128, device=q.device).repeat_interleave(128)[:n_ctx] + 1) * 128
    mask = ((q_position[:, None] - k_position[None, :]) < window_size).tril()
    return torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), scale=softmax_scale, attn_mask=mask[None, None, ...]
    ).transpose(1, 2)
