"""Rotary position embedding, transformers ~4.37 convention (test infrastructure only).

Follows the helpers the reference's callers use: `_rotate_half` / `_apply_key_rotary_pos_emb`
(/root/reference ops/attn_vq.py:54-64) and the `rotary_emb` / `apply_rotary_pos_emb` pair called at
ops/attn_vq.py:291-299 and ops/attn_rerope.py:160-180.
"""
import torch


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """cat(-x[D/2:], x[:D/2])  (ops/attn_vq.py:54-58)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def rope_tables(head_dim: int, n_pos: int, base: float = 10000.0, dtype=torch.float32):
    """cos/sin tables [n_pos, D]: inv_freq_r = base^(-2r/D), emb[p] = cat(p*inv_freq, p*inv_freq)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    pos = torch.arange(n_pos, dtype=torch.float32)
    freqs = torch.outer(pos, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions) -> torch.Tensor:
    """RoPE(x, p) = x*cos[p] + rotate_half(x)*sin[p], evaluated in x's dtype (ops/attn_vq.py:60-64).

    `x` is [..., N, D]; `positions` is an int (one clamped position for every row, the ReRoPE q2 case at
    ops/attn_vq.py:297-299) or a LongTensor [N].
    """
    if isinstance(positions, int):
        c, s = cos[positions], sin[positions]
    else:
        c, s = cos[positions], sin[positions]  # [N, D]
    c = c.to(x.dtype)
    s = s.to(x.dtype)
    return x * c + rotate_half(x) * s
