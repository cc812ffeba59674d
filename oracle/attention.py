"""Naive fp32 attention oracles for every kernel on the VQ-attention path (test infrastructure only).

All functions upcast their inputs to fp32, build the full score matrix per (batch, head), apply the
integer visibility / score-source predicates, and run one softmax.  Layout is [B, H, N, D] unless a
function says otherwise.  Log-sum-exp values are base-2 of the scaled scores (`m + log2(l)` with
scores multiplied by `softmax_scale * log2(e)`), the convention of every reference kernel
(/root/reference ops/triton_fused_vq_attn.py:179, ops/triton_fused_local_attn_rerope.py:214-216).
"""
import math

import torch

LOG2E = 1.4426950408889634  # RCP_LN2, ops/triton_fused_vq_attn.py:17
T_BLOCK = 128  # BLOCK_SIZE "MUST MATCH KERNEL", ops/attn_vq.py:23


def _f32(x):
    return None if x is None else x.detach().to("cpu", torch.float32)


def attend(scores: torch.Tensor, visible: torch.Tensor, v: torch.Tensor):
    """softmax over visible keys, then @ V.

    scores  [..., Nq, Nk] fp32, already multiplied by softmax_scale (natural-log domain)
    visible [..., Nq, Nk] bool (broadcastable)
    v       [..., Nk, D] fp32
    returns (out [..., Nq, D] fp32, lse2 [..., Nq] fp32 base-2).  A row with no visible key gives
    out = 0 and lse2 = -inf (the host-side initialisation at ops/triton_fused_vq_attn.py:214-215).
    """
    s = scores.masked_fill(~visible, float("-inf"))
    m = s.amax(dim=-1, keepdim=True)
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    p = torch.exp(s - m)
    l = p.sum(dim=-1, keepdim=True)
    out = (p @ v) / torch.where(l == 0, torch.ones_like(l), l)
    lse2 = (m + torch.log(l)).squeeze(-1) * LOG2E
    return out, lse2


# ----------------------------------------------------------------------------------------------
# additive-quantiser key scores
# ----------------------------------------------------------------------------------------------
def vq_scores_reconstruct(q, codes, codebooks):
    """q . K_hat^T with K_hat[b,h,j] = sum_m codebooks[h, m, codes[b,h,j,m]]  (dense restatement).

    q [B,H,Nq,D], codes [B,H,Nk,M] uint8/int, codebooks [H,M,K,D] -> [B,H,Nq,Nk] fp32 (unscaled).
    With M = 1 this is the quantised key of ops/mini_vq.py:13-14.
    """
    from .vq import reconstruct_keys

    k_hat = reconstruct_keys(codes, codebooks)
    return _f32(q) @ k_hat.transpose(-1, -2)


def vq_scores_lut(q, codes, codebooks):
    """Same scores by the lookup-table route: LUT[b,h,i,m,c] = <q_i, cb[h,m,c]>, score = sum_m LUT[.., m, code_jm].

    This is how the kernels evaluate it; equality with `vq_scores_reconstruct` pins the gather indexing.
    """
    qf, cb = _f32(q), _f32(codebooks)
    B, H, Nq, D = qf.shape
    Nk, M = codes.shape[2], codes.shape[3]
    lut = torch.einsum("bhid,hmcd->bhimc", qf, cb)  # [B,H,Nq,M,K]
    idx = codes.detach().to("cpu", torch.int64)  # [B,H,Nk,M]
    out = torch.zeros(B, H, Nq, Nk, dtype=torch.float32)
    for m in range(M):
        out += torch.gather(lut[:, :, :, m, :], 3, idx[:, :, None, :, m].expand(B, H, Nq, Nk))
    return out


# ----------------------------------------------------------------------------------------------
# masks
# ----------------------------------------------------------------------------------------------
def far_boundary(n: int, window: int, mode: str) -> torch.Tensor:
    """First key position that is still exact for each query i (keys j < boundary(i) are quantised).

    'block': max(0, floor((i - W)/T) * T)   -- ops/attn_vq.py:311; equals the union rule of the window kernel
             stages (ops/triton_fused_local_attn_rerope.py:38-53) when W is a multiple of T.
    'exact': max(0, i - W)                  -- ops/attn_vq.py:312 (local_boundary)
    """
    i = torch.arange(n)
    if mode == "block":
        return torch.clamp(torch.div(i - window, T_BLOCK, rounding_mode="floor") * T_BLOCK, min=0)
    if mode == "exact":
        return torch.clamp(i - window, min=0)
    raise ValueError(mode)


def local_visible_mask(n: int, window: int, mode: str):
    """(visible, primary) [N,N] bool for the three sliding-window kernels; rows = queries, cols = keys.

    strict : j <= i and i - j <= W                         ops/triton_fused_local_attn.py:65-72
    loose  : j <= i and j >= floor(i/T)*T - W              ops/triton_fused_local_attn2.py:37-46
    rerope : visible as loose; primary (q1.k1) iff i-j<=W  ops/triton_fused_local_attn_rerope.py:68-78
    `primary` is all-true for strict/loose.
    """
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    causal = j <= i
    if mode == "strict":
        return causal & (i - j <= window), torch.ones(n, n, dtype=torch.bool)
    tile_lo = torch.div(i, T_BLOCK, rounding_mode="floor") * T_BLOCK - window
    vis = causal & (j >= tile_lo)
    if mode == "loose":
        return vis, torch.ones(n, n, dtype=torch.bool)
    if mode == "rerope":
        return vis, (i - j <= window)
    raise ValueError(mode)


# ----------------------------------------------------------------------------------------------
# kernels' oracles
# ----------------------------------------------------------------------------------------------
def local_attn(q1, k1, v, window, mode, softmax_scale=None, q2=None, k2=None):
    """Sliding-window exact attention, [B,H,N,D] in, (out [B,H,N,D] fp32, lse2 [B,H,N]) out.

    mode 'strict' = ops/triton_fused_local_attn.py, 'loose' = ops/triton_fused_local_attn2.py,
    'rerope' = ops/triton_fused_local_attn_rerope.py (keys outside the window but inside the stage-1
    tile are scored with the second pair q2.k2 instead of being masked, :73-75).
    """
    q1f, k1f, vf = _f32(q1), _f32(k1), _f32(v)
    n, d = q1f.shape[-2], q1f.shape[-1]
    scale = softmax_scale or 1.0 / math.sqrt(d)
    vis, prim = local_visible_mask(n, window, mode)
    s = q1f @ k1f.transpose(-1, -2)
    if mode == "rerope":
        s2 = _f32(q2) @ _f32(k2).transpose(-1, -2)
        s = torch.where(prim, s, s2)
    return attend(s * scale, vis, vf)


def rerope_full(q1, q2, k1, k2, v, causal, sm_scale, window):
    """Full-context ReRoPE attention (ops/triton_fused_attn_rerope.py:114-167; torch oracle :238-251).

    score(i,j) = q1_i.k1_j if |i-j| < W (strict) else q2_i.k2_j; causal mask j <= i when `causal`.
    """
    q1f, q2f, k1f, k2f, vf = map(_f32, (q1, q2, k1, k2, v))
    n = q1f.shape[-2]
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    s1 = q1f @ k1f.transpose(-1, -2)
    s2 = q2f @ k2f.transpose(-1, -2)
    s = torch.where((i - j).abs() < window, s1, s2)
    vis = (j <= i) if causal else torch.ones(n, n, dtype=torch.bool)
    return attend(s * sm_scale, vis, vf)


def attn_vq_prefill(
    q,
    k_codes,
    codebooks,
    v,
    k_exact=None,
    window_size=0,
    causal=True,
    softmax_scale=None,
    boundary_mode="block",
    q2=None,
    k2=None,
):
    """Prefill attention over additive-quantiser key codes, optionally with an exact sliding window.

    Generalises the naive reference (ops/attn_vq.py:308-333) from one codebook to M:
      keys j <  boundary(i)            : quantised, score = q_far_i . K_hat_j        (:324-330)
      keys boundary(i) <= j < i - W    : exact strip, score = q2_i . k2_j if given    (:317-323)
      keys i - W <= j <= i             : exact window, score = q_i . k_exact_j        (:313-316)
    q_far = q2 when given (the position-clamped query of ReRoPE, :296-299) else q.  Without `k_exact`
    every visible key is quantised.  `causal=False` (all keys visible, all quantised) needs k_exact None.
    Returns (out [B,H,N,D] fp32, lse2 [B,H,N]).
    """
    qf, vf = _f32(q), _f32(v)
    nq, d = qf.shape[-2], qf.shape[-1]
    nk = vf.shape[-2]
    scale = softmax_scale or 1.0 / math.sqrt(d)
    q_far = _f32(q2) if q2 is not None else qf
    s_far = vq_scores_reconstruct(q_far, k_codes, codebooks)
    i = torch.arange(nq)[:, None]
    j = torch.arange(nk)[None, :]
    if not causal:
        assert k_exact is None
        return attend(s_far * scale, torch.ones(nq, nk, dtype=torch.bool), vf)
    assert nq == nk
    vis = j <= i
    if k_exact is None:
        return attend(s_far * scale, vis, vf)
    bnd = far_boundary(nq, window_size, boundary_mode)[:, None]
    s_win = qf @ _f32(k_exact).transpose(-1, -2)
    if q2 is not None and k2 is not None:
        s_strip = _f32(q2) @ _f32(k2).transpose(-1, -2)
    else:
        s_strip = s_win
    s = torch.where(j < bnd, s_far, torch.where(i - j <= window_size, s_win, s_strip))
    return attend(s * scale, vis, vf)


def attn_vq_decode(q, k_codes, codebooks, v, softmax_scale=None):
    """seqlen_q = 1 attention over all N quantised keys, no mask.

    out[b,h] = softmax_j(sum_m <q, cb[h,m,code[b,h,j,m]]> * scale) . V[b,h,j].  The reference only promises this
    kernel (README.md:8; ops/attn_vq.py:445-479 is a non-functional fallback), so the oracle is the dense definition.
    q [B,H,1,D] -> (out [B,H,1,D] fp32, lse2 [B,H,1]).
    """
    return attn_vq_prefill(q, k_codes, codebooks, v, causal=False, softmax_scale=softmax_scale)


def merge_state(o, s, o_other, s_other):
    """Base-2 log-sum-exp merge of two partial attention states (flashinfer.merge_state_in_place as called at
    ops/triton_fused_vq_attn.py:246-250; third-party, restated from its published definition).

    o, o_other [..., D]; s, s_other [...] base-2 LSE.  Returns (o_merged fp32, s_merged fp32).
    A side with s = -inf contributes nothing.
    """
    of, sf, of2, sf2 = map(_f32, (o, s, o_other, s_other))
    m = torch.maximum(sf, sf2)
    m_safe = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    w1 = torch.exp2(sf - m_safe)
    w2 = torch.exp2(sf2 - m_safe)
    den = w1 + w2
    den_safe = torch.where(den == 0, torch.ones_like(den), den)
    out = (of * w1[..., None] + of2 * w2[..., None]) / den_safe[..., None]
    return out, m + torch.log2(den)


def slow_reference(q1, k1, q2, k_raw, k_hat, v, window, softmax_scale=None, block=T_BLOCK):
    """Per-query Python loops, the literal structure of ops/attn_vq.py:305-333 (tiny inputs only).

    q1,k1: rotary at true positions; q2: rotary clamped at W+1; k_raw: un-rotated exact keys; k_hat: quantised
    keys (any number of codebooks, already reconstructed).  All [B,H,N,D].  Returns out [B,H,N,D] fp32.
    """
    q1, k1, q2, k_raw, k_hat, v = map(_f32, (q1, k1, q2, k_raw, k_hat, v))
    B, H, N, D = q1.shape
    scale = softmax_scale or 1.0 / math.sqrt(D)
    out = torch.zeros(B, H, N, D)
    for b in range(B):
        for h in range(H):
            for qi in range(N):
                boundary = max(0, (qi - window) // block * block)
                local_boundary = max(0, qi - window)
                att = [k1[b, h, local_boundary : qi + 1] @ q1[b, h, qi]]
                vv = [v[b, h, local_boundary : qi + 1]]
                if local_boundary > 0:
                    att.append(k_raw[b, h, boundary:local_boundary] @ q2[b, h, qi])
                    vv.append(v[b, h, boundary:local_boundary])
                if boundary > 0:
                    att.append(k_hat[b, h, :boundary] @ q2[b, h, qi])
                    vv.append(v[b, h, :boundary])
                a = torch.softmax(torch.cat(att) * scale, dim=0)
                out[b, h, qi] = a @ torch.cat(vv)
    return out
