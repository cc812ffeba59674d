"""Quantiser-side oracles: key reconstruction, runtime encoder, count-kernel inputs and the count kernel
itself (test infrastructure only)."""
import math

import torch

from .attention import LOG2E, T_BLOCK, _f32, local_attn, merge_state


def reconstruct_keys(codes, codebooks):
    """K_hat[b,h,j,:] = sum_m codebooks[h, m, codes[b,h,j,m], :]   (fp32).

    codes [B,H,N,M] integer, codebooks [H,M,K,D].  Integer gathers, so the selected rows are bit-exact; with M = 1
    this is the gather at /root/reference ops/mini_vq.py:13-14.
    """
    cb = _f32(codebooks)
    idx = codes.detach().to("cpu", torch.int64)
    B, H, N, M = idx.shape
    D = cb.shape[-1]
    out = torch.zeros(B, H, N, D, dtype=torch.float32)
    for h in range(H):
        for m in range(M):
            out[:, h] += cb[h, m][idx[:, h, :, m]]
    return out


def multi_head_single_quantize(inp, codebook):
    """Runtime key encoder (ops/mini_vq.py:4-18): id = argmax_c <k, cb[h,c]> (inner product, first max on ties).

    inp [B,H,N,D], codebook [H,C,D] -> (quantised [B,H,N,D] in inp dtype, ids [B,H,N] int64, onehot [B,H,N,C] int64).
    The product is evaluated in the input dtype like the reference's einsum.
    """
    x = inp.detach().cpu()
    cb = codebook.detach().cpu()
    prod = torch.einsum("bhnd,hcd->bhnc", x, cb)
    ids = prod.argmax(-1)
    H = cb.shape[0]
    quant = torch.stack([cb[h][ids[:, h]] for h in range(H)], dim=1)
    onehot = torch.nn.functional.one_hot(ids, cb.shape[1])
    return quant, ids, onehot


def encode_residual(x, codebooks):
    """Greedy additive (residual) encoder: r = x; for every codebook m: id_m = argmin_c |r - cb[h,m,c]|^2 (first
    minimum on ties), evaluated as argmax_c (<r, c> - |c|^2 / 2) in fp32; r -= cb[h,m,id_m].

    The reference has no runtime encoder for additive codes (its codebooks come from the offline faiss trainer,
    build_quantizer/120_build_additive_quantizer.py:23-32); this is the textbook greedy residual search, pinned by
    brute-force nearest-neighbour search in tests/test_oracle_pins.py.
    x [B,H,N,D], codebooks [H,M,K,D] -> codes [B,H,N,M] int64.
    """
    r = _f32(x).clone()
    cb = _f32(codebooks)
    B, H, N, D = r.shape
    out = torch.zeros(B, H, N, cb.shape[1], dtype=torch.int64)
    for m in range(cb.shape[1]):
        for h in range(H):
            score = r[:, h] @ cb[h, m].T - 0.5 * (cb[h, m] * cb[h, m]).sum(-1)
            idx = score.argmax(-1)
            out[:, h, :, m] = idx
            r[:, h] -= cb[h, m][idx]
    return out


def sort_based_preprocess(ids, v, n_codes, dtype=None, block=T_BLOCK):
    """Inputs of the count kernel, following ops/attn_vq.py:352-384 and the block sampling at :410-413.

    ids [B,H,N] int64 code per key, v [B,H,N,D].
    Returns
      cnt  [B,H,N//block,C] int64 : # keys j' <= (t+1)*block-1 with id == c  (inclusive running count, sampled
                                     at the last key of each block)
      v_vq [B,H,N+1,D]            : keys sorted by (code, position); row 1+r holds the prefix sum of V over the
                                     sorted keys of r's code up to r (global fp32 cumsum minus the cumsum at the
                                     code's segment start, then cast to `dtype`); row 0 is zero
      vi   [B,H,N//block,C] int64 : cnt + start[c], so v_vq[vi[t,c]] = sum_{j' < (t+1)*block, id=c} v_j' when cnt > 0
    """
    ids = ids.detach().cpu().to(torch.int64)
    vf = _f32(v)
    dtype = dtype or v.dtype
    B, H, N = ids.shape
    D = vf.shape[-1]
    assert n_codes < (1 << 13) and N < (1 << 18)  # ops/attn_vq.py:355-356
    onehot = torch.nn.functional.one_hot(ids, n_codes)
    cum = torch.cumsum(onehot, dim=2)  # [B,H,N,C] inclusive
    order = torch.argsort((ids << 18) + torch.arange(N)[None, None, :], dim=-1)
    v_sorted = torch.gather(vf, 2, order[..., None].expand(-1, -1, -1, D))
    S = torch.zeros(B, H, N + 1, D, dtype=torch.float32)
    S[:, :, 1:] = v_sorted
    S = torch.cumsum(S, dim=2)
    total = cum[:, :, -1]  # [B,H,C]
    start = torch.cumsum(total, dim=-1) - total  # exclusive
    seg_base = torch.gather(S, 2, start[..., None].expand(-1, -1, -1, D))  # S at each segment start [B,H,C,D]
    code_sorted = torch.gather(ids, 2, order)
    S[:, :, 1:] -= torch.gather(seg_base, 2, code_sorted[..., None].expand(-1, -1, -1, D))
    vi = cum + start[:, :, None, :]
    return (
        cum[:, :, block - 1 :: block].contiguous(),
        S.to(dtype),
        vi[:, :, block - 1 :: block].contiguous(),
    )


def vq_count_forward(q2, k_vq, k_vq_cnt, v_vq, vi, window_size, softmax_scale=None, block=T_BLOCK):
    """Count-weighted softmax over codewords (ops/triton_fused_vq_attn.py:38-68, 110-187).

    Query tile t covers rows [W+T+tT, W+T+(t+1)T) and uses row t of cnt / vi.  Per row:
      w_c = [cnt_c != 0] * exp(q2 . cb_c * scale);  out = sum_c w_c * v_vq[vi_c] / sum_c w_c * cnt_c
      lse2 = log2(sum_c cnt_c * exp(.))
    Rows i < W+T keep out = 0, lse2 = -inf (ops/triton_fused_vq_attn.py:214-215).
    q2 [B,H,N,D], k_vq [H,C,D], k_vq_cnt/vi [B,H,N//T,C], v_vq [B,H,N+1,D] -> (out [B,H,N,D] fp32, lse2 [B,H,N]).
    """
    qf, cb, cnt, S = _f32(q2), _f32(k_vq), _f32(k_vq_cnt), _f32(v_vq)
    idx = vi.detach().cpu().to(torch.int64)
    B, H, N, D = qf.shape
    scale = softmax_scale or 1.0 / math.sqrt(D)
    out = torch.zeros(B, H, N, D)
    lse2 = torch.full((B, H, N), float("-inf"))
    first = window_size + block
    n_tiles = max(0, -(-(N - first) // block))
    for t in range(n_tiles):
        lo, hi = first + t * block, min(first + (t + 1) * block, N)
        s = torch.einsum("bhid,hcd->bhic", qf[:, :, lo:hi], cb) * scale
        c_t = cnt[:, :, t]  # [B,H,C]
        live = (c_t != 0)[:, :, None, :]
        s = s.masked_fill(~live, float("-inf"))
        m = s.amax(-1, keepdim=True)
        p = torch.exp(s - m)
        vsum = torch.gather(S, 2, idx[:, :, t][..., None].expand(-1, -1, -1, D))  # [B,H,C,D]
        vsum = torch.where(live.transpose(-1, -2), vsum, torch.zeros_like(vsum))
        l = (p * c_t[:, :, None, :]).sum(-1, keepdim=True)
        out[:, :, lo:hi] = (p @ vsum) / l
        lse2[:, :, lo:hi] = ((m + torch.log(l)) * LOG2E).squeeze(-1)
    return out, lse2


def vq_attn_forward(q1, q2, k1, k_vq, k_vq_cnt, k3, v, v_vq, vi, window_size, softmax_scale=None):
    """The reference host op (ops/triton_fused_vq_attn.py:190-251): ReRoPE window attention over exact keys
    merged with the count kernel's far-context state by base-2 LSE.  Returns out [B,H,N,D] fp32."""
    o1, l1 = local_attn(q1, k1, v, window_size, "rerope", softmax_scale, q2=q2, k2=k3)
    o2, l2 = vq_count_forward(q2, k_vq, k_vq_cnt, v_vq, vi, window_size, softmax_scale)
    out, _ = merge_state(o1, l1, o2, l2)
    return out
