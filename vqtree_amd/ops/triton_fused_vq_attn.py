"""VQ far-context prefill host op: ReRoPE window attention + count-weighted codeword attention + LSE merge.
Counterpart of ops/triton_fused_vq_attn.py:190-251 (module name kept for drop-in imports)."""
import math

import torch

from .. import _lib
from ._common import (LOCAL_REROPE, bhn_strides, check_same_16bit, last_dim_contiguous, local_attention_bhnd, ptr)


def merge_state_in_place(v, s, v_other, s_other):
    """flashinfer-compatible merge: v [N, H, D] (16-bit), s [N, H] fp32 base-2 LSE; updates v and s in place."""
    lib = _lib.load()
    _lib.require_gpu(v, s, v_other, s_other)
    sfx = check_same_16bit(v, v_other)
    assert s.dtype == s_other.dtype == torch.float32
    n, h, d = v.shape
    assert v.stride(-1) == 1 and v_other.stride(-1) == 1
    strides = _lib.strides_array(0, v.stride(1), v.stride(0), 0, s.stride(1), s.stride(0),
                                 0, v_other.stride(1), v_other.stride(0), 0, s_other.stride(1), s_other.stride(0))
    with torch.cuda.device(v.device):
        rc = getattr(lib, "vqa_merge_state_inplace_" + sfx)(ptr(v), ptr(s), ptr(v_other), ptr(s_other), 1, h, n, d,
                                                            strides, _lib.current_stream(v.device))
    _lib.check(rc)
    return v, s


def _count_call(q2, k_vq, k_vq_cnt, v_vq, vi, window_size, softmax_scale, out, lse, merge):
    lib = _lib.load()
    _lib.require_gpu(q2, k_vq, k_vq_cnt, v_vq, vi)
    B, H, N, D = q2.shape
    C = k_vq.shape[1]
    integer_counts = k_vq_cnt.dtype == torch.int64  # exact counts, as the preprocessing builds them
    sfx = check_same_16bit(q2, k_vq, None if integer_counts else k_vq_cnt, v_vq)
    assert vi.dtype == torch.int64 and k_vq.shape == (H, C, D) and v_vq.shape[:2] == (B, H)
    assert k_vq_cnt.shape[-1] == C and vi.shape == k_vq_cnt.shape
    n_far = max(0, -(-(N - window_size - 128) // 128))
    assert k_vq_cnt.shape[2] >= n_far, "k_vq_cnt / vi need one row per far-context query tile"
    strides = _lib.strides_array(*bhn_strides(q2), k_vq.stride(0), k_vq.stride(1), *bhn_strides(k_vq_cnt),
                                 *bhn_strides(v_vq), *bhn_strides(vi), *bhn_strides(out))
    with torch.cuda.device(q2.device):
        name = ("vqa_vqcount_merge_" if merge else "vqa_vqcount_fwd_") + ("icnt_" if integer_counts else "")
        rc = getattr(lib, name + sfx)(
            ptr(q2), ptr(k_vq), ptr(k_vq_cnt), ptr(v_vq), ptr(vi), ptr(out), ptr(lse), B, H, N, D, C, strides,
            int(window_size), softmax_scale, _lib.current_stream(q2.device))
    _lib.check(rc)


def vq_count_forward(q2, k_vq, k_vq_cnt, v_vq, vi, window_size, softmax_scale=None):
    """Far-context kernel alone: (o2 [B,H,N,D], lse2 [B,H,N] fp32 base 2); rows i < window+128 are 0 / -inf."""
    q2, k_vq, k_vq_cnt, v_vq, vi = last_dim_contiguous(q2, k_vq, k_vq_cnt, v_vq, vi)
    B, H, N, D = q2.shape
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)
    if D == 16:  # see vq_attn_forward
        pad = lambda x: torch.nn.functional.pad(x, (0, 16))
        o2, l2 = vq_count_forward(pad(q2), pad(k_vq), k_vq_cnt, pad(v_vq), vi, window_size, softmax_scale)
        return o2[..., :16], l2
    o2 = torch.empty((B, H, N, D), dtype=q2.dtype, device=q2.device)
    l2 = torch.empty((B, H, N), dtype=torch.float32, device=q2.device)
    _count_call(q2, k_vq, k_vq_cnt, v_vq, vi, window_size, softmax_scale, o2, l2, merge=False)
    return o2, l2


def vq_attn_forward(q1, q2, k1, k_vq, k_vq_cnt, k3, v, v_vq, vi, window_size, softmax_scale=None, return_lse=False):
    """q1/k1: rotary at true positions; q2: query at the clamped position; k_vq [H,C,D] codebook; k_vq_cnt / vi
    [B,H,N//128,C] running counts (model dtype as in the reference, or int64 for exact counts -- bf16 rounds counts
    above 256) / prefix-sum row indices sampled per 128-key block; k3 raw keys; v_vq [B,H,N+1,D]
    per-code prefix sums of V.  All attention tensors [B,H,N,D].  Returns [B,H,N,D] (with `return_lse`, an extension,
    also the merged base-2 log-sum-exp [B,H,N]).

    Unlike the reference (batch == 1 only, four layout copies around a separate merge launch) the two kernels work on
    the [B,H,N,D] tensors in place, the merge is the count kernel's epilogue, and any batch size is accepted.
    """
    q1, q2, k1, k_vq, k_vq_cnt, k3, v, v_vq, vi = last_dim_contiguous(q1, q2, k1, k_vq, k_vq_cnt, k3, v, v_vq, vi)
    B, H, N, D = q1.shape
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)
    if D == 16:  # the kernels start at head dim 32: zero-padded operands, padded output columns dropped
        pad = lambda x: torch.nn.functional.pad(x, (0, 16))
        res = vq_attn_forward(pad(q1), pad(q2), pad(k1), pad(k_vq), k_vq_cnt, pad(k3), pad(v), pad(v_vq), vi,
                              window_size, softmax_scale, return_lse)
        return (res[0][..., :16], res[1]) if return_lse else res[..., :16]
    o1, l1 = local_attention_bhnd(q1, q2, k1, k3, v, window_size, LOCAL_REROPE, softmax_scale, True)
    # far context, merged into (o1, l1) by the count kernel's epilogue
    _count_call(q2, k_vq, k_vq_cnt, v_vq, vi, window_size, softmax_scale, o1, l1, merge=True)
    return (o1, l1) if return_lse else o1
