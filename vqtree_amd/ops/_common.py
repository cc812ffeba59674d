"""Shared host-side plumbing of the operator modules: argument checks and C-ABI calls."""
import math

import torch

from .. import _lib

SUFFIX = {torch.bfloat16: "bf16", torch.float16: "f16"}

LOCAL_STRICT, LOCAL_LOOSE, LOCAL_REROPE = 0, 1, 2
BOUNDARY = {"block": 0, "exact": 1}


def last_dim_contiguous(*tensors):
    """Make the last dimension contiguous, other strides are honoured (ops/triton_fused_vq_attn.py:193-195)."""
    return [x if x is None or x.stride(-1) == 1 else x.contiguous() for x in tensors]


def bhn_strides(x):
    """(b, h, n) element strides of a [B,H,N,D] tensor (or of a [B,N,H,D] tensor already transposed to that view)."""
    return (x.stride(0), x.stride(1), x.stride(2))


def check_same_16bit(*tensors):
    dt = tensors[0].dtype
    assert all(t.dtype == dt for t in tensors if t is not None), "All tensors must have the same type"
    assert dt in SUFFIX, "Only support fp16 and bf16"
    return SUFFIX[dt]


def ptr(x):
    return None if x is None else x.data_ptr()


def local_attention_bhnd(q1, q2, k1, k2, v, window_size, mode, softmax_scale, return_lse, out_bnhd=False,
                         full_causal=None):
    """Runs vqa_local_attn_* / vqa_rerope_full_* on [B,H,N,D] views.  Returns (out [B,H,N,D] view, lse or None).

    `out_bnhd`: allocate the output as a contiguous [B,N,H,D] buffer (returned as its [B,H,N,D] view), the layout
    the reference's flash_attn_func wrappers return (`empty_like(q, contiguous_format)`).
    `full_causal`: None for the sliding-window modes; True/False selects the full-context ReRoPE kernel.
    """
    lib = _lib.load()
    _lib.require_gpu(q1, q2, k1, k2, v)
    B, H, N, D = q1.shape
    assert k1.shape == (B, H, N, D) and v.shape == (B, H, N, D), "seqlen_q == seqlen_k prefill only"
    assert D in (16, 32, 64, 128), "head dimensions 16, 32, 64 and 128 are supported"
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)
    if D == 16:
        # The kernels start at head dim 32 (one 32-row block of the output tile): zero-padded operands give the same
        # scores, and the padded output columns are dropped.
        pad = lambda x: None if x is None else torch.nn.functional.pad(x, (0, 16))
        out, lse = local_attention_bhnd(pad(q1), pad(q2), pad(k1), pad(k2), pad(v), window_size, mode, softmax_scale,
                                        return_lse, out_bnhd, full_causal)
        return out[..., :16], lse
    sfx = check_same_16bit(q1, q2, k1, k2, v)
    if out_bnhd:
        out = torch.empty((B, N, H, D), dtype=q1.dtype, device=q1.device).transpose(1, 2)
    else:
        out = torch.empty((B, H, N, D), dtype=q1.dtype, device=q1.device)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q1.device) if return_lse else None
    q2_, k2_ = (q2 if q2 is not None else q1), (k2 if k2 is not None else k1)
    strides = _lib.strides_array(*bhn_strides(q1), *bhn_strides(q2_), *bhn_strides(k1), *bhn_strides(k2_),
                                 *bhn_strides(v), *bhn_strides(out))
    with torch.cuda.device(q1.device):
        stream = _lib.current_stream(q1.device)
        if full_causal is None:
            fn = getattr(lib, "vqa_local_attn_" + sfx)
            rc = fn(ptr(q1), ptr(q2), ptr(k1), ptr(k2), ptr(v), ptr(out), ptr(lse), B, H, N, D, strides,
                    int(window_size), mode, softmax_scale, stream)
        else:
            fn = getattr(lib, "vqa_rerope_full_" + sfx)
            rc = fn(ptr(q1), ptr(q2), ptr(k1), ptr(k2), ptr(v), ptr(out), ptr(lse), B, H, N, D, strides,
                    int(window_size), 1 if full_causal else 0, softmax_scale, stream)
    _lib.check(rc)
    return out, lse
