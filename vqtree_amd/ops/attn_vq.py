"""Additive-code VQ attention entry points (counterpart of the reference's ops/attn_vq.py dispatch).

`attn_vq_decode` is the seqlen_q == 1 route the reference dispatches to `naive_attn`
(ops/attn_vq.py:247-248, 445-479) and its README promises as "a separate kernel" (ops/README.md:3).
Layouts follow the reference's attention modules: q, v [B,H,N,D]; codebooks [H,M,K,D]; codes [B,H,N,M] uint8.
"""
import math

import torch

from .. import _lib

_SUFFIX = {torch.bfloat16: "bf16", torch.float16: "f16"}


def _last_dim_contiguous(x):
    return x if x.stride(-1) == 1 else x.contiguous()


def attn_vq_decode(q, k_codes, codebooks, v, *, softmax_scale=None, return_lse=False, num_splits=0):
    """out[b,h] = softmax_j(scale * sum_m <q[b,h], codebooks[h,m,k_codes[b,h,j,m]]>) @ v[b,h]   (no mask).

    q [B,H,1,D] bf16/f16, k_codes [B,H,N,M] uint8, codebooks [H,M,K,D], v [B,H,N,D]  ->  out [B,H,1,D] (q's dtype)
    and, with return_lse, the base-2 log-sum-exp [B,H,1] fp32.
    """
    lib = _lib.load()
    _lib.require_gpu(q, k_codes, codebooks, v)
    assert q.dim() == 4 and q.shape[2] == 1, "decode takes q of shape [B,H,1,D]"
    B, H, _, D = q.shape
    N, M = k_codes.shape[2], k_codes.shape[3]
    K = codebooks.shape[2]
    assert k_codes.shape[:2] == (B, H) and k_codes.dtype == torch.uint8
    assert codebooks.shape == (H, M, K, D), "codebooks must be [H,M,K,D]"
    assert v.shape == (B, H, N, D)
    assert q.dtype == codebooks.dtype == v.dtype, "All tensors must have the same type"
    assert q.dtype in _SUFFIX, "Only support fp16 and bf16"
    q, codebooks, v = map(_last_dim_contiguous, (q, codebooks, v))
    if k_codes.stride(3) != 1 or k_codes.stride(2) != M:
        k_codes = k_codes.contiguous()
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)

    out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, 1), dtype=torch.float32, device=q.device) if return_lse else None
    splits = num_splits if num_splits > 0 else lib.vqa_decode_default_splits(B, H, N)
    ws_bytes = lib.vqa_decode_workspace_bytes(B, H, N, D, M, K, splits)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    strides = _lib.strides_array(
        q.stride(0), q.stride(1),
        k_codes.stride(0), k_codes.stride(1),
        codebooks.stride(0), codebooks.stride(1), codebooks.stride(2),
        v.stride(0), v.stride(1), v.stride(2),
        out.stride(0), out.stride(1),
    )  # fmt: skip
    with torch.cuda.device(q.device):
        fn = getattr(lib, "vqa_decode_" + _SUFFIX[q.dtype])
        _lib.check(
            fn(
                q.data_ptr(), k_codes.data_ptr(), codebooks.data_ptr(), v.data_ptr(), out.data_ptr(),
                lse.data_ptr() if return_lse else None,
                workspace.data_ptr(), ws_bytes, B, H, N, D, M, K, strides, softmax_scale, splits,
                _lib.current_stream(q.device),
            )
        )  # fmt: skip
    return (out, lse) if return_lse else out


def attn_vq_prefill(q, k_codes, codebooks, v, *, k_exact=None, window_size=0, causal=True, softmax_scale=None,
                    return_lse=False, boundary_mode="block", q2=None, k2=None):
    """Prefill attention (seqlen_q == seqlen_k) over additive-quantiser key codes, optionally with an exact window.

    q, v [B,H,N,D] bf16/f16; k_codes [B,H,N,M] uint8; codebooks [H,M,K,D].  With `k_exact` [B,H,N,D]: keys
    j >= boundary(i) are exact (score q.k_exact inside the window i - j <= window_size; the strip between boundary and
    window uses q2.k2 when both are given), older keys use their reconstruction sum_m codebooks[h,m,code] scored
    with q2 if given else q.  boundary(i) = max(0, floor((i - W)/128)*128) for boundary_mode "block" (the rule of
    ops/attn_vq.py:311 and of the window kernel stages), max(0, i - W) for "exact".  One softmax over all visible
    keys: the window and far parts are merged inside the kernel.  Returns out [B,H,N,D] (and base-2 lse [B,H,N]).
    """
    from ._common import BOUNDARY, bhn_strides, check_same_16bit, last_dim_contiguous, ptr

    lib = _lib.load()
    _lib.require_gpu(q, k_codes, codebooks, v, k_exact, q2, k2)
    B, H, N, D = q.shape
    M, K = k_codes.shape[3], codebooks.shape[2]
    assert k_codes.shape == (B, H, N, M) and k_codes.dtype == torch.uint8
    assert codebooks.shape == (H, M, K, D), "codebooks must be [H,M,K,D]"
    assert v.shape == (B, H, N, D), "seqlen_q == seqlen_k prefill only"
    assert causal or k_exact is None, "non-causal attention takes quantised keys only"
    sfx = check_same_16bit(q, codebooks, v, k_exact, q2, k2)
    q, codebooks, v, k_exact, q2, k2 = last_dim_contiguous(q, codebooks, v, k_exact, q2, k2)
    if k_codes.stride(3) != 1 or k_codes.stride(2) != M:
        k_codes = k_codes.contiguous()
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)
    out = torch.empty((B, H, N, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device) if return_lse else None
    ws_bytes = lib.vqa_prefill_workspace_bytes(B, H, N, D)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    dummy = (0, 0, 0)
    strides = _lib.strides_array(
        *bhn_strides(q), k_codes.stride(0), k_codes.stride(1),
        codebooks.stride(0), codebooks.stride(1), codebooks.stride(2), *bhn_strides(v),
        *(bhn_strides(k_exact) if k_exact is not None else dummy),
        *(bhn_strides(q2) if q2 is not None else dummy),
        *(bhn_strides(k2) if k2 is not None else dummy),
        *bhn_strides(out),
    )
    with torch.cuda.device(q.device):
        rc = getattr(lib, "vqa_prefill_" + sfx)(
            ptr(q), ptr(k_codes), ptr(codebooks), ptr(v), ptr(k_exact), ptr(q2), ptr(k2), ptr(out), ptr(lse),
            ptr(workspace), ws_bytes, B, H, N, D, M, K, strides, int(window_size), BOUNDARY[boundary_mode],
            1 if causal else 0, softmax_scale, _lib.current_stream(q.device))
    _lib.check(rc)
    return (out, lse) if return_lse else out
