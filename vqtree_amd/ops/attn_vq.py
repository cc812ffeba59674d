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
