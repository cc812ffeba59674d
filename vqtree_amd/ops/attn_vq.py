"""Additive-code VQ attention entry points (counterpart of the reference's ops/attn_vq.py dispatch).

`attn_vq_decode` is the seqlen_q == 1 route the reference dispatches to `naive_attn`
(ops/attn_vq.py:247-248, 445-479) and its README promises as "a separate kernel" (ops/README.md:3).
Layouts follow the reference's attention modules: q, v [B,H,N,D]; codebooks [H,M,K,D]; codes [B,H,N,M] uint8.
"""
import math
from enum import Enum

import torch

from .. import _lib
from .mini_vq import multi_head_single_quantize, quantize_ids

BLOCK_SIZE = 128  # granularity of the far-context boundary (ops/attn_vq.py:23)

_SUFFIX = {torch.bfloat16: "bf16", torch.float16: "f16"}


def _last_dim_contiguous(x):
    return x if x.stride(-1) == 1 else x.contiguous()


def attn_vq_decode(q, k_codes, codebooks, v, *, softmax_scale=None, return_lse=False, num_splits=0, n_keys=None,
                   out=None, workspace=None, rope=None):
    """out[b,h] = softmax_j(scale * sum_m <q[b,h], codebooks[h,m,k_codes[b,h,j,m]]>) @ v[b,h]   (no mask).

    q [B,H,1,D] bf16/f16, k_codes [B,H,N,M] uint8, codebooks [H,M,K,D], v [B,H,N,D]  ->  out [B,H,1,D] (q's dtype)
    and, with return_lse, the base-2 log-sum-exp [B,H,1] fp32.

    `n_keys` (int32 tensor with one element, on the device): the number of keys to attend is read from it when the
    kernels run, N being only the capacity of the buffers -- for launch sequences recorded once (a HIP graph of a decode
    step) and replayed as the cache grows.  `out` / `workspace` let such a caller provide the buffers.

    `rope = (cos_row, sin_row)` (two [D] rows of the rotary tables, q's dtype): q is the UNROTATED query and is rotated
    to that position inside the lookup-table kernel, with the rounding of `apply_rope` -- the clamped ReRoPE query of a
    generation step without a launch of its own.
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

    if out is None:
        out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    assert out.shape == (B, H, 1, D) and out.dtype == q.dtype and out.stride(-1) == 1
    lse = torch.empty((B, H, 1), dtype=torch.float32, device=q.device) if return_lse else None
    splits = num_splits if num_splits > 0 else lib.vqa_decode_default_splits(B, H, N)
    ws_bytes = lib.vqa_decode_workspace_bytes(B, H, N, D, M, K, splits)
    if workspace is None:
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    assert workspace.numel() >= ws_bytes and workspace.dtype == torch.uint8
    strides = _lib.strides_array(
        q.stride(0), q.stride(1),
        k_codes.stride(0), k_codes.stride(1),
        codebooks.stride(0), codebooks.stride(1), codebooks.stride(2),
        v.stride(0), v.stride(1), v.stride(2),
        out.stride(0), out.stride(1),
    )  # fmt: skip
    if n_keys is not None:
        assert n_keys.dtype == torch.int32 and n_keys.numel() == 1 and n_keys.is_cuda
    with torch.cuda.device(q.device):
        tail = (k_codes.data_ptr(), codebooks.data_ptr(), v.data_ptr(), out.data_ptr(),
                lse.data_ptr() if return_lse else None,
                workspace.data_ptr(), ws_bytes, B, H, N, D, M, K, strides, softmax_scale, splits)  # fmt: skip
        stream = _lib.current_stream(q.device)
        if rope is not None:
            cos_row, sin_row = (t if t.is_contiguous() else t.contiguous() for t in rope)
            assert cos_row.shape == sin_row.shape == (D,) and cos_row.dtype == sin_row.dtype == q.dtype
            _lib.require_gpu(cos_row, sin_row)
            rc = getattr(lib, "vqa_decode_roped_" + _SUFFIX[q.dtype])(
                q.data_ptr(), cos_row.data_ptr(), sin_row.data_ptr(), *tail,
                None if n_keys is None else n_keys.data_ptr(), stream)
        elif n_keys is None:
            rc = getattr(lib, "vqa_decode_" + _SUFFIX[q.dtype])(q.data_ptr(), *tail, stream)
        else:
            rc = getattr(lib, "vqa_decode_devlen_" + _SUFFIX[q.dtype])(q.data_ptr(), *tail, n_keys.data_ptr(), stream)
        _lib.check(rc)
    return (out, lse) if return_lse else out


def attn_exact_decode(q, k, v, *, softmax_scale=None, return_lse=False, num_splits=0):
    """seqlen_q == 1 attention over exact keys: q [B,H,1,D], k / v [B,H,N,D] -> out [B,H,1,D] (and lse [B,H,1] fp32,
    base 2).  No mask: the single query sees every key."""
    lib = _lib.load()
    _lib.require_gpu(q, k, v)
    q, k, v = (_last_dim_contiguous(x) for x in (q, k, v))
    B, H, one, D = q.shape
    N = k.shape[2]
    assert one == 1 and k.shape == (B, H, N, D) and v.shape == (B, H, N, D)
    assert q.dtype == k.dtype == v.dtype and q.dtype in _SUFFIX, "Only support fp16 and bf16"
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)
    out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, 1), dtype=torch.float32, device=q.device) if return_lse else None
    S = num_splits if num_splits > 0 else lib.vqa_decode_default_splits(B, H, N)
    ws = torch.empty(lib.vqa_decode_exact_workspace_bytes(B, H, N, D, S), dtype=torch.uint8, device=q.device)
    strides = _lib.strides_array(q.stride(0), q.stride(1), k.stride(0), k.stride(1), k.stride(2), v.stride(0),
                                 v.stride(1), v.stride(2), out.stride(0), out.stride(1))
    with torch.cuda.device(q.device):
        rc = getattr(lib, "vqa_decode_exact_" + _SUFFIX[q.dtype])(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), None if lse is None else lse.data_ptr(),
            ws.data_ptr(), ws.numel(), B, H, N, D, strides, softmax_scale, S, _lib.current_stream(q.device))
    _lib.check(rc)
    return (out, lse) if return_lse else out


def attn_vq_decode_windowed(q, k_codes, codebooks, v, k_window, *, softmax_scale=None, q_window=None,
                            return_lse=False):
    """seqlen_q == 1 attention with an exact window: the last `k_window.shape[2]` keys are scored exactly
    (k_window [B,H,W,D], with `q_window` when the window uses another query, e.g. another rotary position), every
    earlier key through its codes; v [B,H,N,D] covers both.  One call: the coded and the exact streaming kernels
    write their split states into one workspace and a single merge produces the output."""
    lib = _lib.load()
    q_window = q if q_window is None else q_window
    _lib.require_gpu(q, q_window, k_codes, codebooks, v, k_window)
    B, H, one, D = q.shape
    N, W = v.shape[2], k_window.shape[2]
    M, K = codebooks.shape[1], codebooks.shape[2]
    assert one == 1 and q_window.shape == q.shape and 0 < W <= N and k_codes.shape[2] >= N - W
    assert k_window.shape == (B, H, W, D) and v.shape == (B, H, N, D) and codebooks.shape == (H, M, K, D)
    assert q.dtype == q_window.dtype == codebooks.dtype == v.dtype == k_window.dtype and q.dtype in _SUFFIX
    assert k_codes.dtype == torch.uint8 and k_codes.shape[3] == M
    q, q_window, codebooks, v, k_window = map(_last_dim_contiguous, (q, q_window, codebooks, v, k_window))
    if k_codes.stride(3) != 1 or k_codes.stride(2) != M:
        k_codes = k_codes.contiguous()
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)
    out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, 1), dtype=torch.float32, device=q.device) if return_lse else None
    ws = torch.empty(lib.vqa_decode_windowed_workspace_bytes(B, H, N, W, D, M), dtype=torch.uint8, device=q.device)
    strides = _lib.strides_array(q.stride(0), q.stride(1), q_window.stride(0), q_window.stride(1),
                                 k_codes.stride(0), k_codes.stride(1),
                                 codebooks.stride(0), codebooks.stride(1), codebooks.stride(2),
                                 v.stride(0), v.stride(1), v.stride(2),
                                 k_window.stride(0), k_window.stride(1), k_window.stride(2),
                                 out.stride(0), out.stride(1))
    with torch.cuda.device(q.device):
        rc = getattr(lib, "vqa_decode_windowed_" + _SUFFIX[q.dtype])(
            q.data_ptr(), q_window.data_ptr(), k_codes.data_ptr(), codebooks.data_ptr(), v.data_ptr(),
            k_window.data_ptr(), out.data_ptr(), None if lse is None else lse.data_ptr(), ws.data_ptr(), ws.numel(),
            B, H, N, W, D, M, K, strides, softmax_scale, _lib.current_stream(q.device))
    _lib.check(rc)
    return (out, lse) if return_lse else out


def attn_vq_prefill(q, k_codes, codebooks, v, *, k_exact=None, window_size=0, causal=True, softmax_scale=None,
                    return_lse=False, boundary_mode="block", q2=None, k2=None, schedule="default"):
    """Prefill attention (seqlen_q == seqlen_k) over additive-quantiser key codes, optionally with an exact window.

    q, v [B,H,N,D] bf16/f16; k_codes [B,H,N,M] uint8; codebooks [H,M,K,D].  With `k_exact` [B,H,N,D]: keys
    j >= boundary(i) are exact (score q.k_exact inside the window i - j <= window_size; the strip between boundary and
    window uses q2.k2 when both are given), older keys use their reconstruction sum_m codebooks[h,m,code] scored
    with q2 if given else q.  boundary(i) = max(0, floor((i - W)/128)*128) for boundary_mode "block" (the rule of
    ops/attn_vq.py:311 and of the window kernel stages), max(0, i - W) for "exact".  One softmax over all visible
    keys: the window and far parts are merged inside the kernel.  Returns out [B,H,N,D] (and base-2 lse [B,H,N]).
    `schedule`: "default" picks the route (one codebook with a block boundary: the codeword-space route of
    `vq_attn_forward`; otherwise the per-key kernel, on whichever of its two schedules the library picks for the
    shape); "per_key" forces the per-key kernel; "tiled" / "pipelined" force the per-key kernel on that schedule
    (pipelined: block boundary, window a multiple of 128, no q2 / k2).
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
    if q.dtype == torch.float32:
        return _attn_vq_prefill_f32(q, k_codes, codebooks, v, k_exact, q2, k2, causal, softmax_scale, return_lse)
    if (schedule == "default" and M == 1 and k_exact is not None and causal and boundary_mode == "block"
            and (q2 is None) == (k2 is None) and window_size % BLOCK_SIZE == 0 and N > window_size + BLOCK_SIZE):
        # One codebook: the far context is a softmax over the K codewords weighted by per-code key counts -- cost
        # O(N * K) instead of O(N^2) -- which is the reference's own formulation (ops/triton_fused_vq_attn.py:22-70).
        # The per-key kernel below only wins its place from M = 2 on: 384 us against 641 us at 8192 tokens, 256 codewords.
        from .triton_fused_vq_attn import vq_attn_forward

        ids = k_codes[..., 0].to(torch.int64)
        cnt, v_vq, vi = segmented_preprocess(ids, v, K, want_int64_counts=True)
        return vq_attn_forward(q, q if q2 is None else q2, k_exact, codebooks[:, 0], cnt,
                               k_exact if (q2 is None or k2 is None) else k2, v, v_vq, vi, window_size,
                               softmax_scale=softmax_scale, return_lse=return_lse)
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
    assert schedule in ("default", "per_key", "tiled", "pipelined")
    with torch.cuda.device(q.device):
        if schedule == "pipelined":
            assert q2 is None and k2 is None and boundary_mode == "block"
            rc = getattr(lib, "vqa_prefill_pipelined_" + sfx)(
                ptr(q), ptr(k_codes), ptr(codebooks), ptr(v), ptr(k_exact), ptr(out), ptr(lse), ptr(workspace),
                ws_bytes, B, H, N, D, M, K, strides, int(window_size), 1 if causal else 0, softmax_scale,
                _lib.current_stream(q.device))
        else:
            rc = getattr(lib, ("vqa_prefill_tiled_" if schedule == "tiled" else "vqa_prefill_") + sfx)(
                ptr(q), ptr(k_codes), ptr(codebooks), ptr(v), ptr(k_exact), ptr(q2), ptr(k2), ptr(out), ptr(lse),
                ptr(workspace), ws_bytes, B, H, N, D, M, K, strides, int(window_size), BOUNDARY[boundary_mode],
                1 if causal else 0, softmax_scale, _lib.current_stream(q.device))
    _lib.check(rc)
    return (out, lse) if return_lse else out


def _attn_vq_prefill_f32(q, k_codes, codebooks, v, k_exact, q2, k2, causal, softmax_scale, return_lse):
    """fp32 validation path: every visible key quantised (no exact window), plain fp32 arithmetic."""
    from ._common import bhn_strides, last_dim_contiguous, ptr

    assert k_exact is None and q2 is None and k2 is None, "the fp32 path takes quantised keys only"
    assert q.dtype == codebooks.dtype == v.dtype == torch.float32, "All tensors must have the same type"
    lib = _lib.load()
    B, H, N, D = q.shape
    M, K = k_codes.shape[3], codebooks.shape[2]
    q, codebooks, v = last_dim_contiguous(q, codebooks, v)
    if k_codes.stride(3) != 1 or k_codes.stride(2) != M:
        k_codes = k_codes.contiguous()
    out = torch.empty((B, H, N, D), dtype=torch.float32, device=q.device)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device) if return_lse else None
    strides = _lib.strides_array(*bhn_strides(q), k_codes.stride(0), k_codes.stride(1), codebooks.stride(0),
                                 codebooks.stride(1), codebooks.stride(2), *bhn_strides(v), *bhn_strides(out))
    with torch.cuda.device(q.device):
        rc = lib.vqa_prefill_f32(ptr(q), ptr(k_codes), ptr(codebooks), ptr(v), ptr(out), ptr(lse), B, H, N, D, M, K,
                                 strides, 1 if causal else 0, softmax_scale or 1.0 / math.sqrt(D),
                                 _lib.current_stream(q.device))
    _lib.check(rc)
    return (out, lse) if return_lse else out


# ---------------------------------------------------------------------------------------------------------------------
# Caller layer: the attention core of LlamaFlashAttention2VectorQuantizedReRoPE (ops/attn_vq.py:176-479) without the
# Hugging Face module around it -- projections, o_proj and the transformers Cache base class stay with the model code.
# ---------------------------------------------------------------------------------------------------------------------
class AttentionMode(Enum):
    SLOW_REFERNECE = 0  # (sic) spelling of the reference, ops/attn_vq.py:26-28
    SORT_BASED_LINEAR = 1


class VectorQuantizedReRoPECache:
    """Holds what the reference's cache of the same name configures (ops/attn_vq.py:31-52): the exact-window length,
    the per-head codebook [H,C,D], the `sphere` flag and the attention mode; plus, after a prefill, what its
    `update_prefill` stores for the generation steps (ops/attn_vq.py:89-127): per-codeword key counts and value sums
    (`count_state.CountState`), and -- with `generation_exact_window` -- the buffers of the last exact keys and values
    (`count_state.GenerationWindow`).

    `generation_exact_window=False` (default): a seqlen_q == 1 step attends over ALL keys through their codewords with
    the clamped query, the quantity `attn_vq_decode` computes over a code stream, here in O(C D) per step.
    `generation_exact_window=True`: the step equals the last row of a prefill over the same tokens -- exact window,
    clamped-query strip, codewords before the 128-aligned far boundary."""

    def __init__(self, window_length, codebook, sphere=False, *, attention_mode=AttentionMode.SORT_BASED_LINEAR,
                 generation_exact_window=False):
        assert codebook.shape[1] % 128 == 0
        self.window_length = window_length
        self.codebook = codebook
        self.sphere = sphere
        self.attention_mode = attention_mode
        self.generation_exact_window = generation_exact_window
        # per layer: codeword ids of the prefill, [B,H,N,1] uint8 (int16 above 256 codewords) -- 1 or 2 bytes per key
        # next to the 2 D bytes of a value row, kept as the record of how the prefill was encoded.  The values (and
        # keys) themselves are NOT kept: the generation steps run on the count state, O(C D) per (batch, head).
        self.key_codes = []
        self.decode_state = []   # per layer: CountState or GenerationWindow
        self.seq_lengths = []    # per layer: tokens seen
        self.seen_tokens = 0

    def get_seq_length(self, layer_idx=0):
        return 0 if len(self.seq_lengths) <= layer_idx else self.seq_lengths[layer_idx]

    def get_usable_length(self, new_seq_length, layer_idx=0):
        return self.get_seq_length(layer_idx)

    def get_max_length(self):
        return int(1e8)  # "some safe number", ops/attn_vq.py:85-87

    # what a transformers (5.x) model asks of a cache while it builds its (unused) causal mask
    def get_query_offset(self, layer_idx=0):
        return self.get_seq_length(layer_idx)

    def get_mask_sizes(self, query_length, layer_idx=0):
        return self.get_seq_length(layer_idx) + query_length, 0


def rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


_ROPE_TABLE_CACHE = {}


def rope_tables(head_dim, n_pos, base=10000.0, dtype=torch.float32, device=None):
    """cos / sin [n_pos, D] of the transformers ~4.37 rotary embedding the reference's modules call
    (inv_freq = base^(-2r/D), emb = cat(freqs, freqs)), cast to the model dtype.  Tables are kept per
    (head_dim, base, dtype, device) and grown in powers of two, like the model's own cached rotary module."""
    key = (head_dim, float(base), dtype, str(device))
    have = _ROPE_TABLE_CACHE.get(key)
    if have is None or have[0].shape[0] < n_pos:
        size = 1 << max(0, int(n_pos) - 1).bit_length()
        inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim))
        freqs = torch.outer(torch.arange(size, dtype=torch.float32, device=device), inv_freq)
        emb = torch.cat((freqs, freqs), dim=-1)
        have = (emb.cos().to(dtype), emb.sin().to(dtype))
        _ROPE_TABLE_CACHE[key] = have
    return have[0][:n_pos], have[1][:n_pos]


def apply_rope(x, cos, sin, positions, also_fixed=None):
    """x * cos[p] + rotate_half(x) * sin[p] for x [B,H,N,D]; `positions` is a LongTensor [B,N] or one int for every
    row.  16-bit tensors on the GPU run the HIP rotary kernel, whose rounding (each product and the sum rounded to the
    element type) is that of this very expression evaluated on 16-bit tensors; anything else evaluates the expression
    with torch operators.  `also_fixed = p` (with per-row positions) returns a pair: the rows at their own positions
    and the same rows at the single position p, from one pass over x."""
    from .. import _lib
    from ._common import SUFFIX, bhn_strides, ptr

    if x.is_cuda and x.dtype in SUFFIX and cos.dtype == x.dtype and x.shape[-1] % 16 == 0:
        lib = _lib.load()
        B, H, N, D = x.shape
        x = x if x.stride(-1) == 1 else x.contiguous()
        cos = cos if cos.stride(-1) == 1 else cos.contiguous()
        sin = sin if sin.stride(-1) == 1 and sin.stride(0) == cos.stride(0) else sin.contiguous()
        if sin.stride(0) != cos.stride(0):
            cos = cos.contiguous()
        out = torch.empty((B, H, N, D), dtype=x.dtype, device=x.device)
        fixed = isinstance(positions, int)
        assert also_fixed is None or not fixed
        out2 = torch.empty_like(out) if also_fixed is not None else None
        if not fixed:
            positions = positions.to(torch.int64)
            assert positions.shape == (B, N)
        strides = _lib.strides_array(*bhn_strides(x), *((0, 0) if fixed else (positions.stride(0), positions.stride(1))),
                                     *bhn_strides(out))
        with torch.cuda.device(x.device):
            fixed_pos = positions if fixed else (int(also_fixed) if also_fixed is not None else 0)
            rc = getattr(lib, "vqa_rope_" + SUFFIX[x.dtype])(ptr(x), None if fixed else ptr(positions), ptr(cos),
                                                             ptr(sin), ptr(out), ptr(out2), B, H, N, D, cos.shape[0],
                                                             cos.stride(0), strides, fixed_pos,
                                                             _lib.current_stream(x.device))
        _lib.check(rc)
        return out if also_fixed is None else (out, out2)
    if isinstance(positions, int):
        c, s = cos[positions], sin[positions]
    else:
        c, s = cos[positions].unsqueeze(1), sin[positions].unsqueeze(1)  # [B,1,N,D]
    out = x * c + rotate_half(x) * s
    if also_fixed is None:
        return out
    return out, x * cos[also_fixed] + rotate_half(x) * sin[also_fixed]


def rerope_operands(query_states, key_states, position_ids, window_length, rope_base=10000.0, past_length=0):
    """(q1, k1, q2) of ops/attn_vq.py:402-407: rotary at the true positions, and the query at the clamped position
    window_length + 1.  position_ids [B,N]; states [B,H,N,D].

    The rotary tables are sized on the host, from `past_length + N` (the positions a model hands over are
    past_length .. past_length + N - 1, or smaller with left padding): reading the largest position back from the
    device would stall every layer's prefill on a device-to-host copy and keep the route out of a HIP graph.  A
    position beyond the tables is clamped to their last row by the rotary kernel."""
    B, H, N, D = query_states.shape
    n_pos = max(past_length + N, window_length + 2)
    cos, sin = rope_tables(D, n_pos, rope_base, query_states.dtype, query_states.device)
    q1, q2 = apply_rope(query_states, cos, sin, position_ids, also_fixed=window_length + 1)
    k1 = apply_rope(key_states, cos, sin, position_ids)
    return q1, k1, q2


def sort_based_preprocess(vq_key_ids, vq_key_onehot, value_states, block=BLOCK_SIZE):
    """Inputs of the count kernel from the key codes, following ops/attn_vq.py:352-384, 410-413: running per-code key
    counts, V sorted by (code, position) with per-code prefix sums (fp32 cumsum, cast to the model dtype), and the
    prefix-sum row index per (block, code).  Returns (k_vq_cnt [B,H,N//block,C] int64, v_vq [B,H,N+1,D],
    vi [B,H,N//block,C] int64)."""
    B, H, N = vq_key_ids.shape
    D = value_states.shape[-1]
    dtype, device = value_states.dtype, value_states.device
    assert vq_key_onehot.shape[-1] < (1 << 13) and N < (1 << 18)
    cum = torch.cumsum(vq_key_onehot, dim=2)
    order = ((vq_key_ids.to(torch.int32) << 18) + torch.arange(N, dtype=torch.int32, device=device)).argsort()
    v_vq = torch.zeros((B, H, N + 1, D), device=device, dtype=torch.float32)
    v_vq[:, :, 1:] = torch.gather(value_states, 2, order[..., None].expand(-1, -1, -1, D)).float()
    v_vq = torch.cumsum(v_vq, 2)
    total = cum[:, :, -1]
    start = torch.cumsum(total, dim=-1) - total
    seg_base = v_vq.gather(2, start[..., None].expand(-1, -1, -1, D))
    code_sorted = torch.gather(vq_key_ids, 2, order)
    v_vq[:, :, 1:] -= seg_base.gather(2, code_sorted[..., None].expand(-1, -1, -1, D))
    vi = cum + start[:, :, None, :]
    return cum[:, :, block - 1::block].contiguous(), v_vq.to(dtype), vi[:, :, block - 1::block].contiguous()


def segmented_preprocess(vq_key_ids, value_states, n_codes, block=BLOCK_SIZE, want_int64_counts=False, state=None):
    """Same three tensors as `sort_based_preprocess`, built by the HIP preprocessing kernels (per-block histograms,
    scan, scatter into (code, position) order, one running fp32 sum per code) instead of the one-hot cumulative sum,
    argsort and global prefix sum of ops/attn_vq.py:352-384.  Returns (counts [B,H,N//block,C] in the model dtype, or
    int64 when `want_int64_counts`; v_vq [B,H,N+1,D]; vi [B,H,N//block,C] int64).  `state` (a fresh
    `count_state.CountState`): the same pass also leaves the count state of all N keys in it."""
    from .. import _lib
    from ._common import SUFFIX, bhn_strides, ptr

    assert block == BLOCK_SIZE
    lib = _lib.load()
    _lib.require_gpu(vq_key_ids, value_states)
    B, H, N = vq_key_ids.shape
    D = value_states.shape[-1]
    dtype, device = value_states.dtype, value_states.device
    assert dtype in SUFFIX and vq_key_ids.dtype == torch.int64
    assert n_codes < (1 << 13) and N < (1 << 18), "limits of the reference's sort keys (ops/attn_vq.py:355-359)"
    value_states = value_states if value_states.stride(-1) == 1 else value_states.contiguous()
    NT = N // block
    cnt = torch.empty((B, H, NT, n_codes), dtype=torch.int64 if want_int64_counts else dtype, device=device)
    vi = torch.empty((B, H, NT, n_codes), dtype=torch.int64, device=device)
    v_vq = torch.empty((B, H, N + 1, D), dtype=dtype, device=device)
    ws = torch.empty(lib.vqa_preprocess_workspace_bytes(B, H, N, n_codes), dtype=torch.uint8, device=device)
    strides = _lib.strides_array(*bhn_strides(vq_key_ids), *bhn_strides(value_states), *bhn_strides(cnt),
                                 *bhn_strides(cnt), *bhn_strides(v_vq), *bhn_strides(vi))
    head = (ptr(vq_key_ids), ptr(value_states), ptr(cnt) if want_int64_counts else None,
            None if want_int64_counts else ptr(cnt), ptr(v_vq), ptr(vi))
    tail = (ptr(ws), ws.numel(), B, H, N, D, n_codes, strides, _lib.current_stream(device))
    with torch.cuda.device(device):
        if state is None:
            rc = getattr(lib, "vqa_preprocess_" + SUFFIX[dtype])(*head, *tail)
        else:
            assert state.n_keys == 0 and state.cnt.shape == (B, H, n_codes) and state.vsum.shape == (B, H, n_codes, D)
            rc = getattr(lib, "vqa_preprocess_state_" + SUFFIX[dtype])(*head, ptr(state.cnt), ptr(state.vsum), *tail)
    _lib.check(rc)
    if state is not None:
        state.n_keys = N
    return cnt, v_vq, vi


def long_prefilling_sort_based_linear(query_states, key_states, value_states, position_ids, cache, layer_idx=0,
                                      rope_base=10000.0):
    """Linear-time prefill with VQ memory (ops/attn_vq.py:336-443): encode keys with the head's codebook, build the
    count-kernel inputs, run `vq_attn_forward`.  States [B,H,N,D]; returns [B, N, H*D] like the reference (no o_proj)."""
    from .triton_fused_vq_attn import vq_attn_forward

    B, H, N, D = query_states.shape
    dtype = query_states.dtype
    from .count_state import CountState

    ids = quantize_ids(key_states, cache.codebook)
    # the count state of all keys (what the generation steps of the default mode run on) falls out of the same pass
    state = None
    if not cache.generation_exact_window and len(cache.seq_lengths) <= layer_idx:
        state = CountState(B, H, cache.codebook.shape[1], D, value_states.device)
    cnt, v_vq, vi = segmented_preprocess(ids, value_states, cache.codebook.shape[1], want_int64_counts=True, state=state)
    q1, k1, q2 = rerope_operands(query_states, key_states, position_ids, cache.window_length, rope_base)
    out = vq_attn_forward(q1, q2, k1, cache.codebook, cnt, key_states, value_states, v_vq, vi,
                          cache.window_length, softmax_scale=1 / math.sqrt(D))
    _remember(cache, layer_idx, ids, value_states, N, k1, key_states, state=state)
    return out.transpose(1, 2).contiguous().flatten(2)


def long_prefilling_per_key(query_states, key_states, value_states, position_ids, cache, layer_idx=0,
                            rope_base=10000.0):
    """Same result through the fused per-key kernel (`attn_vq_prefill` with M = 1): no one-hot cumsum, no sort, no
    merge pass.  Needs a codebook of at most 256 entries (uint8 codes)."""
    B, H, N, D = query_states.shape
    assert cache.codebook.shape[1] <= 256
    ids = quantize_ids(key_states, cache.codebook)
    q1, k1, q2 = rerope_operands(query_states, key_states, position_ids, cache.window_length, rope_base)
    out = attn_vq_prefill(q1, ids.to(torch.uint8).unsqueeze(-1), cache.codebook.unsqueeze(1), value_states,
                          k_exact=k1, window_size=cache.window_length, q2=q2, k2=key_states,
                          softmax_scale=1 / math.sqrt(D), schedule="per_key")
    _remember(cache, layer_idx, ids, value_states, N, k1, key_states)
    return out.transpose(1, 2).contiguous().flatten(2)


def _remember(cache, layer_idx, ids, value_states, n_tokens, k1, key_states, state=None):
    """Record a prefill in the cache (what `update_prefill` keeps, ops/attn_vq.py:89-127): the sequence length, so
    that the next seqlen_q == 1 call is recognised as a generation step; the codeword ids; and the state the
    generation steps run on -- the count state over all keys, or, with `generation_exact_window`, the count state
    below the far boundary of the next query plus buffers of window + 256 exact keys above it.  The state is built
    here (a fraction of a millisecond per layer) and nothing of the prefill's [B,H,N,D] tensors is referenced
    afterwards: the memory of the cache is O(C D + window D) per (batch, head) plus the code bytes, whatever N is."""
    from .count_state import CountState, GenerationWindow

    if layer_idx == 0:
        cache.seen_tokens += n_tokens
    if len(cache.seq_lengths) <= layer_idx:
        B, H, _, D = value_states.shape
        C = cache.codebook.shape[1]
        code_dtype = torch.uint8 if C <= 256 else torch.int16
        cache.key_codes.append(ids.to(code_dtype).unsqueeze(-1).contiguous())
        if state is None:  # (else: the preprocessing of the linear prefill has built it)
            state = CountState(B, H, C, D, value_states.device)
            if cache.generation_exact_window:
                state = GenerationWindow(cache.window_length, k1, key_states, value_states, ids, n_tokens, state)
            else:
                state.add(ids, value_states)
        cache.decode_state.append(state)
        cache.seq_lengths.append(n_tokens)


def long_prefilling_slow_reference_impl(query_states, key_states, value_states, position_ids, cache, layer_idx=0,
                                        rope_base=10000.0):
    """Per-query loops of ops/attn_vq.py:278-334, kept for checking the linear-time path (torch operators around the
    HIP key encoder)."""
    B, H, N, D = query_states.shape
    W = cache.window_length
    q1, k1, q2 = rerope_operands(query_states, key_states, position_ids, W, rope_base)
    k_hat, ids, _ = multi_head_single_quantize(key_states, cache.codebook)
    _remember(cache, layer_idx, ids, value_states, N, k1, key_states)
    scale = 1.0 / math.sqrt(D)
    output = torch.zeros_like(query_states, memory_format=torch.contiguous_format)
    for b in range(B):
        for h in range(H):
            for qi in range(N):
                boundary = max(0, (qi - W) // BLOCK_SIZE * BLOCK_SIZE)
                local_boundary = max(0, qi - W)
                attn = [q1[b, h, qi] @ k1[b, h, local_boundary:qi + 1].T]
                v = [value_states[b, h, local_boundary:qi + 1]]
                if local_boundary > 0:
                    attn.append(q2[b, h, qi] @ key_states[b, h, boundary:local_boundary].T)
                    v.append(value_states[b, h, boundary:local_boundary])
                if boundary > 0:
                    attn.append(q2[b, h, qi] @ k_hat[b, h, :boundary].T)
                    v.append(value_states[b, h, :boundary])
                w = torch.softmax(torch.cat(attn).float() * scale, dim=0).to(value_states.dtype)
                output[b, h, qi] = w @ torch.cat(v)
    return output.transpose(1, 2).contiguous().flatten(2)


def dispatch_attn(query_states, key_states, value_states, position_ids, cache, layer_idx=0, rope_base=10000.0):
    """Routing of `_dispatch_attn_impl` (ops/attn_vq.py:225-248): a prefill longer than window + 128 goes to the
    VQ-memory path chosen by `cache.attention_mode`; a shorter prefill is plain causal attention on the rotated
    operands; a seqlen_q == 1 step attends over the cached codes (the route the reference leaves unimplemented)."""
    from .triton_fused_local_attn import flash_attn_func as causal_window_attention

    B, H, q_len, D = query_states.shape
    assert not cache.sphere, "Not implemented"  # as the reference's forward, ops/attn_vq.py:198
    is_prefilling = cache.get_seq_length(layer_idx) == 0
    if is_prefilling and q_len > cache.window_length + BLOCK_SIZE:
        if cache.attention_mode == AttentionMode.SORT_BASED_LINEAR:
            return long_prefilling_sort_based_linear(query_states, key_states, value_states, position_ids, cache,
                                                     layer_idx, rope_base)
        if cache.attention_mode == AttentionMode.SLOW_REFERNECE:
            return long_prefilling_slow_reference_impl(query_states, key_states, value_states, position_ids, cache,
                                                       layer_idx, rope_base)
        raise KeyError(f"Bad attention mode: {cache.attention_mode}")
    if is_prefilling:
        q1, k1, _ = rerope_operands(query_states, key_states, position_ids, cache.window_length, rope_base)
        out = causal_window_attention(q1.transpose(1, 2), k1.transpose(1, 2), value_states.transpose(1, 2), q_len,
                                      softmax_scale=1 / math.sqrt(D))
        ids = quantize_ids(key_states, cache.codebook)
        _remember(cache, layer_idx, ids, value_states, q_len, k1, key_states)
        return out.contiguous().flatten(2)
    assert q_len == 1, "Only support prefilling or generation"
    # Generation step on the state the prefill left (the route the reference leaves unimplemented,
    # ops/attn_vq.py:176-223): O(C D) per step, whatever the context length and the codebook size.
    from .count_state import count_step

    W = cache.window_length
    t = cache.seq_lengths[layer_idx]  # position of the new token
    ids = quantize_ids(key_states, cache.codebook)
    state = cache.decode_state[layer_idx]
    scale = 1 / math.sqrt(D)
    cos, sin = rope_tables(D, max(W + 2, t + 1) if cache.generation_exact_window else W + 2, rope_base,
                           query_states.dtype, query_states.device)
    if cache.generation_exact_window:
        q2 = apply_rope(query_states, cos, sin, W + 1)
        # true-position rotary at the positions the caller gives (per batch row; normally all equal to t)
        q1 = apply_rope(query_states, cos, sin, position_ids)
        k1 = apply_rope(key_states, cos, sin, position_ids)
        state.append(k1, key_states, value_states, ids)
        out = state.attend(q1, q2, cache.codebook, scale)
    else:
        # one launch: the new key into the state, the clamped rotary of the query, the count-weighted softmax
        out = count_step(query_states, cache.codebook, state, ids, value_states, rope=(cos[W + 1], sin[W + 1]),
                         softmax_scale=scale)
    cache.seq_lengths[layer_idx] = t + 1
    if layer_idx == 0:
        cache.seen_tokens += 1
    return out.transpose(1, 2).contiguous().flatten(2)


def __getattr__(name):
    # The transformers modules (`LlamaFlashAttention2VectorQuantizedReRoPE`, `use_rerope`, ops/attn_vq.py:176, 482)
    # live in hf_llama and are imported on first use, so that the operators do not pay for importing transformers.
    if name in ("LlamaFlashAttention2VectorQuantizedReRoPE", "use_rerope"):
        from . import hf_llama

        return hf_llama.use_vq_rerope if name == "use_rerope" else getattr(hf_llama, name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
