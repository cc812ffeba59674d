"""Count state of a single-codebook VQ key cache and the generation step over it.

The reference's cache stores, after a prefill, per-codeword key counts and cumulated values (`update_prefill`,
ops/attn_vq.py:89-127) plus buffers of the last `window_length` keys and values, for a seqlen_q == 1 route it never
implements (ops/attn_vq.py:176-223 raises, 445-479 is a dense fallback).  This module is that route: with one codebook
a quantised key IS a codeword, so attention over all N quantised keys equals count-weighted attention over the C
codewords -- O(C D) per step instead of O(N D).

`CountState` is the far-context state (HIP kernels `vqa_count_state_add_*`, `vqa_count_decode_*`);
`GenerationWindow` adds the buffers of exact keys that keep a generation step identical to the last row of a prefill
over the same tokens (exact window with true-position rotary, clamped-query strip up to the next multiple of 128,
codewords before that).
"""
import math

import torch

from .. import _lib
from ._common import SUFFIX, ptr

BLOCK_SIZE = 128


class CountState:
    """cnt [B,H,C] int32, vsum [B,H,C,D] fp32: counts and value sums of the keys folded in so far, per codeword."""

    def __init__(self, B, H, C, D, device):
        self.cnt = torch.zeros((B, H, C), dtype=torch.int32, device=device)
        self.vsum = torch.zeros((B, H, C, D), dtype=torch.float32, device=device)
        self.n_keys = 0

    def add(self, ids, v):
        """Fold T keys in: ids [B,H,T] int64 codeword indices, v [B,H,T,D] 16-bit values."""
        lib = _lib.load()
        _lib.require_gpu(ids, v, self.cnt)
        B, H, C = self.cnt.shape
        D = self.vsum.shape[-1]
        T = ids.shape[2]
        assert ids.dtype == torch.int64 and ids.shape == (B, H, T) and v.shape == (B, H, T, D)
        assert v.dtype in SUFFIX, "Only support fp16 and bf16"
        if T == 0:
            return self
        v = v if v.stride(-1) == 1 else v.contiguous()
        strides = _lib.strides_array(ids.stride(0), ids.stride(1), ids.stride(2), v.stride(0), v.stride(1), v.stride(2))
        with torch.cuda.device(v.device):
            rc = getattr(lib, "vqa_count_state_add_" + SUFFIX[v.dtype])(
                ptr(ids), ptr(v), ptr(self.cnt), ptr(self.vsum), B, H, T, D, C, strides, _lib.current_stream(v.device))
        _lib.check(rc)
        self.n_keys += T
        return self


def count_decode(q, codebook, state, *, softmax_scale=None, return_lse=False):
    """out[b,h] = sum_c exp(s_c) Vsum[c] / sum_c cnt[c] exp(s_c), s_c = <q[b,h], codebook[h,c]> * scale, over the
    codewords that have keys.  q [B,H,1,D], codebook [H,C,D] -> out [B,H,1,D] (q's dtype) and, with return_lse, the
    base-2 log-sum-exp [B,H,1] fp32 (-inf, with out = 0, for an empty state)."""
    lib = _lib.load()
    _lib.require_gpu(q, codebook, state.cnt)
    B, H, one, D = q.shape
    C = codebook.shape[1]
    assert one == 1 and codebook.shape == (H, C, D) and state.cnt.shape == (B, H, C) and state.vsum.shape[-1] == D
    assert q.dtype == codebook.dtype and q.dtype in SUFFIX, "Only support fp16 and bf16"
    q = q if q.stride(-1) == 1 else q.contiguous()
    codebook = codebook if codebook.stride(-1) == 1 else codebook.contiguous()
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)
    out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, 1), dtype=torch.float32, device=q.device) if return_lse else None
    strides = _lib.strides_array(q.stride(0), q.stride(1), codebook.stride(0), codebook.stride(1), out.stride(0),
                                 out.stride(1))
    with torch.cuda.device(q.device):
        rc = getattr(lib, "vqa_count_decode_" + SUFFIX[q.dtype])(
            ptr(q), ptr(codebook), ptr(state.cnt), ptr(state.vsum), ptr(out), ptr(lse), B, H, C, D, strides,
            softmax_scale, _lib.current_stream(q.device))
    _lib.check(rc)
    return (out, lse) if return_lse else out


def count_step(q, codebook, state, ids, v, *, rope=None, softmax_scale=None, return_lse=False):
    """One generation step on the state in one launch: fold the new key (ids [B,H,1] int64, v [B,H,1,D]) into `state`,
    rotate the raw query q [B,H,1,D] with `rope = (cos_row, sin_row)` (two [D] rows; None: q comes rotated) and attend
    over the updated state.  Equal, bit for bit, to `state.add(ids, v)`, `apply_rope(q, ...)`, `count_decode(...)`."""
    lib = _lib.load()
    _lib.require_gpu(q, codebook, state.cnt, ids, v)
    B, H, one, D = q.shape
    C = codebook.shape[1]
    assert one == 1 and codebook.shape == (H, C, D) and state.cnt.shape == (B, H, C) and state.vsum.shape[-1] == D
    assert ids.shape == (B, H, 1) and ids.dtype == torch.int64 and v.shape == (B, H, 1, D)
    assert q.dtype == codebook.dtype == v.dtype and q.dtype in SUFFIX, "Only support fp16 and bf16"
    q, v = (t if t.stride(-1) == 1 else t.contiguous() for t in (q, v))
    codebook = codebook if codebook.stride(-1) == 1 else codebook.contiguous()
    cos_row = sin_row = None
    if rope is not None:
        cos_row, sin_row = (t if t.is_contiguous() else t.contiguous() for t in rope)
        assert cos_row.shape == sin_row.shape == (D,) and cos_row.dtype == sin_row.dtype == q.dtype
    softmax_scale = softmax_scale or 1.0 / math.sqrt(D)
    out = torch.empty((B, H, 1, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, 1), dtype=torch.float32, device=q.device) if return_lse else None
    strides = _lib.strides_array(q.stride(0), q.stride(1), codebook.stride(0), codebook.stride(1), out.stride(0),
                                 out.stride(1), ids.stride(0), ids.stride(1), v.stride(0), v.stride(1))
    with torch.cuda.device(q.device):
        rc = getattr(lib, "vqa_count_step_" + SUFFIX[q.dtype])(
            ptr(q), ptr(cos_row), ptr(sin_row), ptr(ids), ptr(v), ptr(codebook), ptr(state.cnt), ptr(state.vsum),
            ptr(out), ptr(lse), B, H, C, D, strides, softmax_scale, _lib.current_stream(q.device))
    _lib.check(rc)
    state.n_keys += 1
    return (out, lse) if return_lse else out


def far_boundary(position, window):
    """First key that is NOT replaced by its codeword for the query at `position` (ops/attn_vq.py:283, 311)."""
    return max(0, (position - window) // BLOCK_SIZE * BLOCK_SIZE)


class GenerationWindow:
    """Exact keys of the positions [base, length): the keys at their true rotary positions (k1), unrotated (k, scored
    by the clamped query in the strip between the far boundary and the window), the values and the codeword indices,
    in buffers of window + 2 * 128 rows.  When the far boundary of the next query moves past `base`, the rows in
    between are folded into the count state and the buffers slide."""

    def __init__(self, window, k1, k, v, ids, length, state):
        B, H, _, D = k.shape
        self.window = window
        self.cap = window + 2 * BLOCK_SIZE
        self.state = state
        self.length = length                      # tokens seen
        self.base = far_boundary(length, window)  # boundary of the query that comes next, at position `length`
        state.add(ids[:, :, :self.base], v[:, :, :self.base])
        n = length - self.base
        assert n <= self.cap
        self.k1, self.k, self.v = (torch.zeros((B, H, self.cap, D), dtype=k.dtype, device=k.device) for _ in range(3))
        self.ids = torch.zeros((B, H, self.cap), dtype=torch.int64, device=k.device)
        self.k1[:, :, :n] = k1[:, :, self.base:length]
        self.k[:, :, :n] = k[:, :, self.base:length]
        self.v[:, :, :n] = v[:, :, self.base:length]
        self.ids[:, :, :n] = ids[:, :, self.base:length]

    def append(self, k1, k, v, ids):
        """The key of the new token (position `length`); afterwards the buffers cover what the query at that same
        position treats exactly."""
        t = self.length
        new_base = far_boundary(t, self.window)
        if new_base > self.base:
            m = new_base - self.base
            n = t - self.base
            self.state.add(self.ids[:, :, :m], self.v[:, :, :m])
            for buf in (self.k1, self.k, self.v):
                buf[:, :, :n - m] = buf[:, :, m:n].clone()
            self.ids[:, :, :n - m] = self.ids[:, :, m:n].clone()
            self.base = new_base
        i = t - self.base
        assert i < self.cap
        self.k1[:, :, i], self.k[:, :, i], self.v[:, :, i], self.ids[:, :, i] = k1[:, :, 0], k[:, :, 0], v[:, :, 0], ids[:, :, 0]
        self.length = t + 1

    def attend(self, q1, q2, codebook, softmax_scale):
        """Attention of the query at position length - 1 (its own key appended): exact window with q1 / k1, strip
        with q2 / k, codewords with q2; the three states merged by log-sum-exp.  Returns [B,H,1,D]."""
        from .attn_vq import attn_exact_decode
        from .triton_fused_vq_attn import merge_state_in_place

        t = self.length - 1
        B, H, _, D = q1.shape
        lo = max(0, t - self.window) - self.base  # first buffer row inside the window
        hi = t - self.base + 1
        out, lse = attn_exact_decode(q1, self.k1[:, :, lo:hi], self.v[:, :, lo:hi], softmax_scale=softmax_scale,
                                     return_lse=True)
        flat = lambda o, s: (o.view(1, B * H, D), s.view(1, B * H))
        if lo > 0:
            o2, s2 = attn_exact_decode(q2, self.k[:, :, :lo], self.v[:, :, :lo], softmax_scale=softmax_scale,
                                       return_lse=True)
            merge_state_in_place(*flat(out, lse), *flat(o2, s2))
        if self.base > 0:
            o3, s3 = count_decode(q2, codebook, self.state, softmax_scale=softmax_scale, return_lse=True)
            merge_state_in_place(*flat(out, lse), *flat(o3, s3))
        return out
