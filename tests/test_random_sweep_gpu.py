"""Seeded sweep over randomly drawn shapes, dtypes, windows and modes: every attention entry point against the CPU
oracle (same tolerance as the targeted tests).  The draw is fixed by the seed, so the cases never change."""
import math
import random

import pytest
import torch

import oracle
from vqtree_amd.ops import (triton_fused_attn_rerope, triton_fused_local_attn, triton_fused_local_attn2,
                            triton_fused_local_attn_rerope)
from vqtree_amd.ops.attn_vq import attn_exact_decode, attn_vq_decode, attn_vq_prefill

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 63, 64, 65, 127, 128, 129, 200, 255, 256, 257, 383, 500, 640, 777, 1000, 1300]
WINDOWS = [0, 1, 64, 100, 128, 256, 300, 512]


def _rn(*shape, seed, dtype, std=1.0):
    g = torch.Generator("cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def _close(got, want):
    got, want = got.float().cpu(), want.float()
    return bool(((got - want).abs() <= 2e-2 + 1e-2 * want.abs()).all())


def _draw(it, rng):
    return dict(dtype=rng.choice([torch.bfloat16, torch.float16]), D=rng.choice([64, 128]), B=rng.choice([1, 2]),
                H=rng.choice([1, 2, 3]), N=rng.choice(LENGTHS), W=rng.choice(WINDOWS), M=rng.choice([1, 2, 4, 8]),
                K=rng.choice([32, 64, 256]), mode=rng.choice(["block", "exact"]),
                causal=rng.choice([True, True, False]), rer=rng.choice([False, True]),
                window_mode=rng.choice(["strict", "loose", "rerope"]), seed=1000 + it)


def test_seeded_random_sweep():
    rng = random.Random(0)
    failures = []
    for it in range(80):
        c = _draw(it, rng)
        dtype, D, B, H, N, W, M, K = (c[k] for k in ("dtype", "D", "B", "H", "N", "W", "M", "K"))
        print(f"sweep case {it}: {c}", flush=True)
        q, k, v, q2, k2 = (_rn(B, H, N, D, seed=c["seed"] + i, dtype=dtype, std=0.8) for i in range(5))
        cb = _rn(H, M, K, D, seed=c["seed"] + 9, dtype=dtype, std=0.5 / math.sqrt(M))
        codes = torch.randint(0, K, (B, H, N, M), generator=torch.Generator("cpu").manual_seed(c["seed"] + 10),
                              dtype=torch.int32).to(torch.uint8)
        scale = 1 / math.sqrt(D)
        kind = it % 4
        if kind == 0:  # additive-code prefill, with or without an exact window / ReRoPE strip
            kw = dict(k_exact=k, window_size=W, boundary_mode=c["mode"]) if W > 0 else dict(causal=c["causal"])
            if W > 0 and c["rer"]:
                kw.update(q2=q2, k2=k2)
            want, _ = oracle.attn_vq_prefill(q, codes, cb, v, **kw)
            kw = {a: (b.cuda() if torch.is_tensor(b) else b) for a, b in kw.items()}
            ok = _close(attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), **kw), want)
        elif kind == 1:  # sliding windows
            m = c["window_mode"]
            Wl = max(W, 1) if m == "strict" else max(128, W // 128 * 128)
            want, _ = oracle.local_attn(q, k, v, Wl, m, None, q2=q2, k2=k2)
            t = lambda x: x.transpose(1, 2).contiguous().cuda()
            if m == "strict":
                got = triton_fused_local_attn.flash_attn_func(t(q), t(k), t(v), Wl)
            elif m == "loose":
                got = triton_fused_local_attn2.flash_attn_func(t(q), t(k), t(v), Wl)
            else:
                got = triton_fused_local_attn_rerope.flash_attn_func(t(q), t(q2), t(k), t(k2), t(v), Wl)
            ok = _close(got.transpose(1, 2), want)
        elif kind == 2:  # full-context ReRoPE
            Wf = max(W, 1)
            want, _ = oracle.rerope_full(q, q2, k, k2, v, c["causal"], scale, Wf)
            ok = _close(triton_fused_attn_rerope.attention(q.cuda(), q2.cuda(), k.cuda(), k2.cuda(), v.cuda(),
                                                           c["causal"], scale, Wf), want)
        else:  # coded and exact-key decode
            qd = q[:, :, :1]
            want, _ = oracle.attn_vq_decode(qd, codes, cb, v, scale)
            ok = _close(attn_vq_decode(qd.cuda(), codes.cuda(), cb.cuda(), v.cuda()), want)
            scores = qd.float() @ k.float().transpose(-1, -2) * scale
            want2, _ = oracle.attend(scores, torch.ones(1, N, dtype=torch.bool), v.float())
            ok = ok and _close(attn_exact_decode(qd.cuda(), k.cuda(), v.cuda()), want2)
        if not ok:
            failures.append((it, c))
    assert not failures, failures


def test_seeded_random_sweep_of_the_pipelined_window_kernels():
    """The same at the sizes the long-sequence kernels take over: 2k - 6k tokens that are multiples of 64, windows of
    512 - 3000 keys that are multiples of 128, at least 1024 query tiles; the three window modes and causal
    full-context ReRoPE, both dtypes and head dims.  Three (batch, head) units per case against the oracle."""
    rng = random.Random(5)
    bn = lambda x: x.transpose(1, 2).contiguous()
    failures = []
    for it in range(12):
        D = rng.choice([64, 128, 128])
        dtype = rng.choice([torch.bfloat16, torch.float16])
        N = 64 * rng.randint(32, 90)
        W = 128 * rng.randint(4, max(4, min(24, (N - 64) // 128)))
        H, B = rng.choice([32, 40, 64]), rng.choice([1, 2])
        while ((N + 127) // 128) * B * H < 1024:
            H += 8
        mode = rng.choice(["strict", "loose", "rerope", "full"])
        print(f"pipelined sweep {it}: {mode} B{B} H{H} N{N} D{D} W{W} {dtype}", flush=True)
        g = torch.Generator(device="cuda").manual_seed(100 + it)
        q, k, v, q2, k2 = (torch.randn(B, H, N, D, generator=g, device="cuda").to(dtype) for _ in range(5))
        if mode == "strict":
            out = triton_fused_local_attn.flash_attn_func(bn(q), bn(k), bn(v), W).transpose(1, 2)
        elif mode == "loose":
            out = triton_fused_local_attn2.flash_attn_func(bn(q), bn(k), bn(v), W).transpose(1, 2)
        elif mode == "rerope":
            out = triton_fused_local_attn_rerope.flash_attn_func(bn(q), bn(q2), bn(k), bn(k2), bn(v), W).transpose(1, 2)
        else:
            out = triton_fused_attn_rerope.attention(q, q2, k, k2, v, True, 1.0 / math.sqrt(D), W)
        torch.cuda.synchronize()
        for b, h in ((0, 0), (B - 1, H - 1), (0, H // 2)):
            one = lambda x: x[b:b + 1, h:h + 1].cpu()
            if mode == "full":
                want, _ = oracle.rerope_full(one(q), one(q2), one(k), one(k2), one(v), True, 1.0 / math.sqrt(D), W)
            else:
                want, _ = oracle.local_attn(one(q), one(k), one(v), W, mode, None, q2=one(q2), k2=one(k2))
            if not _close(one(out), want):
                failures.append((it, mode, B, H, N, D, W, dtype, b, h))
        del q, k, v, q2, k2, out
        torch.cuda.empty_cache()
    assert not failures, failures
