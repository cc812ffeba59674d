"""Timing of the reference-shaped long-prefill route (single codebook per head, count-weighted far context) and of its
stages, next to the fused per-key formulation, at the prefill benchmark shape.

    python route_bench.py [--heads 32 --tokens 8192 --window 1024 --codes 512]

Prints one JSON object; times are medians of HIP-event intervals in microseconds."""
import argparse
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from vqtree_amd.ops import attn_vq as A  # noqa: E402
from vqtree_amd.ops import mini_vq as Q  # noqa: E402
from vqtree_amd.ops.count_state import CountState  # noqa: E402
from vqtree_amd.ops.triton_fused_vq_attn import vq_attn_forward  # noqa: E402


def _time(fn, steps=20, warmup=10):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for s, e in ev:
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    t = sorted(s.elapsed_time(e) for s, e in ev)
    return round(t[len(t) // 2] * 1e3, 1)


def run(batch=1, heads=32, tokens=8192, head_dim=128, window=1024, codes=512, device="cuda"):
    B, H, N, D, W, C = batch, heads, tokens, head_dim, window, codes
    g = torch.Generator(device=device).manual_seed(1)
    q, k, v = (torch.randn(B, H, N, D, generator=g, device=device).bfloat16() for _ in range(3))
    cb = torch.randn(H, C, D, generator=g, device=device).bfloat16()
    pos = torch.arange(N, device=device).unsqueeze(0).expand(B, -1)
    q1, k1, q2 = A.rerope_operands(q, k, pos, W)
    ids = Q.quantize_ids(k, cb)
    cnt, v_vq, vi = A.segmented_preprocess(ids, v, C, want_int64_counts=True)
    out = {
        "workload": f"long prefill with VQ memory: batch {B}, {H} heads, {N} tokens, head_dim {D}, window {W}, "
                    f"{C} codewords per head, bf16",
        "encode_keys_us": _time(lambda: Q.quantize_ids(k, cb)),
        "preprocess_us": _time(lambda: A.segmented_preprocess(ids, v, C, want_int64_counts=True)),
        "rotary_operands_us": _time(lambda: A.rerope_operands(q, k, pos, W)),
        "vq_attn_forward_us": _time(lambda: vq_attn_forward(q1, q2, k1, cb, cnt, k, v, v_vq, vi, W)),
        "count_state_build_us": _time(lambda: CountState(B, H, C, D, device).add(ids, v)),
        "dispatch_attn_whole_us": _time(lambda: A.dispatch_attn(q, k, v, pos, A.VectorQuantizedReRoPECache(W, cb))),
    }
    cb256 = cb[:, :256].contiguous()
    # the same attention through the fused per-key kernel (needs uint8 codes: at most 256 codewords)
    ids256 = Q.quantize_ids(k, cb256).to(torch.uint8).unsqueeze(-1)
    out["fused_per_key_256_codewords_us"] = _time(
        lambda: A.attn_vq_prefill(q1, ids256, cb256.unsqueeze(1), v, k_exact=k1, window_size=W, q2=q2, k2=k,
                                  schedule="per_key"))
    out["attn_vq_prefill_default_256_codewords_us"] = _time(  # M = 1: dispatched to the codeword-space route
        lambda: A.attn_vq_prefill(q1, ids256, cb256.unsqueeze(1), v, k_exact=k1, window_size=W, q2=q2, k2=k))
    # one generation step after that prefill, on the cache's count state (O(C D) per step): all keys through their
    # codewords, and with the exact window and strip of a prefill row; next to it the same attention streamed over the
    # N one-byte codes and V rows (O(N D) per step; needs <= 256 codewords)
    one = lambda: torch.randn(B, H, 1, D, generator=g, device=device).bfloat16()
    qs, ks, vs = one(), one(), one()
    for name, exact in (("generation_step_all_coded_us", False), ("generation_step_exact_window_us", True)):
        cache = A.VectorQuantizedReRoPECache(W, cb, generation_exact_window=exact)
        A.dispatch_attn(q, k, v, pos, cache)
        step = [N]

        def gen():
            A.dispatch_attn(qs, ks, vs, torch.full((B, 1), step[0], device=device), cache)
            step[0] += 1

        out[name] = _time(gen, steps=20, warmup=3)  # the first call also builds the state
    codes_u8 = Q.quantize_ids(k, cb256).to(torch.uint8).unsqueeze(-1)
    out["generation_step_streaming_256_codewords_us"] = _time(
        lambda: A.attn_vq_decode(qs, codes_u8, cb256.unsqueeze(1), v))
    # the four-codebook prefill benchmark workload under the two schedules of the fused kernel
    from vqtree_amd.synthetic import prefill_c3

    c = prefill_c3()
    for schedule in ("default", "pipelined"):
        out[f"attn_vq_prefill_4x256_{schedule}_us"] = _time(
            lambda: A.attn_vq_prefill(c.q, c.codes, c.codebooks, c.v, k_exact=c.k_exact, window_size=c.window,
                                      softmax_scale=c.softmax_scale, schedule=schedule))
    # full-context ReRoPE attention (`attention`, ops/triton_fused_attn_rerope.py:185-233) at the window benchmark's
    # shape: batch 2, 32 heads, 16384 tokens, window 512 -- O(N^2): 4 D N (N + 1) / 2 per (batch, head) = 4 398 GFLOP
    from vqtree_amd.ops.triton_fused_attn_rerope import attention

    del q, k, v, q1, k1, q2, c
    torch.cuda.empty_cache()
    Bf, Nf, Wf = 2, 16384, 512
    f1, f2, fk1, fk2, fv = (torch.randn(Bf, H, Nf, D, generator=g, device=device).bfloat16() for _ in range(5))
    us = _time(lambda: attention(f1, f2, fk1, fk2, fv, True, 1 / D ** 0.5, Wf), steps=6, warmup=3)
    out["rerope_full_b2_n16384_w512_us"] = us
    out["rerope_full_b2_n16384_w512_tflops"] = round(4 * D * (Nf * (Nf + 1) / 2) * Bf * H / us / 1e6, 1)
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    for name, default in (("batch", 1), ("heads", 32), ("tokens", 8192), ("window", 1024), ("codes", 512)):
        ap.add_argument("--" + name, type=int, default=default)
    print(json.dumps(run(**vars(ap.parse_args()))))
