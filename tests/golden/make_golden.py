"""Writes tests/golden/vq_attention_golden.npz: small seeded inputs (fp16-representable) and the outputs of the CPU
oracle for every entry point of the VQ-attention path.  The reference stores no vectors and cannot be imported in this
environment, so these fixtures freeze the (independently pinned) oracle: tests/test_golden.py checks that the oracle
still reproduces them, and the GPU tests run the kernels on the same inputs.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vq_attention_golden.npz")


def h(t):  # fp16 inputs, stored as fp16
    return t.to(torch.float16)


def main():
    g = torch.Generator("cpu").manual_seed(20240607)
    rn = lambda *s, std=1.0: h(torch.randn(*s, generator=g) * std)
    ri = lambda hi, *s: torch.randint(0, hi, s, generator=g, dtype=torch.int32).to(torch.uint8)
    z = {}

    # decode
    q, v, cb, codes = rn(1, 2, 1, 64), rn(1, 2, 257, 64), rn(2, 4, 256, 64, std=0.35), ri(256, 1, 2, 257, 4)
    out, lse = oracle.attn_vq_decode(q, codes, cb, v)
    z.update(dec_q=q, dec_v=v, dec_cb=cb, dec_codes=codes, dec_out=out, dec_lse=lse)

    # prefill, every key quantised, causal
    q, v, cb, codes = rn(1, 1, 257, 64), rn(1, 1, 257, 64), rn(1, 2, 256, 64, std=0.5), ri(256, 1, 1, 257, 2)
    out, lse = oracle.attn_vq_prefill(q, codes, cb, v)
    z.update(pf_q=q, pf_v=v, pf_cb=cb, pf_codes=codes, pf_out=out, pf_lse=lse)

    # prefill with exact window (block boundary) and the ReRoPE strip
    N, W = 384, 128
    q, k, v, q2, k2 = (rn(1, 1, N, 64) for _ in range(5))
    cb, codes = rn(1, 2, 256, 64, std=0.35), ri(256, 1, 1, N, 2)
    out, lse = oracle.attn_vq_prefill(q, codes, cb, v, k_exact=k, window_size=W, q2=q2, k2=k2)
    out_exact, _ = oracle.attn_vq_prefill(q, codes, cb, v, k_exact=k, window_size=W, boundary_mode="exact")
    z.update(pw_q=q, pw_k=k, pw_v=v, pw_q2=q2, pw_k2=k2, pw_cb=cb, pw_codes=codes, pw_out=out, pw_lse=lse,
             pw_out_exact=out_exact)

    # the three sliding windows and full ReRoPE share inputs
    for mode in ("strict", "loose", "rerope"):
        out, lse = oracle.local_attn(q, k, v, W, mode, None, q2=q2, k2=k2)
        z[f"win_{mode}_out"], z[f"win_{mode}_lse"] = out, lse
    z["full_causal_out"], _ = oracle.rerope_full(q, q2, k, k2, v, True, 0.125, 64)
    z["full_noncausal_out"], _ = oracle.rerope_full(q, q2, k, k2, v, False, 0.125, 64)

    # reference-shaped single-codebook route
    C = 128
    cb1 = rn(1, C, 64)
    k_hat, ids, _ = oracle.multi_head_single_quantize(k, cb1)
    cnt, v_vq, vi = oracle.sort_based_preprocess(ids, v, C, dtype=torch.float16)
    o2, l2 = oracle.vq_count_forward(q2, cb1, cnt, v_vq, vi, W)
    route = oracle.vq_attn_forward(q, q2, k, cb1, cnt, k2, v, v_vq, vi, W)
    z.update(cr_cb=cb1, cr_ids=ids.to(torch.int16), cr_cnt=cnt.to(torch.int32), cr_vi=vi.to(torch.int32), cr_v_vq=v_vq,
             cr_o2=o2, cr_l2=l2, cr_out=route)

    np.savez_compressed(OUT, **{k_: (t.numpy() if torch.is_tensor(t) else t) for k_, t in z.items()})
    print("wrote", OUT, os.path.getsize(OUT) // 1024, "KiB,", len(z), "arrays")


if __name__ == "__main__":
    main()
