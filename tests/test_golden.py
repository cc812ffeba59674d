"""The oracle reproduces the committed golden vectors (CPU), and the HIP kernels reproduce them too (GPU)."""
import os

import numpy as np
import pytest
import torch

import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vq_attention_golden.npz")


@pytest.fixture(scope="module")
def gold():
    z = np.load(GOLDEN)  # plain arrays, no pickles
    return {k: torch.from_numpy(z[k]) for k in z.files}


def _close(a, b, tol=2e-6):
    a, b = a.float(), b.float()
    both_inf = torch.isinf(a) & torch.isinf(b) & (a == b)
    return bool(((a - b).abs().masked_fill(both_inf, 0) <= tol + tol * b.abs().masked_fill(both_inf, 0)).all())


def test_oracle_reproduces_golden(gold):
    g = gold
    out, lse = oracle.attn_vq_decode(g["dec_q"], g["dec_codes"], g["dec_cb"], g["dec_v"])
    assert _close(out, g["dec_out"]) and _close(lse, g["dec_lse"], 1e-5)
    out, lse = oracle.attn_vq_prefill(g["pf_q"], g["pf_codes"], g["pf_cb"], g["pf_v"])
    assert _close(out, g["pf_out"]) and _close(lse, g["pf_lse"], 1e-5)
    kw = dict(k_exact=g["pw_k"], window_size=128)
    out, lse = oracle.attn_vq_prefill(g["pw_q"], g["pw_codes"], g["pw_cb"], g["pw_v"], q2=g["pw_q2"], k2=g["pw_k2"], **kw)
    assert _close(out, g["pw_out"]) and _close(lse, g["pw_lse"], 1e-5)
    out, _ = oracle.attn_vq_prefill(g["pw_q"], g["pw_codes"], g["pw_cb"], g["pw_v"], boundary_mode="exact", **kw)
    assert _close(out, g["pw_out_exact"])
    for mode in ("strict", "loose", "rerope"):
        out, lse = oracle.local_attn(g["pw_q"], g["pw_k"], g["pw_v"], 128, mode, None, q2=g["pw_q2"], k2=g["pw_k2"])
        assert _close(out, g[f"win_{mode}_out"]) and _close(lse, g[f"win_{mode}_lse"], 1e-5)
    for causal, key in ((True, "full_causal_out"), (False, "full_noncausal_out")):
        out, _ = oracle.rerope_full(g["pw_q"], g["pw_q2"], g["pw_k"], g["pw_k2"], g["pw_v"], causal, 0.125, 64)
        assert _close(out, g[key])
    _, ids, _ = oracle.multi_head_single_quantize(g["pw_k"], g["cr_cb"])
    assert torch.equal(ids, g["cr_ids"].long())
    cnt, v_vq, vi = oracle.sort_based_preprocess(ids, g["pw_v"], 128, dtype=torch.float16)
    assert torch.equal(cnt, g["cr_cnt"].long()) and torch.equal(vi, g["cr_vi"].long()) and torch.equal(v_vq, g["cr_v_vq"])
    o2, l2 = oracle.vq_count_forward(g["pw_q2"], g["cr_cb"], cnt, v_vq, vi, 128)
    assert _close(o2, g["cr_o2"], 1e-5) and _close(l2, g["cr_l2"], 1e-5)


@pytest.mark.gpu
def test_kernels_reproduce_golden(gold):
    from tests.util import assert_close_16, assert_close_lse
    from vqtree_amd.ops import (triton_fused_attn_rerope, triton_fused_local_attn, triton_fused_local_attn2,
                                triton_fused_local_attn_rerope, triton_fused_vq_attn)
    from vqtree_amd.ops.attn_vq import attn_vq_decode, attn_vq_prefill

    g = {k: (v.cuda() if v.dtype in (torch.float16, torch.uint8) else v) for k, v in gold.items()}
    out, lse = attn_vq_decode(g["dec_q"], g["dec_codes"], g["dec_cb"], g["dec_v"], return_lse=True)
    assert_close_16(out, g["dec_out"], "decode"), assert_close_lse(lse, g["dec_lse"])
    out, lse = attn_vq_prefill(g["pf_q"], g["pf_codes"], g["pf_cb"], g["pf_v"], return_lse=True)
    assert_close_16(out, g["pf_out"], "prefill"), assert_close_lse(lse, g["pf_lse"], atol=1e-2)
    kw = dict(k_exact=g["pw_k"], window_size=128)
    out, lse = attn_vq_prefill(g["pw_q"], g["pw_codes"], g["pw_cb"], g["pw_v"], q2=g["pw_q2"], k2=g["pw_k2"],
                               return_lse=True, **kw)
    assert_close_16(out, g["pw_out"], "prefill window"), assert_close_lse(lse, g["pw_lse"], atol=1e-2)
    out = attn_vq_prefill(g["pw_q"], g["pw_codes"], g["pw_cb"], g["pw_v"], boundary_mode="exact", **kw)
    assert_close_16(out, g["pw_out_exact"], "prefill exact boundary")
    t = lambda x: x.transpose(1, 2).contiguous()
    q, k, v, q2, k2 = (t(g[n]) for n in ("pw_q", "pw_k", "pw_v", "pw_q2", "pw_k2"))
    assert_close_16(t(triton_fused_local_attn.flash_attn_func(q, k, v, 128)), g["win_strict_out"], "strict")
    o, l = triton_fused_local_attn2.flash_attn_func(q, k, v, 128, return_lse=True)
    assert_close_16(t(o), g["win_loose_out"], "loose"), assert_close_lse(l, g["win_loose_lse"])
    o, l = triton_fused_local_attn_rerope.flash_attn_func(q, q2, k, k2, v, 128, return_lse=True)
    assert_close_16(t(o), g["win_rerope_out"], "rerope"), assert_close_lse(l, g["win_rerope_lse"])
    for causal, key in ((True, "full_causal_out"), (False, "full_noncausal_out")):
        o = triton_fused_attn_rerope.attention(g["pw_q"], g["pw_q2"], g["pw_k"], g["pw_k2"], g["pw_v"], causal, 0.125, 64)
        assert_close_16(o, g[key], key)
    cnt, vi = g["cr_cnt"].cuda().to(torch.float16), g["cr_vi"].cuda().long()
    o2, l2 = triton_fused_vq_attn.vq_count_forward(g["pw_q2"], g["cr_cb"], cnt, g["cr_v_vq"], vi, 128)
    assert_close_16(o2, g["cr_o2"], "count kernel"), assert_close_lse(l2, g["cr_l2"], atol=5e-3)
    o = triton_fused_vq_attn.vq_attn_forward(g["pw_q"], g["pw_q2"], g["pw_k"], g["cr_cb"], cnt, g["pw_k2"], g["pw_v"],
                                             g["cr_v_vq"], vi, 128)
    assert_close_16(o, g["cr_out"], "count route")
