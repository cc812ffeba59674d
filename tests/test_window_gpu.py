"""GPU parity of the sliding-window / ReRoPE / VQ-prefill MFMA kernels against the CPU oracle."""
import math

import pytest
import torch

import oracle
from tests.util import assert_close_16, assert_close_lse
from vqtree_amd.ops import (triton_fused_attn_rerope, triton_fused_local_attn, triton_fused_local_attn2,
                            triton_fused_local_attn_rerope, triton_fused_vq_attn)
from vqtree_amd.ops.attn_vq import attn_vq_prefill

pytestmark = pytest.mark.gpu


def _randn(*shape, seed, std=1.0, dtype=torch.bfloat16):
    g = torch.Generator("cpu").manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def _bnhd(x):  # [B,H,N,D] -> contiguous [B,N,H,D]
    return x.transpose(1, 2).contiguous()


def _say(msg):
    print(msg, flush=True)


# ------------------------------------------------------------------ strict / loose / rerope-local windows
@pytest.mark.parametrize("N", [2048, 2013])
@pytest.mark.parametrize("mode", ["strict", "loose", "rerope"])
def test_reference_selfcheck_shapes(mode, N):
    """The shapes of the reference's own self-checks: Z=1, H=2, D=64, W=512, sm_scale 0.5, fp16 N(0, 0.5), even and
    uneven lengths (ops/triton_fused_local_attn.py:265-294, ops/triton_fused_local_attn2.py:277-335)."""
    _say(f"window selfcheck {mode} N={N}")
    B, H, D, W, scale = 1, 2, 64, 512, 0.5
    q, k, v, q2, k2 = (_randn(B, H, N, D, seed=s, std=0.5, dtype=torch.float16) for s in range(5))
    want, want_lse = oracle.local_attn(q, k, v, W, mode, scale, q2=q2, k2=k2)
    qd, kd, vd, q2d, k2d = (_bnhd(x).cuda() for x in (q, k, v, q2, k2))
    if mode == "strict":
        out, lse = triton_fused_local_attn.flash_attn_func(qd, kd, vd, W, scale), None
    elif mode == "loose":
        out, lse = triton_fused_local_attn2.flash_attn_func(qd, kd, vd, W, scale, return_lse=True)
    else:
        out, lse = triton_fused_local_attn_rerope.flash_attn_func(qd, q2d, kd, k2d, vd, W, scale, return_lse=True)
    torch.cuda.synchronize()
    assert out.shape == (B, N, H, D) and out.is_contiguous()
    got = out.transpose(1, 2).float().cpu()
    assert (got - want).abs().max() <= 2e-2  # the reference's acceptance: atol 2e-2, rtol 0
    assert_close_16(got, want, mode)
    if lse is not None:
        assert_close_lse(lse, want_lse)


@pytest.mark.parametrize("mode", ["strict", "loose", "rerope"])
@pytest.mark.parametrize("B,H,N,D,W", [(2, 3, 384, 128, 128), (1, 2, 130, 128, 128), (1, 2, 257, 64, 128),
                                        (1, 1, 511, 128, 256), (2, 2, 1000, 128, 384), (1, 2, 64, 64, 128),
                                        (1, 2, 700, 128, 1024), (1, 1, 1, 128, 128), (2, 2, 777, 32, 128),
                                        (1, 3, 300, 32, 256), (1, 2, 500, 16, 128)])
def test_window_modes(mode, B, H, N, D, W):
    _say(f"window {mode} B{B} H{H} N{N} D{D} W{W}")
    q, k, v, q2, k2 = (_randn(B, H, N, D, seed=10 + s) for s in range(5))
    want, want_lse = oracle.local_attn(q, k, v, W, mode, None, q2=q2, k2=k2)
    qd, kd, vd, q2d, k2d = (_bnhd(x).cuda() for x in (q, k, v, q2, k2))
    if mode == "strict":
        out, lse = triton_fused_local_attn.flash_attn_func(qd, kd, vd, W), None
    elif mode == "loose":
        out, lse = triton_fused_local_attn2.flash_attn_func(qd, kd, vd, W, return_lse=True)
    else:
        out, lse = triton_fused_local_attn_rerope.flash_attn_func(qd, q2d, kd, k2d, vd, W, return_lse=True)
    torch.cuda.synchronize()
    assert_close_16(out.transpose(1, 2), want, mode)
    if lse is not None:
        assert_close_lse(lse, want_lse)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mode", ["strict", "loose", "rerope"])
@pytest.mark.parametrize("N,D,W", [(4096, 128, 1024), (4032, 128, 1152), (4096, 64, 2048), (4096, 128, 512),
                                   (4000, 128, 1152)])
def test_window_modes_on_the_pipelined_core(mode, N, D, W, dtype):
    """64 (batch, head) units x ~4000 tokens with a window of >= 512 keys that is a multiple of 128 and a length that
    is a multiple of 64: here vqa_local_attn_* runs the sliding-window kinds of the pipelined core (128-row workgroups
    that walk several query tiles each; for ReRoPE the second pair through a change of the query operand at each
    wave's window-edge tile).  N = 4000 is the same call on the general kernel (length not a multiple of 64).  Three
    units against the oracle."""
    _say(f"window on the pipelined core {mode} N{N} D{D} W{W} {dtype}")
    B, H = 2, 32
    g = torch.Generator(device="cuda").manual_seed(53)
    q, k, v, q2, k2 = (torch.randn(B, N, H, D, generator=g, device="cuda").to(dtype) for _ in range(5))
    if mode == "strict":
        out, lse = triton_fused_local_attn.flash_attn_func(q, k, v, W), None
    elif mode == "loose":
        out, lse = triton_fused_local_attn2.flash_attn_func(q, k, v, W, return_lse=True)
    else:
        out, lse = triton_fused_local_attn_rerope.flash_attn_func(q, q2, k, k2, v, W, return_lse=True)
    torch.cuda.synchronize()
    for b, h in ((0, 0), (1, 17), (1, 31)):
        one = lambda x: x[b:b + 1, :, h:h + 1].transpose(1, 2).cpu()
        want, want_lse = oracle.local_attn(one(q), one(k), one(v), W, mode, None, q2=one(q2), k2=one(k2))
        assert_close_16(one(out), want, f"{mode} unit ({b},{h})")
        if lse is not None:
            # the query operand is scaled by softmax_scale * log2(e) before the products: one more 16-bit rounding
            assert_close_lse(lse[b:b + 1, h:h + 1], want_lse, atol=1e-2 if dtype == torch.bfloat16 else 2e-3)


def test_full_window_causal_attention_at_a_large_shape():
    """A window that covers the sequence is plain causal attention; at 64 heads x 4096 tokens the library runs it on
    the pipelined schedule.  Strict and loose windows are then the same function: checked against each other, against
    a window one short of the sequence (tiled kernel, the first row pair differs by nothing: i - j <= N - 1 always
    holds) and, on two heads, against the oracle."""
    _say("full-window causal H64 N4096")
    B, H, N, D = 1, 64, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(41)
    q, k, v = (torch.randn(B, N, H, D, generator=g, device="cuda").to(torch.bfloat16) for _ in range(3))
    strict = triton_fused_local_attn.flash_attn_func(q, k, v, N)
    loose, lse = triton_fused_local_attn2.flash_attn_func(q, k, v, N, return_lse=True)
    tiled = triton_fused_local_attn.flash_attn_func(q, k, v, N - 1)  # window < N: the tiled kernel, same visible set
    torch.cuda.synchronize()
    assert torch.equal(strict, loose)
    assert (strict.float() - tiled.float()).abs().max() <= 2e-2
    hs = [3, 60]
    bhnd = lambda x: x[:, :, hs].transpose(1, 2).cpu()
    want, want_lse = oracle.local_attn(bhnd(q), bhnd(k), bhnd(v), N, "strict", None)
    assert_close_16(strict[:, :, hs].transpose(1, 2), want, "full-window causal")
    assert_close_lse(lse[:, hs], want_lse, atol=1e-2)


def test_loose_matches_dense_ref_impl_on_device():
    q, k, v = (_bnhd(_randn(1, 2, 640, 64, seed=20 + s, std=0.5, dtype=torch.float16)).cuda() for s in range(3))
    out = triton_fused_local_attn2.flash_attn_func(q, k, v, 256, 0.5)
    ref = triton_fused_local_attn2.local_attn2_ref_impl(q, k, v, 256, 0.5)
    assert torch.allclose(out.float(), ref.float(), atol=2e-2, rtol=0)


def test_window_mask_is_exact():
    """Bit-exact mask check: V rows are one-hot position markers and all scores are equal, so each output row is
    (indicator of the visible key set) / (its size) -- any wrongly visible or hidden key changes an element."""
    N, D, W = 384, 128, 128
    v = torch.zeros(1, 1, N, D, dtype=torch.bfloat16)
    v[0, 0, torch.arange(N), torch.arange(N) % D] = 1.0
    z = torch.zeros(1, 1, N, D, dtype=torch.bfloat16)
    for mode in ("strict", "loose", "rerope"):
        vis, _ = oracle.local_visible_mask(N, W, mode)
        zd, vd = _bnhd(z).cuda(), _bnhd(v).cuda()
        if mode == "strict":
            out = triton_fused_local_attn.flash_attn_func(zd, zd, vd, W)
        elif mode == "loose":
            out = triton_fused_local_attn2.flash_attn_func(zd, zd, vd, W)
        else:
            out = triton_fused_local_attn_rerope.flash_attn_func(zd, zd, zd, zd, vd, W)
        got = out[0, :, 0].float().cpu()  # [N, D]
        cnt = vis.sum(1, keepdim=True).float()
        want = torch.zeros(N, D)
        for c in range(D):
            want[:, c] = vis[:, c::D].sum(1)
        want = want / cnt
        # a wrongly visible / hidden key changes its element by 100% (from or to zero); bf16 rounding by 0.4%
        assert torch.allclose(got, want, atol=1e-5, rtol=5e-3), mode


# ------------------------------------------------------------------ full ReRoPE
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("N,D,W", [(2048, 64, 512), (700, 128, 128), (300, 128, 512), (130, 64, 64), (1100, 32, 256),
                                   (257, 32, 64), (600, 16, 128)])
def test_rerope_full(causal, N, D, W):
    """Includes the reference self-check shape Z=1,H=16->2,N=2048,D=64,W=512 fp16 sm_scale 0.5
    (ops/triton_fused_attn_rerope.py:253-268; it checks the non-causal call)."""
    _say(f"rerope_full causal={causal} N{N} D{D} W{W}")
    B, H = 1, 2
    q1, q2, k1, k2, v = (_randn(B, H, N, D, seed=30 + s, std=0.5, dtype=torch.float16) for s in range(5))
    want, _ = oracle.rerope_full(q1, q2, k1, k2, v, causal, 0.5, W)
    out = triton_fused_attn_rerope.attention(q1.cuda(), q2.cuda(), k1.cuda(), k2.cuda(), v.cuda(), causal, 0.5, W)
    torch.cuda.synchronize()
    assert out.shape == q1.shape
    assert (out.float().cpu() - want).abs().max() <= 2e-2
    assert_close_16(out, want, "rerope_full")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D,W", [(1, 2, 2304, 128, 512), (2, 1, 2100, 128, 64), (1, 2, 3000, 64, 1024),
                                        (1, 1, 2049, 128, 2048), (1, 8, 2176, 128, 192)])
def test_causal_rerope_full_on_the_pipelined_core(B, H, N, D, W, dtype):
    """Causal full-context ReRoPE of 2048 tokens or more with a window that is a multiple of 64 runs on the 256-row
    pipelined kernel (second-pair tiles with the second query, a change-over with a second product at each wave's
    edge tile, first-pair tiles up to the diagonal); ragged lengths and a window that reaches back to key 0 for most
    rows included.  The non-causal call of the same shape stays on the general kernel; both against the oracle."""
    _say(f"causal rerope_full on the pipelined core B{B} H{H} N{N} D{D} W{W} {dtype}")
    q1, q2, k1, k2, v = (_randn(B, H, N, D, seed=130 + s, dtype=dtype) for s in range(5))
    for causal in (True, False):
        scale = 1.0 / math.sqrt(D)
        want, _ = oracle.rerope_full(q1, q2, k1, k2, v, causal, scale, W)
        out = triton_fused_attn_rerope.attention(q1.cuda(), q2.cuda(), k1.cuda(), k2.cuda(), v.cuda(), causal, scale, W)
        torch.cuda.synchronize()
        assert_close_16(out, want, f"rerope_full causal={causal}")


# ------------------------------------------------------------------ VQ prefill (additive codes)
def _codes(B, H, N, M, K=256, seed=0):
    g = torch.Generator("cpu").manual_seed(seed)
    return torch.randint(0, K, (B, H, N, M), generator=g, dtype=torch.int32).to(torch.uint8)


@pytest.mark.parametrize("B,H,N,D,M,K", [(1, 2, 1024, 64, 2, 256), (2, 2, 300, 128, 4, 256), (1, 1, 130, 128, 1, 64),
                                          (1, 2, 777, 64, 8, 256), (1, 1, 64, 128, 4, 256)])
@pytest.mark.parametrize("causal", [True, False])
def test_vq_prefill_all_quantised(B, H, N, D, M, K, causal):
    _say(f"vq prefill far-only B{B} H{H} N{N} D{D} M{M} K{K} causal={causal}")
    q, v = _randn(B, H, N, D, seed=40), _randn(B, H, N, D, seed=41)
    cb = _randn(H, M, K, D, seed=42, std=0.5 / math.sqrt(M))
    codes = _codes(B, H, N, M, K, seed=43)
    want, want_lse = oracle.attn_vq_prefill(q, codes, cb, v, causal=causal)
    out, lse = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), causal=causal, return_lse=True)
    torch.cuda.synchronize()
    assert_close_16(out, want, "vq prefill")
    assert_close_lse(lse, want_lse, atol=1e-2)  # far keys are rounded once to 16 bits before the dot product


@pytest.mark.parametrize("boundary_mode", ["block", "exact"])
@pytest.mark.parametrize("with_rerope", [False, True])
@pytest.mark.parametrize("B,H,N,D,M,W", [(1, 2, 1024, 128, 4, 256), (2, 2, 640, 64, 2, 128), (1, 2, 515, 128, 4, 128),
                                          (1, 1, 300, 128, 4, 384), (1, 2, 900, 128, 1, 200)])
def test_vq_prefill_with_exact_window(B, H, N, D, M, W, with_rerope, boundary_mode):
    _say(f"vq prefill window B{B} H{H} N{N} D{D} M{M} W{W} rerope={with_rerope} {boundary_mode}")
    q, k, v, q2, k2 = (_randn(B, H, N, D, seed=50 + s) for s in range(5))
    cb = _randn(H, M, 256, D, seed=55, std=0.35)
    codes = _codes(B, H, N, M, seed=56)
    kw = dict(k_exact=k, window_size=W, boundary_mode=boundary_mode)
    if with_rerope:
        kw.update(q2=q2, k2=k2)
    want, want_lse = oracle.attn_vq_prefill(q, codes, cb, v, **kw)
    kw = {n: (t.cuda() if torch.is_tensor(t) else t) for n, t in kw.items()}
    out, lse = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), return_lse=True, **kw)
    torch.cuda.synchronize()
    assert_close_16(out, want, "vq prefill window")
    assert_close_lse(lse, want_lse, atol=1e-2)


@pytest.mark.parametrize("with_rerope", [False, True])
def test_vq_prefill_fp16(with_rerope):
    """The fp16 instantiation of the fused prefill (two-pair and three-pair kernels), strided [B,N,H,D]-backed q/k/v."""
    _say(f"vq prefill fp16 rerope={with_rerope}")
    B, H, N, D, M, W = 2, 2, 700, 128, 4, 256
    mk = lambda seed: _bnhd(_randn(B, H, N, D, seed=seed, std=0.7, dtype=torch.float16)).transpose(1, 2)
    q, k, v, q2, k2 = (mk(70 + s) for s in range(5))
    cb = _randn(H, M, 256, D, seed=75, std=0.3, dtype=torch.float16)
    codes = _codes(B, H, N, M, seed=76)
    kw = dict(k_exact=k, window_size=W)
    if with_rerope:
        kw.update(q2=q2, k2=k2)
    want, want_lse = oracle.attn_vq_prefill(q, codes, cb, v, **kw)
    kw = {n: (t.cuda() if torch.is_tensor(t) else t) for n, t in kw.items()}
    out, lse = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), return_lse=True, **kw)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    assert_close_16(out, want, "vq prefill fp16")
    assert_close_lse(lse, want_lse, atol=1e-2)


def test_vq_prefill_far_boundary_is_exact():
    """Mask/source check with little rounding slack: far keys score 1 (weight e), exact keys score 0 (weight 1), V rows
    are position markers; a key taken from the wrong side moves its output element by ~1e-3, rounding by ~1e-5."""
    N, D, W = 640, 128, 128
    q = torch.zeros(1, 1, N, D, dtype=torch.bfloat16)
    q[..., 0] = 1.0
    cb = torch.zeros(1, 1, 256, D, dtype=torch.bfloat16)
    cb[0, 0, :, 0] = 1.0
    codes = torch.zeros(1, 1, N, 1, dtype=torch.uint8)
    k = torch.zeros(1, 1, N, D, dtype=torch.bfloat16)
    v = torch.zeros(1, 1, N, D, dtype=torch.bfloat16)
    v[0, 0, torch.arange(N), torch.arange(N) % D] = 1.0
    for bm in ("block", "exact"):
        want, _ = oracle.attn_vq_prefill(q, codes, cb, v, k_exact=k, window_size=W, boundary_mode=bm, softmax_scale=1.0)
        out = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), k_exact=k.cuda(), window_size=W,
                              boundary_mode=bm, softmax_scale=1.0)
        assert torch.allclose(out.float().cpu(), want, atol=1e-4, rtol=1e-2), bm


# ------------------------------------------------------------------ reference-shaped single-codebook route
def _count_route_case(N, W, C, D, H=2, B=1, dtype=torch.float16, seed=60):
    q, k, v = (_randn(B, H, N, D, seed=seed + s, dtype=dtype) for s in range(3))
    cb = _randn(H, C, D, seed=seed + 3, dtype=dtype)
    cos, sin = oracle.rope_tables(D, N + W + 2)
    pos = torch.arange(N)
    q1, k1 = oracle.apply_rope(q, cos, sin, pos), oracle.apply_rope(k, cos, sin, pos)
    q2 = oracle.apply_rope(q, cos, sin, W + 1)
    k_hat, ids, _ = oracle.multi_head_single_quantize(k, cb)
    cnt, v_vq, vi = oracle.sort_based_preprocess(ids, v, C, dtype=dtype)
    return q1, q2, k1, k, k_hat, ids, cb, v, cnt.to(dtype), v_vq, vi


@pytest.mark.parametrize("N,W,C,D", [(511, 256, 128, 64), (1024, 256, 256, 128), (900, 128, 512, 128),
                                     (1000, 128, 256, 32), (700, 128, 128, 16)])
def test_vq_attn_forward_reference_route(N, W, C, D):
    """vq_attn_forward on inputs built by the sort-based preprocessing, against the naive per-key oracle (includes
    the reference's own check shape: LEN=511, W=256, fp16, 2 heads of dim 64, ops/attn_vq.py:534-556)."""
    _say(f"vq_attn_forward N{N} W{W} C{C} D{D}")
    q1, q2, k1, k, k_hat, ids, cb, v, cnt, v_vq, vi = _count_route_case(N, W, C, D)
    want, _ = oracle.attn_vq_prefill(q1, ids[..., None], cb[:, None], v, k_exact=k1, window_size=W, q2=q2, k2=k)
    dev = [t.cuda() for t in (q1, q2, k1, cb, cnt, k, v, v_vq, vi)]
    out = triton_fused_vq_attn.vq_attn_forward(*dev, W)
    torch.cuda.synchronize()
    assert out.shape == q1.shape
    # oracle of the same route (count kernel on the same 16-bit prefix sums) bounds the kernel error tightly ...
    route = oracle.vq_attn_forward(q1, q2, k1, cb, cnt, k, v, v_vq, vi, W)
    assert_close_16(out, route, "count route")
    # ... and the per-key definition within the reference's own acceptance
    assert_close_16(out, want, "count route vs per-key")


def test_count_route_with_exact_integer_counts():
    """Counts above 256 are not representable in bf16 (the reference casts them to the model dtype,
    ops/attn_vq.py:431); with int64 counts -- what the preprocessing builds -- the count route stays on the per-key
    definition.  1792 keys on 4 used codewords: up to ~450 keys per codeword."""
    _say("count route, integer counts")
    N, W, C, D, H, B = 1792, 128, 128, 128, 2, 1
    dtype = torch.bfloat16
    q, k, v = (_randn(B, H, N, D, seed=70 + s, dtype=dtype) for s in range(3))
    cb = _randn(H, C, D, seed=73, dtype=dtype)
    cos, sin = oracle.rope_tables(D, N + W + 2)
    pos = torch.arange(N)
    q1, k1, q2 = oracle.apply_rope(q, cos, sin, pos), oracle.apply_rope(k, cos, sin, pos), oracle.apply_rope(q, cos, sin, W + 1)
    ids = torch.randint(0, 4, (B, H, N), generator=torch.Generator("cpu").manual_seed(74))
    cnt, v_vq, vi = oracle.sort_based_preprocess(ids, v, C, dtype=dtype)
    assert cnt.dtype == torch.int64 and int(cnt.max()) > 256
    assert not torch.equal(cnt.to(dtype).to(torch.int64), cnt)  # the cast to bf16 does round these counts
    want, _ = oracle.attn_vq_prefill(q1, ids[..., None], cb[:, None], v, k_exact=k1, window_size=W, q2=q2, k2=k)
    dev = lambda *ts: [t.cuda() for t in ts]
    out = triton_fused_vq_attn.vq_attn_forward(*dev(q1, q2, k1, cb, cnt, k, v, v_vq, vi), W)
    route = oracle.vq_attn_forward(q1, q2, k1, cb, cnt, k, v, v_vq, vi, W)
    assert_close_16(out, route, "count route, int64 counts")
    assert_close_16(out, want, "count route, int64 counts, vs per-key")
    o2, l2 = triton_fused_vq_attn.vq_count_forward(*dev(q2, cb, cnt, v_vq, vi), W)
    want_o, want_l = oracle.vq_count_forward(q2, cb, cnt, v_vq, vi, W)
    assert_close_16(o2, want_o, "count kernel, int64 counts")
    assert_close_lse(l2, want_l, atol=5e-3)
    # the log-sum-exp is where rounded counts show: with bf16 counts it is off by up to log2(1 + 2^-8)
    _, l2_rounded = triton_fused_vq_attn.vq_count_forward(*dev(q2, cb, cnt.to(dtype), v_vq, vi), W)
    far = slice(W + 128, N)
    assert (l2[:, :, far].cpu() - want_l[:, :, far]).abs().max() < (l2_rounded[:, :, far].cpu() - want_l[:, :, far]).abs().max()


def test_count_kernel_and_merge_separately():
    N, W, C, D = 700, 128, 256, 128
    q1, q2, k1, k, k_hat, ids, cb, v, cnt, v_vq, vi = _count_route_case(N, W, C, D, B=2, dtype=torch.bfloat16)
    want_o, want_l = oracle.vq_count_forward(q2, cb, cnt, v_vq, vi, W)
    o2, l2 = triton_fused_vq_attn.vq_count_forward(q2.cuda(), cb.cuda(), cnt.cuda(), v_vq.cuda(), vi.cuda(), W)
    torch.cuda.synchronize()
    assert_close_16(o2, want_o, "count kernel")
    assert_close_lse(l2, want_l, atol=5e-3)
    assert torch.isinf(l2[:, :, : W + 128]).all() and (o2[:, :, : W + 128] == 0).all()
    # merge in flashinfer's [N, B*H, D] layout against the oracle merge
    o1, l1 = oracle.local_attn(q1, k1, v, W, "rerope", None, q2=q2, k2=k)
    B, H = q1.shape[:2]
    a = o1.to(torch.bfloat16).reshape(B * H, N, D).transpose(0, 1).contiguous().cuda()
    sa = l1.reshape(B * H, N).transpose(0, 1).contiguous().cuda()
    b = o2.reshape(B * H, N, D).transpose(0, 1).contiguous()
    sb = l2.reshape(B * H, N).transpose(0, 1).contiguous()
    want_m, want_s = oracle.merge_state(a, sa, b, sb)
    triton_fused_vq_attn.merge_state_in_place(a, sa, b, sb)
    torch.cuda.synchronize()
    assert_close_16(a, want_m, "merge")
    assert_close_lse(sa, want_s)


# ------------------------------------------------------------------ fp32 validation instantiation
@pytest.mark.parametrize("B,H,N,D,M,K,causal", [(1, 8, 1024, 64, 2, 256, True), (2, 2, 333, 128, 4, 256, True),
                                                 (1, 2, 1500, 64, 1, 100, False), (1, 1, 70, 128, 8, 256, True)])
def test_vq_prefill_fp32_config1(B, H, N, D, M, K, causal):
    """Validation configuration 1 (batch 1, 8 heads, 1024 tokens, head_dim 64, fp32, 2 x 256 codebooks ~N(0, 0.5)) and
    variations, against the naive softmax(Q K_hat^T / sqrt(d)) V to 1e-4."""
    _say(f"vq prefill fp32 B{B} H{H} N{N} D{D} M{M} K{K} causal={causal}")
    g = torch.Generator("cpu").manual_seed(1)
    q, v = torch.randn(B, H, N, D, generator=g), torch.randn(B, H, N, D, generator=g)
    cb = torch.randn(H, M, K, D, generator=g) * 0.5
    codes = torch.randint(0, K, (B, H, N, M), generator=g, dtype=torch.int32).to(torch.uint8)
    want, want_lse = oracle.attn_vq_prefill(q, codes, cb, v, causal=causal)
    out, lse = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), causal=causal, return_lse=True)
    torch.cuda.synchronize()
    assert out.dtype == torch.float32
    assert (out.cpu() - want).abs().max() <= 1e-4
    assert (lse.cpu() - want_lse).abs().max() <= 1e-4


# ------------------------------------------------------------------ reconstructed keys, bit for bit
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,D", [(1, 256, 128), (2, 256, 64), (4, 256, 128), (8, 256, 128), (4, 200, 64),
                                   (16, 96, 128)])
def test_reconstructed_keys_are_bit_exact(M, K, D, dtype):
    """The code gathers of the prefill: the workspace of vqa_prefill_* holds K_hat = sum_m codebooks[h,m,code_m]
    (fp32 sum in codebook order, rounded once) for every key some query scores as a far key: all of them without exact
    keys, those below the last row's far boundary (rounded up to a block of 128) with a window.  Called through ctypes
    with a workspace of the test's own and compared with the oracle's reconstruction by torch.equal."""
    from vqtree_amd import _lib
    from vqtree_amd.synthetic import prefill_case

    _say(f"reconstructed keys M{M} K{K} D{D} {dtype}")
    B, H, N = 2, 3, 333
    case = prefill_case(B, H, N, D, M, 128, K=K, dtype=dtype, seed=40 + M)
    lib = _lib.load()
    sfx = {torch.bfloat16: "bf16", torch.float16: "f16"}[dtype]
    ws_bytes = lib.vqa_prefill_workspace_bytes(B, H, N, D)
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device="cuda")
    out = torch.empty_like(case.q)
    s3 = lambda t: (t.stride(0), t.stride(1), t.stride(2))
    cb = case.codebooks
    strides = _lib.strides_array(*s3(case.q), case.codes.stride(0), case.codes.stride(1), cb.stride(0), cb.stride(1),
                                 cb.stride(2), *s3(case.v), *s3(case.k_exact), 0, 0, 0, 0, 0, 0, *s3(out))
    want = oracle.reconstruct_keys(case.codes, cb).to(dtype)
    far_keys = ((N - 1 - 128) // 128 * 128 + 127) // 128 * 128  # below the far boundary of row N - 1, in blocks of 128
    for k_exact, n_hat in ((case.k_exact, far_keys), (None, N)):
        ws.zero_()
        rc = getattr(lib, "vqa_prefill_" + sfx)(case.q.data_ptr(), case.codes.data_ptr(), cb.data_ptr(),
                                                case.v.data_ptr(), k_exact.data_ptr() if k_exact is not None else None,
                                                None, None, out.data_ptr(), None, ws.data_ptr(), ws_bytes, B, H, N, D, M,
                                                K, strides, 128, 0, 1, case.softmax_scale,
                                                _lib.current_stream(case.q.device))
        _lib.check(rc)
        torch.cuda.synchronize()
        k_hat = ws[: B * H * N * D * 2].view(dtype).view(B, H, N, D).cpu()
        assert torch.equal(k_hat[:, :, :n_hat], want[:, :, :n_hat])
        assert not k_hat[:, :, n_hat:].any()  # keys no query scores as far keys are not reconstructed
        want_out, _ = oracle.attn_vq_prefill(case.q, case.codes, cb, case.v, k_exact=k_exact, window_size=128)
        assert_close_16(out, want_out, "prefill around the reconstruction")


# ------------------------------------------------------------------ software-pipelined schedule of the long prefill
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D,M,W", [(1, 2, 1024, 128, 4, 256), (2, 2, 640, 64, 2, 128), (1, 2, 515, 128, 4, 128),
                                          (1, 1, 300, 128, 4, 384), (1, 2, 777, 64, 8, 0), (2, 1, 1300, 128, 1, 1024),
                                          (1, 3, 65, 128, 2, 128), (1, 1, 1, 128, 4, 128)])
def test_vq_prefill_pipelined_schedule(B, H, N, D, M, W, dtype):
    """vqa_prefill_pipelined_*: block boundary with a window that is a multiple of 128, or (W = 0 here) every key
    quantised; against the oracle and against the default kernel."""
    _say(f"vq prefill pipelined B{B} H{H} N{N} D{D} M{M} W{W} {dtype}")
    q, k, v = (_randn(B, H, N, D, seed=90 + s, dtype=dtype) for s in range(3))
    cb = _randn(H, M, 256, D, seed=95, std=0.35, dtype=dtype)
    codes = _codes(B, H, N, M, seed=96)
    kw = dict(k_exact=k, window_size=W) if W else {}
    want, want_lse = oracle.attn_vq_prefill(q, codes, cb, v, **kw)
    kw = {n: (t.cuda() if torch.is_tensor(t) else t) for n, t in kw.items()}
    out, lse = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), return_lse=True, schedule="pipelined", **kw)
    ref, _ = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), return_lse=True, **kw)
    torch.cuda.synchronize()
    assert_close_16(out, want, "pipelined vq prefill")
    assert_close_lse(lse, want_lse, atol=1e-2)
    assert (out.float() - ref.float()).abs().max() <= 2e-2


def test_vq_prefill_schedule_choice_at_a_large_shape():
    """64 heads x 4096 tokens: vqa_prefill_* takes the pipelined schedule from 2048 tokens on.  The default call must
    be bit-identical to the forced pipelined one, within tolerance of the forced tiled one, and two heads are checked
    against the oracle (heads are independent)."""
    _say("vq prefill schedule choice H64 N4096")
    B, H, N, D, M, W = 1, 64, 4096, 128, 4, 1024
    g = torch.Generator(device="cuda").manual_seed(97)
    q, k, v = (torch.randn(B, H, N, D, generator=g, device="cuda").to(torch.bfloat16) for _ in range(3))
    cb = (torch.randn(H, M, 256, D, generator=g, device="cuda") * 0.35).to(torch.bfloat16)
    codes = torch.randint(0, 256, (B, H, N, M), generator=g, device="cuda", dtype=torch.uint8)
    run = lambda schedule: attn_vq_prefill(q, codes, cb, v, k_exact=k, window_size=W, return_lse=True, schedule=schedule)
    (auto, auto_l), (tiled, tiled_l), (piped, piped_l) = run("default"), run("tiled"), run("pipelined")
    torch.cuda.synchronize()
    assert torch.equal(auto, piped) and torch.equal(auto_l, piped_l)
    assert not torch.equal(auto, tiled)  # two kernels, two summation orders
    assert (auto.float() - tiled.float()).abs().max() <= 2e-2
    hs = [0, 37]
    want, want_l = oracle.attn_vq_prefill(q[:, hs].cpu(), codes[:, hs].cpu(), cb[hs].cpu(), v[:, hs].cpu(),
                                          k_exact=k[:, hs].cpu(), window_size=W)
    assert_close_16(auto[:, hs], want, "auto schedule")
    assert_close_16(tiled[:, hs], want, "tiled schedule")
    assert_close_lse(auto_l[:, hs], want_l, atol=1e-2)
    # a short sequence of the same kind stays on the tiled schedule
    n = 1536
    small = lambda schedule: attn_vq_prefill(q[:, :2, :n], codes[:, :2, :n], cb[:2], v[:, :2, :n], k_exact=k[:, :2, :n],
                                             window_size=W, schedule=schedule)
    assert torch.equal(small("default"), small("tiled"))


def test_vq_prefill_pipelined_refuses_other_configurations():
    from vqtree_amd._lib import VqaError

    q, k, v = (_randn(1, 1, 256, 128, seed=s).cuda() for s in range(3))
    cb = _randn(1, 2, 256, 128, seed=4, std=0.35).cuda()
    codes = _codes(1, 1, 256, 2, seed=5).cuda()
    with pytest.raises(VqaError):  # window not a multiple of 128
        attn_vq_prefill(q, codes, cb, v, k_exact=k, window_size=100, schedule="pipelined")


@pytest.mark.parametrize("with_rerope", [False, True])
@pytest.mark.parametrize("B,H,N,D,K,W", [(1, 2, 1024, 128, 256, 256), (2, 2, 900, 64, 128, 128), (1, 1, 700, 128, 200, 384),
                                          (1, 2, 650, 128, 256, 0), (2, 1, 333, 64, 128, 0)])
def test_single_codebook_prefill_takes_the_codeword_route(B, H, N, D, K, W, with_rerope):
    """M = 1 with the block boundary: `attn_vq_prefill` runs the window kernel + count-weighted codeword kernel (far
    context in O(N*K)); same oracle, and the per-key kernel forced on the same inputs agrees.  Includes lengths that
    are no multiple of 128 and a window of 0 (only the keys of the query's own 128-block are exact)."""
    _say(f"single-codebook prefill B{B} H{H} N{N} D{D} K{K} W{W} rerope={with_rerope}")
    q, k, v, q2, k2 = (_randn(B, H, N, D, seed=110 + s) for s in range(5))
    cb = _randn(H, 1, K, D, seed=115, std=0.5)
    codes = _codes(B, H, N, 1, K, seed=116)
    kw = dict(k_exact=k, window_size=W)
    if with_rerope:
        kw.update(q2=q2, k2=k2)
    want, want_lse = oracle.attn_vq_prefill(q, codes, cb, v, **kw)
    kw = {n: (t.cuda() if torch.is_tensor(t) else t) for n, t in kw.items()}
    out, lse = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), return_lse=True, **kw)
    per_key = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), schedule="per_key", **kw)
    torch.cuda.synchronize()
    assert_close_16(out, want, "codeword-route prefill")
    assert_close_lse(lse, want_lse, atol=1e-2)
    assert_close_16(per_key, want, "per-key prefill, M = 1")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_pipelined_core_with_large_and_drifting_scores(dtype):
    """The pipelined core keeps a LAZY reference maximum per row (it moves only when a tile exceeds it by 2^8) and adds
    -m inside the score product.  Scores here are several times the usual size (up to +-40 in base 2) and drift
    upwards along the sequence (keys grow with their position), so that the maximum of most rows moves again and
    again, late in their key loop; plus a block of rows whose first visible keys score hugely negative (-50).  Finite
    results, oracle tolerance, on the VQ prefill kernel, plain causal attention and the sliding-window kernel.
    (The core rounds the query to 16 bits once more after scaling it: a score error of 1.1e-3 |q o k| scale log2(e),
    the size of the error the 16-bit inputs carry themselves.  With keys of several times this norm competing for one
    row, that error exceeds the 16-bit output tolerance in bf16; f16 has 8 x the margin.)"""
    _say(f"pipelined core, large drifting scores {dtype}")
    B, H, N, D, W = 1, 2, 2304, 128, 512
    g = torch.Generator("cpu").manual_seed(77)
    q = (torch.randn(B, H, N, D, generator=g) * 1.5).to(dtype)
    ramp = torch.linspace(0.5, 2.0, N).view(1, 1, N, 1)
    k = (torch.randn(B, H, N, D, generator=g) * ramp).to(dtype)
    k[:, :, :64] = (-2.0 * q[:, :, 1000:1064].float().sign()).to(dtype)   # score -50 for rows 1000..1063, +-15 elsewhere
    v = torch.randn(B, H, N, D, generator=g).to(dtype)
    scale = 1.0 / math.sqrt(D)
    # (1) plain causal attention through the window entry (window >= N)
    want, want_lse = oracle.local_attn(q, k, v, N, "strict", scale)
    out = triton_fused_local_attn.flash_attn_func(_bnhd(q).cuda(), _bnhd(k).cuda(), _bnhd(v).cuda(), N, scale)
    assert_close_16(out.transpose(1, 2), want, "causal, large scores")
    # (2) the sliding-window kernel, block rule and ReRoPE pair rule (second pair: the same tensors negated twice over)
    for mode in ("loose", "rerope"):
        want, want_lse = oracle.local_attn(q, k, v, W, mode, scale, q2=q, k2=k)
        args = [_bnhd(x).cuda() for x in (q, k, v)]
        if mode == "loose":
            out, lse = triton_fused_local_attn2.flash_attn_func(*args, W, scale, return_lse=True)
        else:
            out, lse = triton_fused_local_attn_rerope.flash_attn_func(args[0], args[0], args[1], args[1], args[2], W,
                                                                      scale, return_lse=True)
        assert_close_16(out.transpose(1, 2), want, f"{mode}, large scores")
        assert torch.isfinite(lse).all()
        assert_close_lse(lse, want_lse, atol=3e-2)
    # (3) the VQ prefill kernel: every key quantised, codebooks scaled up
    cb = (torch.randn(H, 2, 256, D, generator=g) * 1.0).to(dtype)
    codes = _codes(B, H, N, 2, 256, seed=78)
    want, _ = oracle.attn_vq_prefill(q, codes, cb, v, k_exact=k, window_size=W, softmax_scale=scale)
    out = attn_vq_prefill(q.cuda(), codes.cuda(), cb.cuda(), v.cuda(), k_exact=k.cuda(), window_size=W,
                          softmax_scale=scale, schedule="pipelined")
    assert_close_16(out, want, "vq prefill, large scores")
