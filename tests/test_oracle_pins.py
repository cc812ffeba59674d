"""Pins the CPU oracle to facts that do not depend on it: torch library routines, brute-force loops on tiny
inputs, closed forms and algebraic identities.  A dropped term, wrong sign/index or transposed operand in the
oracle fails at least one of these."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle.attention import T_BLOCK


def _rand(*shape, seed=0, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * std


def _codes(B, H, N, M, K=256, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, K, (B, H, N, M), generator=g).to(torch.uint8)


# ------------------------------------------------------------------ key reconstruction / gathers
def test_reconstruct_keys_bruteforce():
    B, H, N, M, K, D = 2, 3, 17, 4, 256, 8
    cb = _rand(H, M, K, D, seed=1)
    codes = _codes(B, H, N, M, seed=2)
    got = oracle.reconstruct_keys(codes, cb)
    for b in range(B):
        for h in range(H):
            for j in range(N):
                want = torch.zeros(D)
                for m in range(M):
                    want += cb[h, m, int(codes[b, h, j, m])]
                assert torch.equal(got[b, h, j], want)


def test_lut_route_equals_reconstruct_route_exactly():
    # integer-valued data: every product and sum is exact in fp32, so the two routes must agree bit for bit
    B, H, N, M, K, D = 1, 2, 33, 4, 256, 16
    g = torch.Generator().manual_seed(3)
    cb = torch.randint(-4, 5, (H, M, K, D), generator=g).float()
    q = torch.randint(-4, 5, (B, H, 5, D), generator=g).float()
    codes = _codes(B, H, N, M, seed=4)
    assert torch.equal(oracle.vq_scores_lut(q, codes, cb), oracle.vq_scores_reconstruct(q, codes, cb))


# ------------------------------------------------------------------ naive VQ attention
def test_vq_prefill_equals_sdpa_on_reconstructed_keys():
    B, H, N, M, D = 2, 2, 150, 2, 16
    q, v = _rand(B, H, N, D, seed=5), _rand(B, H, N, D, seed=6)
    cb = _rand(H, M, 256, D, seed=7, std=0.5)
    codes = _codes(B, H, N, M, seed=8)
    out, lse2 = oracle.attn_vq_prefill(q, codes, cb, v)
    k_hat = oracle.reconstruct_keys(codes, cb)
    want = F.scaled_dot_product_attention(q, k_hat, v, is_causal=True)
    assert torch.allclose(out, want, atol=2e-6)
    s = (q @ k_hat.transpose(-1, -2)) / math.sqrt(D)
    s = s.masked_fill(~torch.ones(N, N, dtype=torch.bool).tril(), float("-inf"))
    assert torch.allclose(lse2, torch.logsumexp(s, -1) / math.log(2.0), atol=1e-5)


def test_vq_decode_equals_sdpa():
    B, H, N, M, D = 2, 3, 97, 4, 32
    q, v = _rand(B, H, 1, D, seed=9), _rand(B, H, N, D, seed=10)
    cb = _rand(H, M, 256, D, seed=11, std=0.35)
    codes = _codes(B, H, N, M, seed=12)
    out, _ = oracle.attn_vq_decode(q, codes, cb, v)
    want = F.scaled_dot_product_attention(q, oracle.reconstruct_keys(codes, cb), v)
    assert torch.allclose(out, want, atol=2e-6)


def test_zero_codebooks_give_running_mean_of_v():
    B, H, N, D = 1, 2, 64, 8
    v = _rand(B, H, N, D, seed=13)
    out, lse2 = oracle.attn_vq_prefill(_rand(B, H, N, D, seed=14), _codes(B, H, N, 2), torch.zeros(H, 2, 256, D), v)
    want = torch.cumsum(v, 2) / torch.arange(1, N + 1)[None, None, :, None]
    assert torch.allclose(out, want, atol=1e-6)
    assert torch.allclose(lse2, torch.log2(torch.arange(1, N + 1).float()).expand(B, H, N), atol=1e-6)


def test_dominant_code_selects_its_value_row():
    # one key has a codeword aligned with q and a huge norm: softmax collapses onto that key's V row
    B, H, N, D = 1, 1, 40, 8
    q = torch.ones(B, H, 1, D)
    cb = torch.zeros(H, 1, 256, D)
    cb[0, 0, 7] = 100.0
    codes = torch.zeros(B, H, N, 1, dtype=torch.uint8)
    codes[0, 0, 23, 0] = 7
    v = _rand(B, H, N, D, seed=15)
    out, _ = oracle.attn_vq_decode(q, codes, cb, v)
    assert torch.allclose(out[0, 0, 0], v[0, 0, 23], atol=1e-6)


# ------------------------------------------------------------------ window masks against the kernels' tile stages
def _stage_simulation(n, w, mode, T=T_BLOCK):
    """Walk the tile stages the way the window kernels do and record, per (i, j), whether the key is scored and
    with which operand pair.  Written from the stage bounds, not from the closed-form predicates."""
    vis = np.zeros((n, n), dtype=bool)
    prim = np.ones((n, n), dtype=bool)
    for t in range((n + T - 1) // T):
        rows = range(t * T, min((t + 1) * T, n))
        if mode in ("strict", "rerope"):
            lo1, hi1 = max(t * T - w, 0), max(t * T - w + T, 0)
            for j in range(lo1, min(hi1, n)):
                for i in rows:
                    inside = i <= j + w
                    if mode == "strict":
                        vis[i, j] |= inside
                    else:
                        vis[i, j] = True
                        prim[i, j] = inside
            lo2, hi2 = max(t * T - w + T, 0), t * T
            for j in range(lo2, hi2):
                for i in rows:
                    vis[i, j] = True
        else:  # loose: one unmasked stage [tT - W, tT)
            for j in range(max(t * T - w, 0), t * T):
                for i in rows:
                    vis[i, j] = True
        for j in range(t * T, min((t + 1) * T, n)):
            for i in rows:
                if i >= j:
                    vis[i, j] = True
    return vis, prim


@pytest.mark.parametrize("mode", ["strict", "loose", "rerope"])
@pytest.mark.parametrize("n,w", [(384, 128), (300, 128), (511, 256), (130, 128), (257, 128), (700, 384)])
def test_window_masks_match_stage_walk(mode, n, w):
    vis, prim = oracle.local_visible_mask(n, w, mode)
    svis, sprim = _stage_simulation(n, w, mode)
    assert np.array_equal(vis.numpy(), svis)
    if mode == "rerope":
        assert np.array_equal((prim & vis).numpy(), sprim & svis)


def test_loose_mask_equals_reference_ref_impl_formula():
    n, w = 512, 256
    qpos = torch.arange(n)
    kpos = (torch.arange(n // 128).repeat_interleave(128) + 1) * 128
    want = ((qpos[:, None] - kpos[None, :]) < w).tril()
    vis, _ = oracle.local_visible_mask(n, w, "loose")
    assert torch.equal(vis, want)


def test_rerope_window_union_is_block_boundary():
    for n, w in [(640, 256), (515, 128)]:
        vis, _ = oracle.local_visible_mask(n, w, "rerope")
        bnd = oracle.far_boundary(n, w, "block")
        for i in range(n):
            cols = torch.nonzero(vis[i]).flatten()
            assert cols[0] == bnd[i] and cols[-1] == i and len(cols) == i - bnd[i] + 1


def test_strict_window_equals_sdpa_with_mask():
    B, H, N, D, W = 1, 2, 300, 16, 128
    q, k, v = (_rand(B, H, N, D, seed=s) for s in (20, 21, 22))
    out, _ = oracle.local_attn(q, k, v, W, "strict", softmax_scale=0.5)
    i, j = torch.arange(N)[:, None], torch.arange(N)[None, :]
    want = F.scaled_dot_product_attention(q, k, v, attn_mask=(j <= i) & (i - j <= W), scale=0.5)
    assert torch.allclose(out, want, atol=2e-6)


@pytest.mark.parametrize("mode", ["strict", "loose", "rerope"])
def test_window_covering_everything_is_causal_sdpa(mode):
    B, H, N, D = 1, 2, 200, 16
    q, k, v = (_rand(B, H, N, D, seed=s) for s in (23, 24, 25))
    junk = _rand(B, H, N, D, seed=26)
    out, _ = oracle.local_attn(q, k, v, 256, mode, q2=junk, k2=junk)
    assert torch.allclose(out, F.scaled_dot_product_attention(q, k, v, is_causal=True), atol=2e-6)


# ------------------------------------------------------------------ full ReRoPE
def test_rerope_full_large_window_is_sdpa():
    B, H, N, D = 1, 2, 160, 16
    q1, k1, v = (_rand(B, H, N, D, seed=s) for s in (30, 31, 32))
    junk = _rand(B, H, N, D, seed=33)
    out, _ = oracle.rerope_full(q1, junk, k1, junk, v, True, 0.3, N)
    assert torch.allclose(out, F.scaled_dot_product_attention(q1, k1, v, is_causal=True, scale=0.3), atol=2e-6)
    out, _ = oracle.rerope_full(q1, junk, k1, junk, v, False, 0.3, N)
    assert torch.allclose(out, F.scaled_dot_product_attention(q1, k1, v, scale=0.3), atol=2e-6)


def test_rerope_full_selects_by_strict_distance():
    # q1.k1 == 1 and q2.k2 == 0 everywhere: weights are e inside |i-j| < W and 1 outside, so the output is known
    N, D, W = 12, 4, 3
    q1 = torch.zeros(1, 1, N, D); q1[..., 0] = 1
    k1 = q1.clone()
    z = torch.zeros(1, 1, N, D)
    v = _rand(1, 1, N, D, seed=34)
    out, _ = oracle.rerope_full(q1, z, k1, z, v, True, 1.0, W)
    for i in range(N):
        wts = torch.tensor([math.e if i - j < W else 1.0 for j in range(i + 1)])
        want = (wts[:, None] * v[0, 0, : i + 1]).sum(0) / wts.sum()
        assert torch.allclose(out[0, 0, i], want, atol=1e-6)


def test_rope_shift_identity_and_tables():
    D, P = 16, 64
    cos, sin = oracle.rope_tables(D, P)
    # table closed form
    r = torch.arange(D // 2).float()
    inv = 10000.0 ** (-2 * r / D)
    assert torch.allclose(cos[5, : D // 2], torch.cos(5 * inv)) and torch.allclose(sin[5, D // 2 :], torch.sin(5 * inv))
    q, k = _rand(1, 1, 1, D, seed=35), _rand(1, 1, 1, D, seed=36)
    # <RoPE(q,p), RoPE(k,0)> == <RoPE(q,i), RoPE(k,i-p)>
    for i, p in [(40, 7), (63, 33)]:
        a = (oracle.apply_rope(q, cos, sin, p) * oracle.apply_rope(k, cos, sin, 0)).sum()
        b = (oracle.apply_rope(q, cos, sin, i) * oracle.apply_rope(k, cos, sin, i - p)).sum()
        assert torch.allclose(a, b, atol=1e-4)
    assert torch.equal(oracle.apply_rope(k, cos, sin, 0), k)  # k2 = RoPE(k, 0) = k


# ------------------------------------------------------------------ LSE merge (closed form: partition of the keys)
def test_merge_of_a_partition_equals_softmax_over_union():
    B, H, N, D = 1, 2, 90, 8
    q, k, v = (_rand(B, H, N, D, seed=s) for s in (40, 41, 42))
    s = (q @ k.transpose(-1, -2)) * 0.4
    i, j = torch.arange(N)[:, None], torch.arange(N)[None, :]
    vis = j <= i
    part = (j % 3 == 0)
    o_a, l_a = oracle.attend(s, vis & part, v)
    o_b, l_b = oracle.attend(s, vis & ~part, v)
    o_u, l_u = oracle.attend(s, vis, v)
    o_m, l_m = oracle.merge_state(o_a, l_a, o_b, l_b)
    assert torch.allclose(o_m, o_u, atol=2e-6) and torch.allclose(l_m, l_u, atol=1e-5)
    # rows where one side is empty (-inf) are passed through
    empty = torch.isinf(l_b)
    assert empty.any() and torch.equal(o_m[empty], o_a[empty])


# ------------------------------------------------------------------ quantiser, preprocessing, count kernel
def test_quantize_bruteforce_and_first_max_ties():
    B, H, N, C, D = 2, 2, 20, 8, 4
    x = _rand(B, H, N, D, seed=50)
    cb = _rand(H, C, D, seed=51)
    cb[:, 5] = cb[:, 2]  # exact tie between code 2 and 5 -> 2 must win whenever it is the max
    quant, ids, onehot = oracle.multi_head_single_quantize(x, cb)
    for b in range(B):
        for h in range(H):
            for n in range(N):
                best, arg = -1e30, -1
                for c in range(C):
                    p = float((x[b, h, n] * cb[h, c]).sum())
                    if p > best:
                        best, arg = p, c
                assert int(ids[b, h, n]) == arg and arg != 5
                assert torch.equal(quant[b, h, n], cb[h, arg])
    assert torch.equal(onehot.argmax(-1), ids) and onehot.sum(-1).eq(1).all()


def test_encode_residual_is_stagewise_nearest_neighbour():
    """Each stage picks the codeword closest (L2, torch.cdist) to the running residual; first minimum on exact ties;
    the reconstruction error never grows when the codebook holds the zero vector."""
    B, H, N, M, K, D = 2, 2, 24, 3, 8, 4
    x = _rand(B, H, N, D, seed=54)
    cb = _rand(H, M, K, D, seed=55)
    cb[:, :, 6] = cb[:, :, 1]  # exact duplicate: code 6 must never be chosen
    cb[:, :, 0] = 0.0
    codes = oracle.encode_residual(x, cb)
    assert codes.shape == (B, H, N, M) and not (codes == 6).any()
    r = x.clone().double()
    prev = (r * r).sum(-1)
    for m in range(M):
        for h in range(H):
            dist = torch.cdist(r[:, h], cb[h, m].double())  # [B,N,K]
            assert torch.equal(dist.argmin(-1), codes[:, h, :, m])
            r[:, h] -= cb[h, m].double()[codes[:, h, :, m]]
        err = (r * r).sum(-1)
        assert (err <= prev + 1e-9).all()
        prev = err
    # reconstruction through the key-reconstruction oracle leaves exactly that residual
    torch.testing.assert_close(x.double() - oracle.reconstruct_keys(codes, cb).double(), r, atol=1e-5, rtol=0)


def test_preprocess_invariants_bruteforce():
    B, H, N, C, D = 1, 2, 384, 8, 4
    g = torch.Generator().manual_seed(52)
    ids = torch.randint(0, C - 1, (B, H, N), generator=g)  # code C-1 never occurs -> cnt == 0 column
    v = _rand(B, H, N, D, seed=53)
    cnt, v_vq, vi = oracle.sort_based_preprocess(ids, v, C, dtype=torch.float32)
    assert cnt.shape == (B, H, N // 128, C) and v_vq.shape == (B, H, N + 1, D)
    for t in range(N // 128):
        assert (cnt[:, :, t].sum(-1) == 128 * (t + 1)).all()
        for h in range(H):
            for c in range(C):
                sel = ids[0, h, : 128 * (t + 1)] == c
                assert int(cnt[0, h, t, c]) == int(sel.sum())
                if sel.any():
                    assert torch.allclose(v_vq[0, h, vi[0, h, t, c]], v[0, h, : 128 * (t + 1)][sel].sum(0), atol=1e-4)
    assert (cnt[..., C - 1] == 0).all() and torch.equal(v_vq[:, :, 0], torch.zeros(B, H, D))


def _rerope_case(N, W, C, D, H=2, seed=60):
    q, k, v = (_rand(1, H, N, D, seed=seed + s) for s in range(3))
    cb = _rand(H, C, D, seed=seed + 3)
    cos, sin = oracle.rope_tables(D, N + W + 2)
    pos = torch.arange(N)
    q1, k1 = oracle.apply_rope(q, cos, sin, pos), oracle.apply_rope(k, cos, sin, pos)
    q2 = oracle.apply_rope(q, cos, sin, W + 1)
    k_hat, ids, _ = oracle.multi_head_single_quantize(k, cb)
    return q1, q2, k1, k, k_hat, ids, cb, v


@pytest.mark.parametrize("N,W", [(511, 256), (640, 128)])
def test_count_kernel_path_equals_slow_reference_and_per_key_form(N, W):
    C, D = 128, 16
    q1, q2, k1, k, k_hat, ids, cb, v = _rerope_case(N, W, C, D)
    want = oracle.slow_reference(q1, k1, q2, k, k_hat, v, W)
    # per-key additive-code formulation with M = 1
    per_key, _ = oracle.attn_vq_prefill(
        q1, ids[..., None], cb[:, None], v, k_exact=k1, window_size=W, q2=q2, k2=k, boundary_mode="block"
    )
    assert torch.allclose(per_key, want, atol=5e-6)
    # reference-shaped route: sort preprocessing -> window kernel + count kernel -> merge
    n_pad = (N // 128) * 128  # the reference samples whole blocks only (ops/attn_vq.py:411-413)
    cnt, v_vq, vi = oracle.sort_based_preprocess(ids, v, C, dtype=torch.float32)
    got = oracle.vq_attn_forward(q1, q2, k1, cb, cnt, k, v, v_vq, vi, W)
    assert n_pad >= W + 128
    assert torch.allclose(got, want, atol=2e-4)  # fp32 cumsum cancellation of the sort route


def test_exact_boundary_mode_partitions_at_i_minus_w():
    N, W, D = 300, 128, 8
    q, k, v = (_rand(1, 1, N, D, seed=s) for s in (70, 71, 72))
    cb = _rand(1, 2, 256, D, seed=73, std=0.5)
    codes = _codes(1, 1, N, 2, seed=74)
    out, _ = oracle.attn_vq_prefill(q, codes, cb, v, k_exact=k, window_size=W, boundary_mode="exact")
    k_hat = oracle.reconstruct_keys(codes, cb)
    for i in (0, 127, 128, 129, 299):
        lb = max(0, i - W)
        s = torch.cat([k_hat[0, 0, :lb] @ q[0, 0, i], k[0, 0, lb : i + 1] @ q[0, 0, i]]) / math.sqrt(D)
        want = torch.softmax(s, 0) @ v[0, 0, : i + 1]
        assert torch.allclose(out[0, 0, i], want, atol=2e-6)
