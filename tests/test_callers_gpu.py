"""GPU tests of the caller layer (the attention core of the reference's HF module): dispatch, preprocessing, the
linear-time prefill against the per-query slow reference, and a generation step over the cached codes."""
import math

import pytest
import torch

import oracle
from tests.util import assert_close_16
from vqtree_amd.ops import attn_vq as A

pytestmark = pytest.mark.gpu


def _states(B, H, N, D, dtype, seed):
    g = torch.Generator("cpu").manual_seed(seed)
    mk = lambda: torch.randn(B, H, N, D, generator=g).to(dtype).cuda()
    return mk(), mk(), mk()


def test_reference_selfcheck_linear_vs_slow():
    """The reference's own check (ops/attn_vq.py:534-556): 2 heads of dim 64, fp16, LEN = 511, window 256,
    codebook randn(2,128,64); SORT_BASED_LINEAR against SLOW_REFERNECE through the dispatcher."""
    print("callers: linear vs slow, LEN=511 W=256", flush=True)
    B, H, N, D, W = 1, 2, 511, 64, 256
    q, k, v = _states(B, H, N, D, torch.float16, 1)
    codebook = torch.randn(H, 128, D, generator=torch.Generator("cpu").manual_seed(2)).half().cuda()
    pos = torch.arange(N, device="cuda").unsqueeze(0)
    fast = A.dispatch_attn(q, k, v, pos, A.VectorQuantizedReRoPECache(W, codebook))
    slow = A.dispatch_attn(q, k, v, pos, A.VectorQuantizedReRoPECache(W, codebook, attention_mode=A.AttentionMode.SLOW_REFERNECE))
    per_key = A.long_prefilling_per_key(q, k, v, pos, A.VectorQuantizedReRoPECache(W, codebook))
    torch.cuda.synchronize()
    assert fast.shape == (B, N, H * D)
    assert (fast.float() - slow.float()).abs().max() <= 2e-2
    assert (per_key.float() - slow.float()).abs().max() <= 2e-2
    # rows inside the window see no far context: both fast paths are plain exact attention there
    assert (fast[:, :W].float() - slow[:, :W].float()).abs().max() <= 1e-2


def test_preprocess_matches_oracle_bit_exact_indices():
    B, H, N, C, D = 2, 2, 640, 128, 64
    _, k, v = _states(B, H, N, D, torch.bfloat16, 3)
    cb = torch.randn(H, C, D, generator=torch.Generator("cpu").manual_seed(4)).to(torch.bfloat16).cuda()
    _, ids, onehot = A.multi_head_single_quantize(k, cb)
    cnt, v_vq, vi = A.sort_based_preprocess(ids, onehot, v)
    want_cnt, want_vvq, want_vi = oracle.sort_based_preprocess(ids.cpu(), v.cpu(), C, dtype=torch.bfloat16)
    assert torch.equal(cnt.cpu(), want_cnt) and torch.equal(vi.cpu(), want_vi)  # integer work: bit-exact
    assert torch.allclose(v_vq.float().cpu(), want_vvq.float(), atol=3e-2, rtol=1e-2)  # fp32 cumsum order differs
    # the encoder's ids are the first arg-max of the inner product evaluated in the model dtype
    want_ids = oracle.multi_head_single_quantize(k.cpu(), cb.cpu())[1]
    assert (ids.cpu() != want_ids).float().mean() < 5e-3  # bf16 matmul accumulation order may flip near-ties


@pytest.mark.parametrize("N,W,C", [(900, 256, 256), (1536, 512, 128)])
def test_linear_prefill_vs_oracle(N, W, C):
    print(f"callers: linear prefill N{N} W{W} C{C}", flush=True)
    B, H, D = 2, 2, 128
    q, k, v = _states(B, H, N, D, torch.bfloat16, 5)
    cb = torch.randn(H, C, D, generator=torch.Generator("cpu").manual_seed(6)).to(torch.bfloat16).cuda()
    pos = torch.arange(N, device="cuda").unsqueeze(0).expand(B, -1)
    cache = A.VectorQuantizedReRoPECache(W, cb)
    out = A.dispatch_attn(q, k, v, pos, cache)
    q1, k1, q2 = A.rerope_operands(q, k, pos, W)
    ids = cache.key_codes[0]
    want, _ = oracle.attn_vq_prefill(q1, ids, cb.unsqueeze(1), v, k_exact=k1, window_size=W, q2=q2, k2=k)
    assert_close_16(out.view(B, N, H, D).transpose(1, 2), want, "linear prefill")


def test_short_prefill_then_generation_steps():
    """Prefill shorter than window + 128 is exact causal attention; each later seqlen_q == 1 step attends over the
    cached key codes with the clamped query (dense oracle on the reconstructed keys)."""
    B, H, N, D, W, C = 2, 4, 300, 128, 256, 256
    q, k, v = _states(B, H, N, D, torch.bfloat16, 7)
    cb = torch.randn(H, C, D, generator=torch.Generator("cpu").manual_seed(8)).to(torch.bfloat16).cuda()
    pos = torch.arange(N, device="cuda").unsqueeze(0).expand(B, -1)
    cache = A.VectorQuantizedReRoPECache(W, cb)
    out = A.dispatch_attn(q, k, v, pos, cache)
    q1, k1, _ = A.rerope_operands(q, k, pos, W)
    want, _ = oracle.local_attn(q1, k1, v, N, "strict")
    assert_close_16(out.view(B, N, H, D).transpose(1, 2), want, "short prefill")
    assert cache.get_seq_length(0) == N and cache.seen_tokens == N
    all_ids, all_v = cache.key_codes[0].long(), v
    for step in range(3):
        qs, ks, vs = _states(B, H, 1, D, torch.bfloat16, 20 + step)
        o = A.dispatch_attn(qs, ks, vs, torch.full((B, 1), N + step, device="cuda"), cache)
        n_now = N + step + 1
        assert cache.get_seq_length(0) == n_now and o.shape == (B, 1, H * D)
        all_ids = torch.cat([all_ids, A.quantize_ids(ks, cb).unsqueeze(-1)], dim=2)
        all_v = torch.cat([all_v, vs], dim=2)
        cos, sin = A.rope_tables(D, W + 2, dtype=torch.bfloat16, device="cuda")
        q2 = qs * cos[W + 1] + A.rotate_half(qs) * sin[W + 1]
        want, _ = oracle.attn_vq_decode(q2, all_ids, cb.unsqueeze(1), all_v, 1 / math.sqrt(D))
        assert_close_16(o.view(B, 1, H, D).transpose(1, 2), want, f"generation step {step}")


def test_decode_harness_matches_dense_reference():
    """Small Llama-shaped decode loop over a VQ key cache: the HIP decode kernel inside the loop against dense fp32
    attention over the reconstructed keys, step by step on identical state."""
    from vqtree_amd.decode_harness import VQDecodeModel, encode_residual

    def dense_attention(q2, codes, codebooks, v, softmax_scale):
        out, _ = oracle.attn_vq_decode(q2, codes, codebooks, v, softmax_scale)
        return out.to(q2.dtype).cuda()

    kw = dict(layers=2, hidden=256, heads=2, head_dim=128, ffn=512, vocab=1000, n_codebooks=4, window=128,
              capacity=400, batch=2)
    a, b = VQDecodeModel(**kw), VQDecodeModel(**kw)
    a.fill_random_context(300), b.fill_random_context(300)
    tok = torch.tensor([3, 777], device="cuda")
    for step in range(3):
        ta, la = a.step(tok, return_logits=True)
        tb, lb = b.step(tok, attention=dense_attention, return_logits=True)
        assert (la.float() - lb.float()).abs().max() <= 2e-2 * max(1.0, float(lb.float().abs().max()))
        assert torch.equal(a.layers[0]["codes"][:, :, 300 + step], b.layers[0]["codes"][:, :, 300 + step])
        tok = tb
    assert a.length == 303
    # the greedy residual encoder picks, stage by stage, the nearest codeword of the running residual
    x = torch.randn(1, 2, 5, 128, device="cuda").bfloat16()
    cb = a.layers[0]["codebooks"]
    codes = encode_residual(x, cb)
    r = x[0, 1, 2].float()
    for m in range(4):
        d = ((r[None] - cb[1, m].float()) ** 2).sum(-1)
        assert int(codes[0, 1, 2, m]) == int(d.argmin())
        r = r - cb[1, m, int(codes[0, 1, 2, m])].float()


def test_decode_harness_with_exact_window_matches_dense_reference():
    """Same loop with the last W keys kept exactly: coded far keys scored with the clamped query, window keys with
    the query at its true position, against dense fp32 softmax over [reconstructed far keys ; window keys].  W = 4
    and 12 steps make the 2W-row window buffer compact itself during the test."""
    from vqtree_amd.decode_harness import VQDecodeModel

    def dense_attention(q_far, q_win, codes, codebooks, v, k_win, softmax_scale):
        n, w = v.shape[2], k_win.shape[2]
        k_hat = oracle.reconstruct_keys(codes[:, :, : n - w].cpu(), codebooks.cpu())
        s_far = q_far.float().cpu() @ k_hat.transpose(-1, -2)
        s_win = q_win.float().cpu() @ k_win.float().cpu().transpose(-1, -2)
        scores = torch.cat([s_far, s_win], dim=-1) * softmax_scale
        out, _ = oracle.attend(scores, torch.ones(1, n, dtype=torch.bool), v.float().cpu())
        return out.to(q_far.dtype).cuda()

    kw = dict(layers=2, hidden=256, heads=2, head_dim=128, ffn=512, vocab=1000, n_codebooks=4, window=128,
              capacity=400, batch=2, exact_window=4)
    a, b = VQDecodeModel(**kw), VQDecodeModel(**kw)
    a.fill_random_context(300), b.fill_random_context(300)
    tok = torch.tensor([5, 42], device="cuda")
    for step in range(12):
        ta, la = a.step(tok, return_logits=True)
        tb, lb = b.step(tok, attention=dense_attention, return_logits=True)
        assert (la.float() - lb.float()).abs().max() <= 2e-2 * max(1.0, float(lb.float().abs().max())), step
        # layer 0 sees identical inputs in both models: its window rows must agree bit for bit
        assert torch.equal(a.layers[0]["kwin"][:, :, a.kwin_len - 4: a.kwin_len],
                           b.layers[0]["kwin"][:, :, b.kwin_len - 4: b.kwin_len])
        tok = tb
    assert a.length == 312 and a.kwin_len <= 8
    # a cache shorter than the window is plain exact attention
    c = VQDecodeModel(**dict(kw, exact_window=64))
    c.fill_random_context(10)
    d = VQDecodeModel(**dict(kw, exact_window=64))
    d.fill_random_context(10)
    _, lc = c.step(tok, return_logits=True)
    _, ld = d.step(tok, attention=dense_attention, return_logits=True)
    assert (lc.float() - ld.float()).abs().max() <= 2e-2 * max(1.0, float(ld.float().abs().max()))


def test_decode_harness_recorded_step_matches_eager_steps():
    """The decode step recorded once as a HIP graph (cache position and key count in device memory) and replayed,
    against the eager step on a twin model: same tokens, logits within tolerance, same appended codes."""
    from vqtree_amd.decode_harness import VQDecodeModel

    kw = dict(layers=2, hidden=256, heads=2, head_dim=128, ffn=512, vocab=1000, n_codebooks=4, window=128,
              capacity=400, batch=2)
    a, b = VQDecodeModel(**kw), VQDecodeModel(**kw)
    a.fill_random_context(300), b.fill_random_context(300)
    tok = torch.tensor([3, 777], device="cuda")
    with torch.no_grad():
        b.record_step(tok)  # runs one (warm-up) step eagerly on a side stream, then records
        ta, la = a.step(tok, return_logits=True)
        assert torch.equal(ta, b.tok) and b.length == a.length == 301
        for step in range(6):
            ta, la = a.step(ta, return_logits=True)
            tb = b.replay_step()
            torch.cuda.synchronize()
            assert (la.float() - b.logits.float()).abs().max() <= 2e-2 * max(1.0, float(la.float().abs().max())), step
            assert torch.equal(ta, tb), step
            n = a.length - 1
            assert torch.equal(a.layers[0]["codes"][:, :, n], b.layers[0]["codes"][:, :, n])
            _ = (a.layers[1]["values"][:, :, :8].float().sum(), torch.cuda.synchronize())  # eager work between replays
    assert b.length == a.length == 307


def test_rerope_caller_routes():
    """Attention core of the ReRoPE module: long prefill through the full ReRoPE kernel against the dense oracle,
    cache contents after it, a short prefill (plain causal) and a generation step against dense softmax over the
    cached keys."""
    from vqtree_amd.ops.attn_rerope import ReRoPECache, rerope_attn_forward
    from vqtree_amd.ops.attn_vq import rope_tables, rotate_half

    print("callers: rerope module core, N=300 W=128", flush=True)
    B, H, N, D, W = 1, 4, 300, 64, 128
    q, k, v = _states(B, H, N, D, torch.bfloat16, 11)
    pos = torch.arange(N, device="cuda").unsqueeze(0)
    cache = ReRoPECache(W)
    out = rerope_attn_forward(q, k, v, pos, cache)
    torch.cuda.synchronize()
    assert out.shape == (B, N, H * D)
    cos, sin = rope_tables(D, N + 1, dtype=torch.bfloat16, device="cuda")
    rope = lambda x, p: x * cos[p] + rotate_half(x) * sin[p]
    q1, k1, q2 = rope(q, pos[0]), rope(k, pos[0]), rope(q, W)
    ref, _ = oracle.rerope_full(q1.cpu(), q2.cpu(), k1.cpu(), k.cpu(), v.cpu(), True, 1 / math.sqrt(D), W)
    assert_close_16(out.view(B, N, H, D).transpose(1, 2).cpu(), ref)
    assert cache.get_seq_length() == N
    assert torch.equal(cache.key_cache[0][:, :, -W:], k1[:, :, -W:])
    assert torch.equal(cache.key_cache[0][:, :, :-W], rope(k, N - W)[:, :, :-W])

    # generation step: dense softmax over the keys the cache returns after the append
    g = torch.Generator("cpu").manual_seed(12)
    qn, kn, vn = (torch.randn(B, H, 1, D, generator=g).bfloat16().cuda() for _ in range(3))
    step = rerope_attn_forward(qn, kn, vn, torch.tensor([[N]], device="cuda"), cache)
    keys, vals = cache.key_cache[0].float().cpu(), cache.value_cache[0].float().cpu()
    cos2, sin2 = rope_tables(D, N + 1, dtype=torch.bfloat16, device="cuda")
    qr = (qn * cos2[N] + rotate_half(qn) * sin2[N]).float().cpu()
    want = torch.softmax(qr @ keys.transpose(-1, -2) / math.sqrt(D), -1) @ vals
    assert cache.get_seq_length() == N + 1
    assert_close_16(step.view(B, 1, H, D).transpose(1, 2).cpu(), want)

    # short prefill: window covers everything -> causal attention on the rotated operands
    Ns = 100
    short = rerope_attn_forward(q[:, :, :Ns], k[:, :, :Ns], v[:, :, :Ns], pos[:, :Ns], ReRoPECache(W))
    scores = q1[:, :, :Ns].float().cpu() @ k1[:, :, :Ns].float().cpu().transpose(-1, -2) / math.sqrt(D)
    ref_s, _ = oracle.attend(scores, torch.ones(Ns, Ns, dtype=torch.bool).tril(), v[:, :, :Ns].float().cpu())
    assert_close_16(short.view(B, Ns, H, D).transpose(1, 2).cpu(), ref_s)


def _largest_tensor(obj, seen=None):
    """Largest number of elements of any tensor reachable from obj (attributes, lists, tuples, dicts)."""
    seen = set() if seen is None else seen
    if id(obj) in seen:
        return 0
    seen.add(id(obj))
    if torch.is_tensor(obj):
        return obj.numel()
    if isinstance(obj, (list, tuple)):
        return max([_largest_tensor(x, seen) for x in obj] + [0])
    if isinstance(obj, dict):
        return max([_largest_tensor(x, seen) for x in obj.values()] + [0])
    if hasattr(obj, "__dict__"):
        return _largest_tensor(vars(obj), seen)
    return 0


@pytest.mark.parametrize("exact_window", [False, True])
def test_cache_keeps_no_tensor_of_the_prefill_size(exact_window):
    """What the VQ memory is for: after a long prefill (and after a generation step) the cache holds the count state
    [B,H,C,D], window buffers and one code byte per key -- no [B,H,N,D] tensor, and no closure over one."""
    import gc
    import weakref

    B, H, N, D, W, C = 1, 2, 4096, 128, 256, 128
    q, k, v = _states(B, H, N, D, torch.bfloat16, 41)
    cb = torch.randn(H, C, D, generator=torch.Generator("cpu").manual_seed(42)).to(torch.bfloat16).cuda()
    pos = torch.arange(N, device="cuda").unsqueeze(0)
    cache = A.VectorQuantizedReRoPECache(W, cb, generation_exact_window=exact_window)
    A.dispatch_attn(q, k, v, pos, cache)
    limit = B * H * max(C, W + 256) * D  # count-state sums / window buffers; the code bytes are B*H*N
    assert _largest_tensor(cache) <= max(limit, B * H * N)
    assert not hasattr(cache, "value_cache")
    refs = [weakref.ref(t) for t in (k, v)]
    del q, k, v
    gc.collect()
    assert all(r() is None for r in refs), "the cache still references the prefill's keys / values"
    qs, ks, vs = _states(B, H, 1, D, torch.bfloat16, 43)
    out = A.dispatch_attn(qs, ks, vs, torch.full((B, 1), N, device="cuda"), cache)
    torch.cuda.synchronize()
    assert out.shape == (B, 1, H * D) and torch.isfinite(out.float()).all()
    assert _largest_tensor(cache) <= max(limit, B * H * (N + 1))


def test_long_prefill_route_records_into_a_hip_graph():
    """The linear-time prefill route makes no device-to-host copy (rotary tables are sized on the host), so it can be
    recorded once and replayed: every replay must reproduce the eager result bit for bit."""
    B, H, N, D, W, C = 1, 4, 2048, 128, 512, 256
    q, k, v = _states(B, H, N, D, torch.bfloat16, 51)
    cb = torch.randn(H, C, D, generator=torch.Generator("cpu").manual_seed(52)).to(torch.bfloat16).cuda()
    pos = torch.arange(N, device="cuda").unsqueeze(0)
    run = lambda: A.dispatch_attn(q, k, v, pos, A.VectorQuantizedReRoPECache(W, cb))
    eager = run()  # also the warm-up: per-device set-up of the kernels happens outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = run()
    for i in range(3):
        recorded.zero_()
        torch.cuda.synchronize()
        graph.replay()
        _ = (q.float() * 2).sum().item()  # eager work and a synchronisation between the replays
        torch.cuda.synchronize()
        assert torch.equal(recorded, eager), f"replay {i}"
