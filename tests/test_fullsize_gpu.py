"""GPU checks at the full benchmark sizes.  The dense oracle cannot produce whole outputs at these sizes in seconds, so
every case is checked (1) on sampled (head, query-row) pairs against the oracle's per-row statement (dense fp32 softmax
over the keys the row may see, with the oracle's own boundary / mask rules) and (2) through the causal prefix property:
the rows of a shorter prefix of the same inputs are reproduced bit for bit where the tiling is identical and within
tolerance elsewhere."""
import math

import pytest
import torch

import oracle
from tests.util import assert_close_16
from vqtree_amd.ops.attn_vq import attn_vq_prefill, rope_tables, rotate_half
from vqtree_amd.ops.triton_fused_local_attn_rerope import flash_attn_func as local_rerope
from vqtree_amd.synthetic import prefill_c3

pytestmark = pytest.mark.gpu


def _row_reference(q_row, keys, values, scale):
    """softmax(q . keys^T * scale) @ values in fp32 for one query row."""
    s = (keys.float() @ q_row.float()) * scale
    p = torch.softmax(s, dim=0)
    return p @ values.float()


@pytest.mark.parametrize("schedule", ["default", "tiled"])
def test_vq_prefill_benchmark_size_sampled_rows_and_prefix(schedule):
    """At this size the default call runs the pipelined schedule; "tiled" forces the other kernel."""
    print(f"fullsize: VQ prefill batch 1, 32 heads, 8192 tokens, window 1024, schedule {schedule}", flush=True)
    case = prefill_c3("cuda")
    B, H, N, D = case.q.shape
    W = case.window
    out = attn_vq_prefill(case.q, case.codes, case.codebooks, case.v, k_exact=case.k_exact, window_size=W,
                          softmax_scale=case.softmax_scale, schedule=schedule)
    torch.cuda.synchronize()
    bnd = oracle.far_boundary(N, W, "block")
    rows = [0, 1, 127, 128, W + 127, W + 128, W + 129, 2047, 4096, 5000, N - 129, N - 1]
    for h in (0, 13, 31):
        k_hat = oracle.reconstruct_keys(case.codes[:, h:h + 1].cpu(), case.codebooks[h:h + 1].cpu())[0, 0]  # [N,D]
        k_ex, v, q = case.k_exact[0, h].cpu(), case.v[0, h].cpu(), case.q[0, h].cpu()
        for i in rows:
            b = int(bnd[i])
            keys = torch.cat([k_hat[:b], k_ex[b:i + 1].float()])
            want = _row_reference(q[i], keys, v[:i + 1], case.softmax_scale)
            assert_close_16(out[0, h, i].cpu(), want, f"head {h} row {i}")
    # prefix property: the first 4096 tokens alone give the same rows
    half = N // 2
    out_half = attn_vq_prefill(case.q[:, :, :half], case.codes[:, :, :half], case.codebooks, case.v[:, :, :half],
                               k_exact=case.k_exact[:, :, :half], window_size=W, softmax_scale=case.softmax_scale,
                               schedule=schedule)
    torch.cuda.synchronize()
    diff = (out_half.float() - out[:, :, :half].float()).abs().max().item()
    assert diff <= 2e-2, diff


def test_local_rerope_benchmark_size_sampled_rows_and_prefix():
    print("fullsize: local ReRoPE window batch 2, 32 heads, 16384 tokens, window 512", flush=True)
    B, H, N, D, W = 2, 32, 16384, 128, 512
    g = torch.Generator(device="cuda").manual_seed(4)
    q, k, v = (torch.randn(B, N, H, D, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
               for _ in range(3))
    cos, sin = rope_tables(D, N, dtype=torch.bfloat16, device="cuda")
    rope = lambda x, c, s_: x * c + rotate_half(x) * s_
    q1, k1 = rope(q, cos[None, :, None], sin[None, :, None]), rope(k, cos[None, :, None], sin[None, :, None])
    q2 = rope(q, cos[W + 1], sin[W + 1])
    scale = 1.0 / math.sqrt(D)
    out = local_rerope(q1, q2, k1, k, v, W, scale)  # [B,N,H,D]
    torch.cuda.synchronize()
    rows = [0, 127, 128, W, W + 1, W + 127, W + 128, 4095, 9999, N - 1]
    for b, h in ((0, 0), (1, 17), (1, 31)):
        q1h, q2h, k1h, kh, vh = (x[b, :, h].cpu().float() for x in (q1, q2, k1, k, v))
        for i in rows:
            lo = max(0, i // 128 * 128 - W)  # loose visibility: ops/triton_fused_local_attn2.py:37-46
            j = torch.arange(lo, i + 1)
            primary = (i - j) <= W            # in-window keys use the true-position pair
            s = torch.where(primary, k1h[lo:i + 1] @ q1h[i], kh[lo:i + 1] @ q2h[i]) * scale
            want = torch.softmax(s, 0) @ vh[lo:i + 1]
            assert_close_16(out[b, i, h].cpu(), want, f"b{b} h{h} row {i}")
    # the oracle's mask rules agree with the per-row statement used above on a small case
    vis, prim = oracle.local_visible_mask(700, 256, "rerope")
    for i in (0, 300, 699):
        lo = max(0, i // 128 * 128 - 256)
        assert vis[i].nonzero().flatten().tolist() == list(range(lo, i + 1))
        assert torch.equal(prim[i, lo:i + 1], (i - torch.arange(lo, i + 1)) <= 256)
    # prefix property
    half = N // 2
    out_half = local_rerope(q1[:, :half], q2[:, :half], k1[:, :half], k[:, :half], v[:, :half], W, scale)
    torch.cuda.synchronize()
    assert (out_half.float() - out[:, :half].float()).abs().max().item() <= 2e-2


def test_reference_shaped_route_benchmark_length_sampled_rows():
    """The whole caller chain (encoder -> preprocessing kernels -> rotary -> window kernel -> count kernel with fused
    merge) at 8192 tokens, window 1024, 512 codewords: sampled rows against the per-query statement of the reference's
    slow path (ops/attn_vq.py:305-333): exact keys in the window, raw keys with the clamped query on the strip down to
    the block boundary, quantised keys with the clamped query below it."""
    from vqtree_amd.ops import attn_vq as A

    print("fullsize: reference-shaped route, 4 heads, 8192 tokens, window 1024, 512 codewords", flush=True)
    B, H, N, D, W, C = 1, 4, 8192, 128, 1024, 512
    g = torch.Generator(device="cuda").manual_seed(9)
    q, k, v = (torch.randn(B, H, N, D, generator=g, device="cuda").bfloat16() for _ in range(3))
    cb = torch.randn(H, C, D, generator=g, device="cuda").bfloat16()
    pos = torch.arange(N, device="cuda").unsqueeze(0)
    cache = A.VectorQuantizedReRoPECache(W, cb)
    out = A.dispatch_attn(q, k, v, pos, cache).view(B, N, H, D)
    torch.cuda.synchronize()
    q1, k1, q2 = A.rerope_operands(q, k, pos, W)
    ids = cache.key_codes[0][..., 0].long().cpu() if cache.key_codes else None
    if ids is None:  # more than 256 codewords: the cache keeps no uint8 codes; encode again
        from vqtree_amd.ops.mini_vq import quantize_ids
        ids = quantize_ids(k, cb).cpu()
    scale = 1.0 / math.sqrt(D)
    for h in (0, 3):
        k_hat = cb[h].float().cpu()[ids[0, h]]  # [N,D]
        q1h, q2h, k1h, kh, vh = (x[0, h].float().cpu() for x in (q1, q2, k1, k, v))
        for i in (0, 1000, W + 127, W + 128, 3000, 5555, N - 1):
            boundary = max(0, (i - W) // 128 * 128)
            local = max(0, i - W)
            s = torch.cat([k_hat[:boundary] @ q2h[i], kh[boundary:local] @ q2h[i], k1h[local:i + 1] @ q1h[i]]) * scale
            want = torch.softmax(s, 0) @ vh[:i + 1]
            assert_close_16(out[0, i, h].cpu(), want, f"head {h} row {i}")
