"""GPU parity of the seqlen_q = 1 VQ-attention kernel against the CPU oracle (through the C ABI via ctypes)."""
import math

import pytest
import torch

import oracle
from tests.util import assert_close_16, assert_close_lse
from vqtree_amd.ops.attn_vq import attn_vq_decode
from vqtree_amd.synthetic import decode_case

pytestmark = pytest.mark.gpu


def _check(case, num_splits=0, what=""):
    print(f"decode case {what} q{tuple(case.q.shape)} codes{tuple(case.codes.shape)} splits={num_splits}", flush=True)
    out, lse = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, softmax_scale=case.softmax_scale,
                              return_lse=True, num_splits=num_splits)
    torch.cuda.synchronize()
    want, want_lse = oracle.attn_vq_decode(case.q, case.codes, case.codebooks, case.v, case.softmax_scale)
    assert out.dtype == case.q.dtype and out.shape == case.q.shape
    assert_close_16(out, want, what)
    assert_close_lse(lse, want_lse)


@pytest.mark.parametrize("N", [1, 5, 63, 64, 65, 255, 256, 257, 1000, 4097])
def test_ragged_lengths(N):
    _check(decode_case(2, 3, N, 128, 4, seed=N), what=f"N={N}")


@pytest.mark.parametrize("splits", [1, 2, 3, 7, 16])
def test_split_counts(splits):
    # more splits than 256-key chunks leaves some splits empty: they must merge as no-ops
    _check(decode_case(1, 4, 1500, 128, 4, seed=7), num_splits=splits, what=f"splits={splits}")


@pytest.mark.parametrize("D,M,K", [(128, 1, 256), (128, 2, 256), (128, 8, 256), (64, 4, 256), (64, 1, 100), (128, 4, 37),
                                   (64, 8, 256), (64, 2, 16)])
def test_codebook_shapes(D, M, K):
    _check(decode_case(2, 2, 777, D, M, K, seed=D + M + K), what=f"D={D} M={M} K={K}")


def test_f16():
    _check(decode_case(2, 2, 900, 128, 4, dtype=torch.float16, seed=11), what="f16")
    _check(decode_case(1, 2, 300, 64, 2, dtype=torch.float16, seed=12), what="f16 D64")


def test_batch_larger_than_one_lut_tile():
    # the lookup-table kernel sweeps the batch 16 rows at a time
    _check(decode_case(19, 2, 130, 128, 4, seed=13), what="B=19")


def test_strided_v_and_q():
    # V given as a [B,N,H,D] buffer viewed as [B,H,N,D] (row stride H*D), q as a slice of a longer sequence
    case = decode_case(2, 4, 600, 128, 4, seed=14)
    v_bnhd = case.v.transpose(1, 2).contiguous()
    q_long = torch.randn(2, 4, 5, 128, device="cuda").to(torch.bfloat16)
    q_long[:, :, 3:4] = case.q
    case.v = v_bnhd.transpose(1, 2)
    case.q = q_long[:, :, 3:4]
    assert not case.v.is_contiguous() and not case.q.is_contiguous()
    _check(case, what="strided")


def test_zero_codebooks_give_mean_of_v():
    # every score is 0: the kernel reduces to a streaming mean of V, a closed form independent of the oracle
    case = decode_case(2, 2, 3000, 128, 4, seed=15)
    case.codebooks.zero_()
    out, lse = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, return_lse=True)
    want = case.v.float().mean(dim=2, keepdim=True)
    assert torch.allclose(out.float(), want, atol=4e-3)
    assert torch.allclose(lse, torch.full_like(lse, math.log2(3000)), atol=1e-4)


def test_dominant_key_selects_its_value_row():
    case = decode_case(1, 2, 2048, 128, 1, seed=16)
    case.codebooks.zero_()
    case.codebooks[:, 0, 9] = (case.q[0, :, 0] * 4).to(case.codebooks.dtype)  # aligned with q, huge score
    case.codes.zero_()
    case.codes[0, 0, 1234, 0] = 9
    case.codes[0, 1, 77, 0] = 9
    out = attn_vq_decode(case.q, case.codes, case.codebooks, case.v)
    assert torch.equal(out[0, 0, 0], case.v[0, 0, 1234]) and torch.equal(out[0, 1, 0], case.v[0, 1, 77])


def test_large_scores_do_not_overflow():
    case = decode_case(1, 2, 1024, 128, 4, seed=17, cb_std=3.0)
    _check(case, what="large scores")


def test_full_size_sampled_units():
    """Benchmark shape (B16 H32 N32768 D128 M4): every output finite, sampled (b,h) units checked against the
    oracle, and the split count does not change the result beyond rounding."""
    from vqtree_amd.synthetic import decode_c2

    case = decode_c2()
    out, lse = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, return_lse=True)
    out2 = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, num_splits=3)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    assert (out.float() - out2.float()).abs().max() <= 2e-3
    for b, h in [(0, 0), (3, 17), (15, 31), (8, 5)]:
        want, want_lse = oracle.attn_vq_decode(case.q[b:b + 1, h:h + 1], case.codes[b:b + 1, h:h + 1],
                                               case.codebooks[h:h + 1], case.v[b:b + 1, h:h + 1], case.softmax_scale)
        assert_close_16(out[b:b + 1, h:h + 1], want, f"unit {b},{h}")
        assert_close_lse(lse[b:b + 1, h:h + 1], want_lse)


def test_harness_layer_shape_with_default_splits():
    """The per-layer shape of the 32-layer decode harness (B4 H32 N65536 D128 M4: 128 units, so the default split
    count is above one and the merge kernel runs): sampled (b, h) units against the oracle, and a call with one split
    per unit (direct store, no merge) agrees beyond rounding."""
    from vqtree_amd import _lib

    B, H, N, D, M = 4, 32, 65536, 128, 4
    print(f"decode at the harness layer shape B{B} H{H} N{N}", flush=True)
    assert _lib.load().vqa_decode_default_splits(B, H, N) > 1
    case = decode_case(B, H, N, D, M, device="cuda", seed=31, on_device=True)
    out, lse = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, return_lse=True)
    one = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, num_splits=1)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    assert (out.float() - one.float()).abs().max() <= 2e-3
    for b, h in [(0, 0), (1, 9), (3, 31), (2, 20)]:
        cpu = lambda t: t.cpu()
        want, want_lse = oracle.attn_vq_decode(cpu(case.q[b:b + 1, h:h + 1]), cpu(case.codes[b:b + 1, h:h + 1]),
                                               cpu(case.codebooks[h:h + 1]), cpu(case.v[b:b + 1, h:h + 1]),
                                               case.softmax_scale)
        assert_close_16(out[b:b + 1, h:h + 1], want, f"unit {b},{h}")
        assert_close_lse(lse[b:b + 1, h:h + 1], want_lse)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D,M", [(3, 4, 700, 128, 4), (17, 2, 300, 64, 2), (1, 1, 64, 128, 1)])
def test_query_rotated_inside_the_table_kernel(dtype, B, H, N, D, M):
    """rope=(cos_row, sin_row): the lookup-table kernel rotates the raw query itself.  The table it builds must be the
    one built from a query rotated by the rotary kernel beforehand, so the two calls agree bit for bit; the rotated
    query is also pinned against the oracle's operator-by-operator expression, and the result against the oracle."""
    from vqtree_amd.ops.attn_vq import apply_rope, rope_tables

    print(f"decode with the rotary folded in: {dtype} B{B} H{H} N{N} D{D} M{M}", flush=True)
    case = decode_case(B, H, N, D, M, device="cuda", seed=33, dtype=dtype)
    pos = 257
    cos, sin = rope_tables(D, 400, dtype=dtype, device="cuda")
    q_rot = apply_rope(case.q, cos, sin, pos)
    want_rot = oracle.apply_rope(case.q.cpu(), cos.cpu(), sin.cpu(), pos)
    assert torch.equal(q_rot.cpu(), want_rot)
    ref, ref_lse = attn_vq_decode(q_rot, case.codes, case.codebooks, case.v, return_lse=True)
    got, got_lse = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, return_lse=True, rope=(cos[pos], sin[pos]))
    torch.cuda.synchronize()
    assert torch.equal(got, ref) and torch.equal(got_lse, ref_lse)
    want, want_lse = oracle.attn_vq_decode(want_rot, case.codes.cpu(), case.codebooks.cpu(), case.v.cpu(),
                                           case.softmax_scale)
    assert_close_16(got, want, "decode with the rotary folded in")
    assert_close_lse(got_lse, want_lse)
    # with the key count in device memory (the recorded-step form)
    n_sub = N - N // 3
    n_dev = torch.tensor([n_sub], dtype=torch.int32, device="cuda")
    got2 = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, rope=(cos[pos], sin[pos]), n_keys=n_dev)
    ref2 = attn_vq_decode(q_rot, case.codes[:, :, :n_sub], case.codebooks, case.v[:, :, :n_sub])
    assert (got2.float() - ref2.float()).abs().max() <= 2e-3


# ------------------------------------------------------------------ exact-key decode
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D", [(2, 3, 1000, 128), (1, 2, 1, 128), (1, 1, 63, 64), (2, 2, 64, 128), (1, 2, 65, 64),
                                     (1, 4, 4097, 128), (3, 1, 300, 64)])
def test_exact_decode_matches_dense_softmax(dtype, B, H, N, D):
    from vqtree_amd.ops.attn_vq import attn_exact_decode

    print(f"exact decode: {dtype} B{B} H{H} N{N} D{D}", flush=True)
    g = torch.Generator("cpu").manual_seed(21)
    q = torch.randn(B, H, 1, D, generator=g).to(dtype)
    k = torch.randn(B, N, H, D, generator=g).to(dtype).transpose(1, 2)  # strided [B,H,N,D] view
    v = torch.randn(B, H, N, D, generator=g).to(dtype)
    scale = 1.0 / math.sqrt(D)
    want, want_lse = oracle.attend(q.float() @ k.float().transpose(-1, -2) * scale,
                                   torch.ones(1, N, dtype=torch.bool), v.float())
    out, lse = attn_exact_decode(q.cuda(), k.cuda(), v.cuda(), return_lse=True)
    assert_close_16(out.cpu(), want, "exact decode")
    assert_close_lse(lse.cpu()[..., 0], want_lse[..., 0])
    for splits in (1, 3, 7):
        o2 = attn_exact_decode(q.cuda(), k.cuda(), v.cuda(), num_splits=splits)
        assert_close_16(o2.cpu(), want, f"exact decode, {splits} splits")


def test_hybrid_decode_state_merge():
    """Far keys through their codes, the last `W` keys exactly, merged by log-sum-exp: equals dense attention over
    [reconstructed far keys ; exact window keys]."""
    from vqtree_amd.ops.attn_vq import attn_vq_decode_windowed

    B, H, N, D, M, W = 2, 4, 900, 128, 4, 200
    case = decode_case(B, H, N, D, M, device="cuda", seed=22)
    g = torch.Generator("cpu").manual_seed(23)
    k_win = torch.randn(B, H, W, D, generator=g).bfloat16().cuda()
    far = N - W
    merged, lse = attn_vq_decode_windowed(case.q, case.codes, case.codebooks, case.v, k_win, return_lse=True)
    k_hat = oracle.reconstruct_keys(case.codes[:, :, :far].cpu(), case.codebooks.cpu())
    keys = torch.cat([k_hat, k_win.float().cpu()], dim=2)
    scores = case.q.float().cpu() @ keys.transpose(-1, -2) * case.softmax_scale
    want, want_lse = oracle.attend(scores, torch.ones(1, N, dtype=torch.bool), case.v.float().cpu())
    assert_close_16(merged.cpu(), want, "hybrid decode")
    assert_close_lse(lse.cpu()[..., 0], want_lse[..., 0], atol=1e-2)
    # the window may cover everything (no coded keys), and may use its own query
    g2 = torch.Generator("cpu").manual_seed(24)
    k_all = torch.randn(B, H, N, D, generator=g2).bfloat16().cuda()
    q_w = torch.randn(B, H, 1, D, generator=g2).bfloat16().cuda()
    full = attn_vq_decode_windowed(case.q, case.codes, case.codebooks, case.v, k_all, q_window=q_w)
    sc = q_w.float().cpu() @ k_all.float().cpu().transpose(-1, -2) * case.softmax_scale
    want_full, _ = oracle.attend(sc, torch.ones(1, N, dtype=torch.bool), case.v.float().cpu())
    assert_close_16(full.cpu(), want_full, "window covers every key")
    mixed = attn_vq_decode_windowed(case.q, case.codes, case.codebooks, case.v, k_win, q_window=q_w)
    s_mixed = torch.cat([case.q.float().cpu() @ k_hat.transpose(-1, -2),
                         q_w.float().cpu() @ k_win.float().cpu().transpose(-1, -2)], dim=-1) * case.softmax_scale
    want_mixed, _ = oracle.attend(s_mixed, torch.ones(1, N, dtype=torch.bool), case.v.float().cpu())
    assert_close_16(mixed.cpu(), want_mixed, "separate window query")


def test_decode_with_device_side_key_count_and_graph_replay():
    """The key count read from device memory equals slicing the cache on the host, eagerly and inside a HIP graph that
    is recorded once and replayed for growing counts (with eager work and synchronisations between the replays)."""
    B, H, N_max, D, M = 2, 4, 3000, 128, 4
    case = decode_case(B, H, N_max, D, M, device="cuda", seed=31)
    n_dev = torch.zeros(1, dtype=torch.int32, device="cuda")
    lib_splits = 6
    counts = [1, 63, 64, 257, 1024, 2999, 3000]
    eager = {}
    for n in counts:
        eager[n] = attn_vq_decode(case.q, case.codes[:, :, :n], case.codebooks, case.v[:, :, :n], num_splits=lib_splits)
        n_dev.fill_(n)
        got = attn_vq_decode(case.q, case.codes, case.codebooks, case.v, num_splits=lib_splits, n_keys=n_dev)
        assert_close_16(got.cpu(), eager[n].float().cpu(), f"device-side count {n}")
    # a count beyond the capacity is clamped; zero keys give a zero row
    n_dev.fill_(10 ** 6)
    assert torch.equal(attn_vq_decode(case.q, case.codes, case.codebooks, case.v, num_splits=lib_splits, n_keys=n_dev),
                       attn_vq_decode(case.q, case.codes, case.codebooks, case.v, num_splits=lib_splits))
    n_dev.fill_(0)
    assert not attn_vq_decode(case.q, case.codes, case.codebooks, case.v, num_splits=lib_splits, n_keys=n_dev).any()

    from vqtree_amd import _lib
    out = torch.empty_like(case.q)
    ws = torch.empty(_lib.load().vqa_decode_workspace_bytes(B, H, N_max, D, M, 256, lib_splits), dtype=torch.uint8,
                     device="cuda")
    n_dev.fill_(counts[0])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream before recording
        attn_vq_decode(case.q, case.codes, case.codebooks, case.v, num_splits=lib_splits, n_keys=n_dev, out=out,
                       workspace=ws)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        attn_vq_decode(case.q, case.codes, case.codebooks, case.v, num_splits=lib_splits, n_keys=n_dev, out=out,
                       workspace=ws)
    for round_ in range(2):
        for n in counts:
            n_dev.fill_(n)
            graph.replay()
            torch.cuda.synchronize()
            assert_close_16(out.cpu(), eager[n].float().cpu(), f"graph replay, count {n}, round {round_}")
            _ = (case.v[:, :, :64].float().sum(), torch.cuda.synchronize())  # unrelated eager work between replays
