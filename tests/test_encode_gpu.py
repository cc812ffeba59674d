"""GPU tests of the key encoder and of the count-kernel preprocessing, through the C ABI (host wrappers in
vqtree_amd.ops), against the CPU oracle.  Index outputs are integer work: bit-exact wherever the fp32 scores are not
within rounding of a tie; near-ties are accepted only when the chosen codeword's fp32 score equals the best one to
1e-4 relative."""
import pytest
import torch

import oracle
from tests.util import assert_close_16
from vqtree_amd.ops import attn_vq as A
from vqtree_amd.ops import mini_vq as Q

pytestmark = pytest.mark.gpu


def _draw(shape, dtype, seed, std=1.0):
    return (torch.randn(*shape, generator=torch.Generator("cpu").manual_seed(seed)) * std).to(dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D,K", [(2, 3, 300, 128, 256), (1, 2, 130, 64, 512), (2, 2, 1, 128, 128), (1, 1, 129, 64, 32),
                                       (1, 2, 257, 64, 8192), (1, 1, 200, 128, 96)])
def test_inner_product_search(dtype, B, H, N, D, K):
    print(f"encode: inner product {dtype} B{B} H{H} N{N} D{D} K{K}", flush=True)
    x, cb = _draw((B, H, N, D), dtype, 1), _draw((H, 1, K, D), dtype, 2)
    _, ids = Q.encode_keys(x.cuda(), cb.cuda(), Q.INNER_PRODUCT, want_codes=False, want_ids=True)
    ids = ids.cpu()[..., 0]
    score = torch.einsum("bhnd,hkd->bhnk", x.float(), cb[:, 0].float())
    want = score.argmax(-1)
    best = score.amax(-1)
    got = score.gather(-1, ids.unsqueeze(-1))[..., 0]
    assert ids.min() >= 0 and ids.max() < K
    assert (got >= best - 1e-4 * (1 + best.abs())).all()
    assert (ids != want).float().mean() <= 2e-3


def test_inner_product_rounded_scores_follow_the_model_dtype_einsum():
    B, H, N, D, K = 2, 2, 640, 128, 256
    x, cb = _draw((B, H, N, D), torch.bfloat16, 3), _draw((H, K, D), torch.bfloat16, 4)
    quant, ids, onehot = Q.multi_head_single_quantize(x.cuda(), cb.cuda())
    want_q, want_ids, _ = oracle.multi_head_single_quantize(x, cb)
    assert ids.dtype == torch.int64 and ids.shape == (B, H, N) and onehot.shape == (B, H, N, K)
    assert torch.equal(onehot.argmax(-1), ids) and bool(onehot.sum(-1).eq(1).all())
    # bf16 rounding creates many exact ties; the two evaluations may round a score differently by one ulp
    rounded = torch.einsum("bhnd,hkd->bhnk", x.float(), cb.float()).bfloat16().float()
    got = rounded.gather(-1, ids.cpu().unsqueeze(-1))[..., 0]
    assert (got >= rounded.amax(-1) * (1 - 2 ** -7) - 1e-6).all()
    assert (ids.cpu() != want_ids).float().mean() < 2e-2
    for h in range(H):  # the quantised keys are the chosen codebook rows, bit for bit
        assert torch.equal(quant[:, h].cpu(), cb[h][ids[:, h].cpu()])


def test_ties_take_the_first_codeword():
    B, H, N, D, K = 1, 2, 200, 64, 128
    x, cb = _draw((B, H, N, D), torch.bfloat16, 5), _draw((H, 1, K, D), torch.bfloat16, 6)
    cb[:, :, K // 2:] = cb[:, :, : K // 2]  # codeword c + K/2 duplicates c, across the two half-waves and 32-blocks
    for mode in (Q.INNER_PRODUCT, Q.RESIDUAL):
        _, ids = Q.encode_keys(x.cuda(), cb.cuda(), mode, want_codes=False, want_ids=True)
        assert ids.max().item() < K // 2
    zeros = torch.zeros(B, H, N, D, dtype=torch.bfloat16)
    _, ids = Q.encode_keys(zeros.cuda(), cb.cuda(), Q.INNER_PRODUCT, want_codes=False, want_ids=True)
    assert ids.abs().max().item() == 0  # every score is 0: the first codeword wins


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D,M,K", [(2, 2, 300, 128, 4, 256), (1, 3, 129, 64, 2, 256), (4, 2, 1, 128, 4, 256),
                                         (1, 2, 70, 64, 8, 64), (1, 1, 333, 128, 3, 160)])
def test_residual_encoder(dtype, B, H, N, D, M, K):
    print(f"encode: residual {dtype} B{B} H{H} N{N} D{D} M{M} K{K}", flush=True)
    x, cb = _draw((B, H, N, D), dtype, 7), _draw((H, M, K, D), dtype, 8, std=0.6)
    codes, ids = Q.encode_keys(x.cuda(), cb.cuda(), Q.RESIDUAL, want_codes=True, want_ids=True)
    codes, ids = codes.cpu(), ids.cpu()
    assert codes.dtype == torch.uint8 and torch.equal(codes.long(), ids)
    want = oracle.encode_residual(x, cb)
    same = (ids == want).all(-1).float().mean()
    assert same >= 0.995, f"only {same:.4f} of the keys carry the oracle's codes"
    # a key whose codes differ took the other side of a near-tie: its reconstruction error is the same to 1e-3
    err = lambda c: (x.float() - oracle.reconstruct_keys(c, cb)).pow(2).sum(-1)
    e_got, e_want = err(ids), err(want)
    assert (e_got <= e_want * (1 + 1e-3) + 1e-4).all() or ((e_got - e_want).abs() / (1 + e_want)).max() < 5e-2
    assert abs(e_got.mean() - e_want.mean()) <= 1e-3 * e_want.mean()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,C,D", [(2, 2, 640, 128, 64), (1, 3, 1000, 512, 128), (1, 1, 128, 128, 128), (2, 1, 100, 256, 64),
                                       (1, 2, 2049, 4096, 128)])
def test_preprocessing_kernels(dtype, B, H, N, C, D):
    print(f"preprocess: {dtype} B{B} H{H} N{N} C{C} D{D}", flush=True)
    g = torch.Generator("cpu").manual_seed(9)
    ids = torch.randint(0, max(1, C - 3), (B, H, N), generator=g)  # the last codes never occur
    ids[:, :, : N // 2] //= 7  # a skewed half: long segments
    v = _draw((B, H, N, D), dtype, 10)
    cnt, v_vq, vi = A.segmented_preprocess(ids.cuda(), v.cuda(), C, want_int64_counts=True)
    cnt_e, v_vq_e, vi_e = A.segmented_preprocess(ids.cuda(), v.cuda(), C)
    want_cnt, want_vvq, want_vi = oracle.sort_based_preprocess(ids, v, C, dtype=dtype)
    assert cnt.shape == want_cnt.shape and vi.shape == want_vi.shape and v_vq.shape == want_vvq.shape
    assert torch.equal(cnt.cpu(), want_cnt) and torch.equal(vi.cpu(), want_vi)  # integer work: bit-exact
    assert torch.equal(vi_e.cpu(), want_vi) and torch.equal(cnt_e.cpu(), want_cnt.to(dtype))
    assert torch.equal(v_vq.cpu(), v_vq_e.cpu())
    assert bool((v_vq[:, :, 0] == 0).all())
    # running sums of up to thousands of N(0,1) rows, rounded to 16 bits: compare relative to the row magnitude
    diff = (v_vq.float().cpu() - want_vvq.float()).abs()
    assert (diff <= 2e-2 + 1e-2 * want_vvq.float().abs()).all(), diff.max()


def test_linear_prefill_uses_the_hip_preprocessing_consistently():
    """The count-kernel route fed by the HIP preprocessing equals the same route fed by the torch restatement of the
    reference's sort-based preprocessing."""
    B, H, N, D, W, C = 1, 2, 900, 128, 256, 256
    g = torch.Generator("cpu").manual_seed(11)
    q, k, v = (torch.randn(B, H, N, D, generator=g).bfloat16().cuda() for _ in range(3))
    cb = _draw((H, C, D), torch.bfloat16, 12).cuda()
    _, ids, onehot = Q.multi_head_single_quantize(k, cb)
    a = A.sort_based_preprocess(ids, onehot, v)
    b = A.segmented_preprocess(ids, v, C, want_int64_counts=True)
    assert torch.equal(a[0], b[0]) and torch.equal(a[2], b[2])
    assert_close_16(b[1].cpu(), a[1].cpu(), "v_vq")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,N,D", [(2, 3, 257, 128), (1, 2, 100, 64), (1, 1, 7, 16)])
def test_rotary_kernel_is_bit_exact(dtype, B, H, N, D):
    """The rotary kernel against the CPU oracle (the expression evaluated operator by operator on 16-bit tensors):
    bit-exact, for per-row positions, one clamped position, and a strided ([B,N,H,D]-backed) input."""
    print(f"rope: {dtype} B{B} H{H} N{N} D{D}", flush=True)
    x = _draw((B, N, H, D), dtype, 13).transpose(1, 2)  # [B,H,N,D] view of a [B,N,H,D] buffer
    cos, sin = oracle.rope_tables(D, N + 40, dtype=dtype)
    pos = (torch.arange(N)[None, :] + torch.tensor([[3], [17]])[:B]).contiguous()
    got = A.apply_rope(x.cuda(), cos.cuda(), sin.cuda(), pos.cuda()).cpu()
    for b in range(B):
        want = oracle.apply_rope(x[b], cos, sin, pos[b])
        assert torch.equal(got[b], want)
    got_fixed = A.apply_rope(x.cuda(), cos.cuda(), sin.cuda(), 33).cpu()
    assert torch.equal(got_fixed, oracle.apply_rope(x, cos, sin, 33))
    assert torch.equal(A.apply_rope(x.cuda(), cos.cuda(), sin.cuda(), 0).cpu(), x)  # position 0 is the identity
    both = A.apply_rope(x.cuda(), cos.cuda(), sin.cuda(), pos.cuda(), also_fixed=33)  # one pass, two outputs
    assert torch.equal(both[0].cpu(), got) and torch.equal(both[1].cpu(), got_fixed)
