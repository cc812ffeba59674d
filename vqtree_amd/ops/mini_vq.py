"""Runtime key encoders.  `multi_head_single_quantize` is the counterpart of ops/mini_vq.py:4-18 (one codebook per
head, inner-product search); `encode_keys` is the general entry: inner-product or greedy residual (additive) search
against [H,M,K,D] codebooks.  16-bit inputs run the HIP encoder (matrix cores, fp32 scores); fp32 inputs, which only
the fp32 validation configuration uses, are scored with a torch einsum on the device."""
import torch

from .. import _lib
from ._common import SUFFIX, bhn_strides, ptr

INNER_PRODUCT, RESIDUAL = 0, 1


def encode_keys(x, codebooks, mode=RESIDUAL, round_scores=False, want_codes=True, want_ids=False):
    """x [B,H,N,D]; codebooks [H,M,K,D].  Returns (codes [B,H,N,M] uint8 or None, ids [B,H,N,M] int64 or None).

    mode INNER_PRODUCT: id_m = argmax_c <x, cb[h,m,c]> per codebook; RESIDUAL: greedy nearest codeword (L2) of the
    running residual.  `round_scores` rounds scores to the input dtype before the comparison (inner-product mode),
    which is what an einsum evaluated in the model dtype compares."""
    B, H, N, D = x.shape
    Hc, M, K, Dc = codebooks.shape
    assert (Hc, Dc) == (H, D) and x.dtype == codebooks.dtype
    _lib.require_gpu(x, codebooks)
    if x.dtype not in SUFFIX:
        return _encode_keys_torch(x, codebooks, mode, want_codes, want_ids)
    lib = _lib.load()
    x = x if x.stride(-1) == 1 else x.contiguous()
    codebooks = codebooks if codebooks.stride(-1) == 1 else codebooks.contiguous()
    codes = torch.empty((B, H, N, M), dtype=torch.uint8, device=x.device) if want_codes else None
    ids = torch.empty((B, H, N, M), dtype=torch.int64, device=x.device) if want_ids else None
    strides = _lib.strides_array(*bhn_strides(x), codebooks.stride(0), codebooks.stride(1), codebooks.stride(2),
                                 *(bhn_strides(codes) if want_codes else (0, 0, 0)),
                                 *(bhn_strides(ids) if want_ids else (0, 0, 0)))
    with torch.cuda.device(x.device):
        rc = getattr(lib, "vqa_encode_keys_" + SUFFIX[x.dtype])(ptr(x), ptr(codebooks), ptr(codes), ptr(ids), B, H, N,
                                                                 D, M, K, strides, int(mode), int(bool(round_scores)),
                                                                 _lib.current_stream(x.device))
    _lib.check(rc)
    return codes, ids


def _encode_keys_torch(x, codebooks, mode, want_codes, want_ids):
    r = x
    out = []
    for m in range(codebooks.shape[1]):
        cb = codebooks[:, m]
        score = torch.einsum("bhnd,hkd->bhnk", r, cb)
        if mode == RESIDUAL:
            score = score - 0.5 * (cb * cb).sum(-1)[None, :, None, :]
        idx = score.argmax(-1)
        out.append(idx)
        if mode == RESIDUAL:
            r = r - cb.unsqueeze(0).expand(x.shape[0], -1, -1, -1).gather(
                2, idx.unsqueeze(-1).expand(-1, -1, -1, x.shape[-1]))
    ids = torch.stack(out, dim=-1)
    return (ids.to(torch.uint8) if want_codes else None), (ids if want_ids else None)


def quantize_ids(inp, codebook):
    """ids [B,H,N] int64 of the inner-product search against one codebook per head [H,C,D]."""
    _, ids = encode_keys(inp, codebook.unsqueeze(1), INNER_PRODUCT, round_scores=True, want_codes=False, want_ids=True)
    return ids[..., 0]


def multi_head_single_quantize(inp: torch.Tensor, codebook: torch.Tensor):
    """inp: batch x head x seqlen x d_hidden; codebook: head x codebook_size x d_hidden.

    code id = argmax_c <inp, codebook[h, c]> (inner product; first maximum on ties).
    Returns (quantised input [B,H,N,D], ids [B,H,N] int64, one-hot [B,H,N,C] int64).
    """
    B, H, N, D = inp.shape
    ids = quantize_ids(inp, codebook)
    quantized = codebook.unsqueeze(0).expand(B, -1, -1, -1).gather(2, ids.unsqueeze(-1).expand(-1, -1, -1, D))
    onehot = torch.nn.functional.one_hot(ids, codebook.shape[1])
    return quantized, ids, onehot
