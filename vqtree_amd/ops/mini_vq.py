"""Runtime key encoder with one codebook per head.  Counterpart of ops/mini_vq.py:4-18."""
import torch


def multi_head_single_quantize(inp: torch.Tensor, codebook: torch.Tensor):
    """inp: batch x head x seqlen x d_hidden; codebook: head x codebook_size x d_hidden.

    code id = argmax_c <inp, codebook[h, c]> (inner product; first maximum on ties).
    Returns (quantised input [B,H,N,D], ids [B,H,N] int64, one-hot [B,H,N,C] int64).
    """
    head = inp.shape[1]
    product = torch.einsum("zhqx,hcx->zhqc", inp, codebook)
    ids = product.argmax(-1)
    quantized = torch.stack([codebook[h][ids[:, h]] for h in range(head)], dim=1)
    onehot = torch.nn.functional.one_hot(ids, codebook.shape[1])
    return quantized, ids, onehot
