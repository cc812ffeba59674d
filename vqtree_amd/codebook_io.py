"""On-disk format of trained additive codebooks: a pickle of `{(layer, head): [M arrays of shape (2**bits, D), float32]}`
as the reference's offline trainers write it (build_quantizer/120_build_additive_quantizer.py:51-66; the sphere variant,
trained on L2-normalised keys, uses the same container: build_quantizer/121_build_sphere_additive_quantizer.py:46,64).

Reading goes through an unpickler that resolves only the handful of numpy globals an ndarray needs, so a file cannot
run code; anything else in the stream raises `pickle.UnpicklingError`."""
import pickle

import numpy as np
import torch

_ALLOWED = {
    ("numpy.core.multiarray", "_reconstruct"),
    ("numpy._core.multiarray", "_reconstruct"),
    ("numpy", "ndarray"),
    ("numpy", "dtype"),
}


class _ArrayOnlyUnpickler(pickle.Unpickler):
    def find_class(self, module, name):
        if (module, name) in _ALLOWED:
            return super().find_class(module, name)
        raise pickle.UnpicklingError(f"codebook file names {module}.{name}: only numpy arrays are accepted")


def read_codebook_dict(path):
    """{(layer, head): [M x ndarray(K, D) float32]} exactly as stored."""
    with open(path, "rb") as f:
        table = _ArrayOnlyUnpickler(f).load()
    if not isinstance(table, dict) or not table:
        raise ValueError("codebook file does not hold a non-empty {(layer, head): [arrays]} dictionary")
    for key, books in table.items():
        if not (isinstance(key, tuple) and len(key) == 2 and all(isinstance(i, (int, np.integer)) for i in key)):
            raise ValueError(f"bad key {key!r}: expected (layer, head)")
        if isinstance(books, np.ndarray) and books.ndim == 3:
            continue
        if not (isinstance(books, (list, tuple)) and all(isinstance(a, np.ndarray) and a.ndim == 2 for a in books)):
            raise ValueError(f"entry {key!r} is not a list of (K, D) arrays")
    return table


def load_codebooks(path, dtype=torch.bfloat16, device="cpu"):
    """Tensor [L, H, M, K, D] (layers and heads in index order) in `dtype` on `device`; `[layer]` is the [H,M,K,D]
    operand of the attention entry points."""
    table = read_codebook_dict(path)
    layers = sorted({int(k[0]) for k in table})
    heads = sorted({int(k[1]) for k in table})
    if layers != list(range(len(layers))) or heads != list(range(len(heads))) or len(table) != len(layers) * len(heads):
        raise ValueError("codebook file does not cover a full (layer, head) grid")
    first = np.stack(list(table[(0, 0)]))
    out = np.empty((len(layers), len(heads)) + first.shape, dtype=np.float32)
    for (layer, head), books in table.items():
        arr = np.stack(list(books))
        if arr.shape != first.shape:
            raise ValueError(f"entry {(layer, head)} has shape {arr.shape}, expected {first.shape}")
        out[int(layer), int(head)] = arr
    return torch.from_numpy(out).to(dtype).to(device)


def save_codebooks(path, codebooks):
    """Write a [L, H, M, K, D] tensor in the trainers' container."""
    cb = codebooks.detach().float().cpu().numpy()
    table = {(layer, head): [np.ascontiguousarray(cb[layer, head, m]) for m in range(cb.shape[2])]
             for layer in range(cb.shape[0]) for head in range(cb.shape[1])}
    with open(path, "wb") as f:
        pickle.dump(table, f)
