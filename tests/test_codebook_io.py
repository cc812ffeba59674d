"""Codebook container (CPU): round trip through the trainers' pickle layout, and refusal of streams that name
anything but numpy arrays."""
import pickle

import numpy as np
import pytest
import torch

from vqtree_amd.codebook_io import load_codebooks, read_codebook_dict, save_codebooks


def test_round_trip_and_layout(tmp_path):
    L, H, M, K, D = 2, 3, 4, 16, 8
    cb = torch.randn(L, H, M, K, D, generator=torch.Generator().manual_seed(0))
    path = tmp_path / "ncb4-bits4-mbsz6-lut1.pkl"
    save_codebooks(path, cb)
    raw = pickle.load(open(path, "rb"))  # written by this test: the plain layout a trainer produces
    assert set(raw) == {(l, h) for l in range(L) for h in range(H)}
    assert len(raw[(1, 2)]) == M and raw[(1, 2)][3].shape == (K, D) and raw[(1, 2)][3].dtype == np.float32
    assert torch.equal(load_codebooks(path, dtype=torch.float32), cb)
    assert torch.equal(load_codebooks(path, dtype=torch.bfloat16), cb.bfloat16())
    assert np.array_equal(read_codebook_dict(path)[(0, 1)][2], cb[0, 1, 2].numpy())


def test_stacked_array_entries_are_accepted(tmp_path):
    # faiss' helper may hand back the M codebooks of one quantiser as a single (M, K, D) array
    table = {(0, h): np.arange(2 * 4 * 3, dtype=np.float32).reshape(2, 4, 3) + h for h in range(2)}
    path = tmp_path / "stacked.pkl"
    pickle.dump(table, open(path, "wb"))
    out = load_codebooks(path, dtype=torch.float32)
    assert out.shape == (1, 2, 2, 4, 3) and out[0, 1, 1, 2, 0] == 1 + 12 + 6


class _Boom:
    def __reduce__(self):
        return (print, ("must never run",))


def test_foreign_globals_are_refused(tmp_path, capsys):
    path = tmp_path / "bad.pkl"
    pickle.dump({(0, 0): [_Boom()]}, open(path, "wb"))
    with pytest.raises(pickle.UnpicklingError):
        load_codebooks(path)
    assert "must never run" not in capsys.readouterr().out


def test_incomplete_grid_is_refused(tmp_path):
    path = tmp_path / "holes.pkl"
    pickle.dump({(0, 0): [np.zeros((4, 2), np.float32)], (1, 1): [np.zeros((4, 2), np.float32)]}, open(path, "wb"))
    with pytest.raises(ValueError):
        load_codebooks(path)
