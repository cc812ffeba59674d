"""Shared helpers for the GPU parity tests."""
import torch

BF16_ATOL, BF16_RTOL = 2e-2, 1e-2  # 16-bit outputs vs the fp32 oracle
F32_TOL = 1e-4


def assert_close_16(got, want, what=""):
    """|got - want| <= 2e-2 + 1e-2 * |want| element-wise (bf16 / f16 kernels vs fp32 oracle)."""
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - want).abs()
    bound = BF16_ATOL + BF16_RTOL * want.abs()
    bad = err > bound
    assert not bad.any(), f"{what}: {int(bad.sum())} elements out of tolerance, max abs err {float(err.max()):.4g}"
    return float(err.max())


def assert_close_lse(got, want, atol=2e-3, what="lse"):
    got = got.detach().float().cpu()
    want = want.detach().float().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    both_inf = torch.isinf(got) & torch.isinf(want) & (got == want)
    err = torch.where(both_inf, torch.zeros_like(got), (got - want).abs())
    assert not torch.isnan(err).any() and float(err.max()) <= atol, f"{what}: max err {float(err.max()):.4g}"
