"""Seeded synthetic inputs for the benchmark configurations of the VQ-attention path.

Small cases are drawn on the CPU (fp32, `torch.Generator('cpu')`), cast, then copied to the device, so a CPU
checker and the GPU kernels see identical bits.  The full-size decode case draws directly on the device (its V
tensor alone is 4 GiB); a checker copies the (batch, head) units it wants back to the host.
"""
import math
from dataclasses import dataclass

import torch


@dataclass
class DecodeCase:
    q: torch.Tensor          # [B,H,1,D]
    codes: torch.Tensor      # [B,H,N,M] uint8
    codebooks: torch.Tensor  # [H,M,K,D]
    v: torch.Tensor          # [B,H,N,D]
    softmax_scale: float

    @property
    def algorithmic_bytes(self) -> int:
        """codes + V + codebooks + q + out, each touched once per decode step."""
        e = self.q.element_size()
        return (
            self.codes.numel()
            + self.v.numel() * e
            + self.codebooks.numel() * e
            + 2 * self.q.numel() * e
        )


def decode_case(B, H, N, D, M, K=256, dtype=torch.bfloat16, device="cuda", seed=2, cb_std=0.35, on_device=False):
    """q, V ~ N(0,1); codebooks ~ N(0, cb_std); codes uniform in [0,K)."""
    if on_device:
        g = torch.Generator(device=device).manual_seed(seed)
        q = torch.randn(B, H, 1, D, generator=g, device=device, dtype=torch.float32).to(dtype)
        codebooks = (torch.randn(H, M, K, D, generator=g, device=device, dtype=torch.float32) * cb_std).to(dtype)
        codes = torch.randint(0, K, (B, H, N, M), generator=g, device=device, dtype=torch.uint8)
        v = torch.empty(B, H, N, D, device=device, dtype=dtype)
        for b in range(B):  # per-batch draws keep the fp32 staging buffer small
            v[b] = torch.randn(H, N, D, generator=g, device=device, dtype=torch.float32).to(dtype)
    else:
        g = torch.Generator("cpu").manual_seed(seed)
        q = torch.randn(B, H, 1, D, generator=g).to(dtype).to(device)
        codebooks = (torch.randn(H, M, K, D, generator=g) * cb_std).to(dtype).to(device)
        codes = torch.randint(0, K, (B, H, N, M), generator=g, dtype=torch.int32).to(torch.uint8).to(device)
        v = torch.randn(B, H, N, D, generator=g).to(dtype).to(device)
    return DecodeCase(q, codes, codebooks, v, 1.0 / math.sqrt(D))


def decode_c2(device="cuda"):
    """Decode benchmark: batch 16, 32 heads, head_dim 128, 32768 keys, 4 codebooks x 256 codewords, bf16."""
    return decode_case(16, 32, 32768, 128, 4, 256, torch.bfloat16, device, seed=2, cb_std=0.35, on_device=True)


@dataclass
class PrefillCase:
    q: torch.Tensor          # [B,H,N,D]
    k_exact: torch.Tensor    # [B,H,N,D] exact keys of the sliding window
    v: torch.Tensor          # [B,H,N,D]
    codes: torch.Tensor      # [B,H,N,M] uint8
    codebooks: torch.Tensor  # [H,M,K,D]
    window: int
    softmax_scale: float

    def algorithmic_flops(self, boundary_mode="block") -> int:
        """LUT (2*N*M*K*D) + exact QK^T (2*D*P_exact) + P.V (2*D*(P_exact + P_far)) per (batch, head), pairs counted
        from the mask: P_far = sum_i boundary(i), P_exact = sum_i (i + 1 - boundary(i))."""
        B, H, N, D = self.q.shape
        M, K = self.codes.shape[3], self.codebooks.shape[2]
        i = torch.arange(N, dtype=torch.int64)
        if boundary_mode == "block":
            bnd = torch.clamp(torch.div(i - self.window, 128, rounding_mode="floor") * 128, min=0)
        else:
            bnd = torch.clamp(i - self.window, min=0)
        p_far = int(bnd.sum())
        p_exact = int((i + 1 - bnd).sum())
        per_head = 2 * N * M * K * D + 2 * D * p_exact + 2 * D * (p_exact + p_far)
        return B * H * per_head


def prefill_case(B, H, N, D, M, W, K=256, dtype=torch.bfloat16, device="cuda", seed=3, cb_std=0.35, on_device=False):
    """q, k_exact, V ~ N(0,1); codebooks ~ N(0, cb_std); codes uniform in [0,K)."""
    if on_device:
        g = torch.Generator(device=device).manual_seed(seed)
        mk = lambda *s: torch.randn(*s, generator=g, device=device, dtype=torch.float32)
        q, k, v = mk(B, H, N, D).to(dtype), mk(B, H, N, D).to(dtype), mk(B, H, N, D).to(dtype)
        cb = (mk(H, M, K, D) * cb_std).to(dtype)
        codes = torch.randint(0, K, (B, H, N, M), generator=g, device=device, dtype=torch.uint8)
    else:
        g = torch.Generator("cpu").manual_seed(seed)
        mk = lambda *s: torch.randn(*s, generator=g)
        q, k, v = (mk(B, H, N, D).to(dtype).to(device) for _ in range(3))
        cb = (mk(H, M, K, D) * cb_std).to(dtype).to(device)
        codes = torch.randint(0, K, (B, H, N, M), generator=g, dtype=torch.int32).to(torch.uint8).to(device)
    return PrefillCase(q, k, v, codes, cb, W, 1.0 / math.sqrt(D))


def prefill_c3(device="cuda"):
    """Prefill benchmark, Llama-2-7B shape: batch 1, 32 heads, head_dim 128, 8192 tokens, exact window 1024,
    4 codebooks x 256 codewords, bf16 (codebook std 0.35, not fixed by the configuration)."""
    return prefill_case(1, 32, 8192, 128, 4, 1024, device=device, seed=3, on_device=True)
