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
