"""Seeded synthetic inputs of the benchmark configurations and bf16 <-> numpy helpers for tests."""
from __future__ import annotations

import numpy as np
import torch

GROUP = 128


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> numpy uint16 bit patterns (CPU copy)."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(a: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16).to(device)


def pack_codes(codes: torch.Tensor) -> torch.Tensor:
    """uint8 codes [..] (0..15) -> native int8 bytes, even index in the high nibble."""
    c = codes.reshape(-1, 2).to(torch.uint8)
    return ((c[:, 0] << 4) | c[:, 1]).view(torch.int8).contiguous()


def make_w4(N, K, seed, zero_lo=6, zero_hi=9):
    """Codes U{0..15}, scales |N(0,0.02)|/7 (bf16), zeros U{zero_lo..zero_hi} (bf16)."""
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    scales = (torch.randn(N * K // GROUP, 1, generator=g) * 0.02).abs().div(7).to(torch.bfloat16)
    scales = torch.where(scales == 0, torch.full_like(scales, 2.0 ** -10), scales)
    zeros = torch.randint(zero_lo, zero_hi + 1, (N * K // GROUP, 1), generator=g).to(torch.bfloat16)
    return codes, pack_codes(codes), scales, zeros


def randn_bf16(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(torch.bfloat16)


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.double().reshape(-1)
    b = b.double().reshape(-1)
    return float((a - b).norm() / b.norm().clamp_min(1e-300))
