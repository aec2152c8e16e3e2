"""Shared test helpers (size generators follow the reference's tests/utils.py:17-28)."""

from __future__ import annotations

import random

import numpy as np
import torch


def get_1d_tensor_sizes(log_max_power_of_2: int = 15, max_offset: int = 10, num_not_powers_of_2: int = 50) -> list[int]:
    rng = random.Random(0)
    sizes = set()
    for i in range(log_max_power_of_2):
        for j in range(max_offset):
            sizes.add(2**i + j)
    for _ in range(num_not_powers_of_2):
        sizes.add(3000 + rng.randint(-1000, 1000))
    return sorted(sizes)


def zipf_ids(n: int, num_experts: int, s: float, seed: int, dtype=torch.int32) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    p = torch.arange(1, num_experts + 1, dtype=torch.float64) ** (-s)
    return torch.multinomial(p / p.sum(), n, replacement=True, generator=g).to(dtype)


def nerr(got: torch.Tensor, want: torch.Tensor) -> float:
    """max-abs-normalised error, the measure the 1e-2 bf16 parity bar is stated on"""
    want = want.double().cpu()
    got = got.double().cpu()
    denom = want.abs().max().item()
    err = (got - want).abs().max().item() if want.numel() else 0.0
    return err / denom if denom > 0 else err


def np_of(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu()
    if t.dtype == torch.uint32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.numpy()
