"""Seeded inputs shared by the CPU and GPU tests (the five benchmark
configurations, generated on the CPU so oracle and device see the same bits)."""
from __future__ import annotations

import numpy as np
import torch

TORCH_DT = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}
INT_VIEW = {2: torch.int16, 4: torch.int32}


def uniform(n: int, lo: float, hi: float, seed: int, dtype=torch.float16) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(n, generator=g) * (hi - lo) + lo).to(dtype)


def normal(n: int, seed: int, dtype=torch.float16) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, generator=g).to(dtype)


def rank_rows(world: int, n: int, dt: str, seed0: int = 3000) -> list[torch.Tensor]:
    """Per-rank (world, n) buffers, seed = seed0 + rank, drawn in f32 then cast."""
    return [normal(world * n, seed0 + r, TORCH_DT[dt]).reshape(world, n) for r in range(world)]


def as_bytes(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy().reshape(-1)


def random_bits(n: int, bits: int, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.integers(0, 1 << bits, n, dtype=np.uint64).astype(np.uint16 if bits == 16 else np.uint32)


def special_values_f16() -> np.ndarray:
    """Bit patterns around every boundary of binary16."""
    base = [0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x0401, 0x7BFF, 0xFBFF, 0x7C00,
            0xFC00, 0x3C00, 0xBC00, 0x3C01, 0x6800, 0x6801, 0x3555, 0x0200, 0x8200, 0x7800,
            0x7E00, 0x7C01]
    return np.array(base, dtype=np.uint16)
