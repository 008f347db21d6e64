"""Seeded synthetic tensors of the benchmark configurations: what ``bench.py``, the smoke test and the test suite
feed the kernels (there are no datasets or checkpoints on this path)."""
from __future__ import annotations

import numpy as np
import torch


def activations(shape, seed, outliers=True) -> torch.Tensor:
    """N(0,1) with 0.1 % of entries scaled x20 (the benchmark's activation distribution), bf16, on the CPU."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g)
    if outliers:
        mask = torch.rand(shape, generator=g) < 1e-3
        x = torch.where(mask, x * 20, x)
    return x.bfloat16()


def weights(shape, seed) -> torch.Tensor:
    """N(0, 0.02) weights, bf16, on the CPU."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * 0.02).bfloat16()


def bits_of(t: torch.Tensor) -> np.ndarray:
    """bf16 torch tensor -> uint16 numpy bit pattern."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def u8(t: torch.Tensor) -> np.ndarray:
    """Any one-byte tensor (uint8, float8) -> uint8 numpy array."""
    return t.detach().cpu().contiguous().view(torch.uint8).numpy().copy()
