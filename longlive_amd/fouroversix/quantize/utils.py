"""Scale-factor layout helpers (mirror of fouroversix/src/fouroversix/quantize/utils.py:88-96 and
quantize/quantized_tensor.py:10-18).  Pure index shuffles on whatever device the tensor lives on."""
from __future__ import annotations

import torch


def to_blocked(a: torch.Tensor) -> torch.Tensor:
    """[rows, cols] (rows % 128 == 0, cols % 4 == 0) -> 1-D in 128x4-tile blocked order."""
    rows, cols = a.shape
    return (
        a.reshape(rows // 128, 4, 32, cols // 4, 4)  # (rb, r/32, r%32, cb, c)
        .permute(0, 3, 2, 1, 4)                      # (rb, cb, r%32, r/32, c)
        .reshape(-1)
    )


def from_blocked(a: torch.Tensor, orig_shape: tuple[int, int]) -> torch.Tensor:
    """Inverse of :func:`to_blocked`."""
    rows, cols = orig_shape
    return (
        a.reshape(rows // 128, cols // 4, 32, 4, 4)  # (rb, cb, r%32, r/32, c)
        .permute(0, 3, 2, 1, 4)                      # (rb, r/32, r%32, cb, c)
        .reshape(rows, cols)
    )
