"""Shared helpers of the test-suite: bf16 bit views and the benchmark input distributions."""
import numpy as np
import torch


def bits_of(t: torch.Tensor) -> np.ndarray:
    """bf16 torch tensor -> uint16 numpy bit pattern."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def from_bits(b: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16).to(device)


def f32_of(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def activations(shape, seed, outliers=True) -> torch.Tensor:
    """N(0,1) with 0.1 % of entries scaled x20 (the benchmark's activation distribution), bf16."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g)
    if outliers:
        mask = torch.rand(shape, generator=g) < 1e-3
        x = torch.where(mask, x * 20, x)
    return x.bfloat16()


def weights(shape, seed) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * 0.02).bfloat16()


def u8(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy().copy()
