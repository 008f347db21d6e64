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


def hardware_convert(x: torch.Tensor, mode: int) -> torch.Tensor:
    """fp32 -> e4m3 byte (mode 0) or e2m1 nibble (mode 1) with the gfx950 conversion instructions, through the
    test-only library built next to the product library (longlive_amd/csrc/test_hooks.hip)."""
    import ctypes
    import os

    from longlive_amd import _native

    path = os.path.join(os.path.dirname(_native.LIB_PATH), "libll_nvfp4_testhooks.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: run `make -C longlive_amd/csrc`")
    lib = ctypes.CDLL(path)
    lib.ll_test_convert.restype = ctypes.c_int
    lib.ll_test_convert.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    x = x.contiguous().float()
    out = torch.empty(x.numel(), dtype=torch.uint8, device=x.device)
    code = lib.ll_test_convert(x.data_ptr(), x.numel(), mode, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    if code != 0:
        raise RuntimeError(f"ll_test_convert failed with {code}")
    return out
