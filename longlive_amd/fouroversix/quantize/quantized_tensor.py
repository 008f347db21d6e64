"""QuantizedTensor: packed e2m1 values + blocked e4m3 scales + tensor amax
(mirror of fouroversix/src/fouroversix/quantize/quantized_tensor.py:57-246)."""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ... import _native
from ..utils import DataType, ScaleRule
from .utils import from_blocked, to_blocked  # noqa: F401  (from_blocked is imported from here by LongLive)


class QuantizedTensor:
    """NVFP4 tensor.

    ``values`` u8 [Mp, Kp/2] (low nibble = even column), ``scale_factors`` float8_e4m3fn, 1-D in
    blocked order (2-D row-major scales are padded and blocked on construction), ``amax`` f32.
    ``padded_shape`` = ``original_shape`` rounded up to multiples of (128, 64).
    """

    def __init__(self, values, scale_factors, amax, dtype, original_shape, scale_rule, padded_shape=None) -> None:
        if isinstance(dtype, str):
            dtype = DataType(dtype)
        if isinstance(scale_rule, str):
            scale_rule = ScaleRule(scale_rule)
        original_shape = tuple(int(v) for v in original_shape)
        if padded_shape is not None:
            padded_shape = tuple(int(v) for v in padded_shape)
        if dtype != DataType.nvfp4:
            raise ValueError(f"only {DataType.nvfp4} tensors are supported, got {dtype}")
        self.dtype = dtype
        self.original_shape = original_shape
        self.scale_rule = scale_rule
        self.padded_shape = padded_shape

        if self.padded_shape is None:
            block = dtype.block_size()
            self.padded_shape = _native.padded_shape(original_shape)
            n_packed = self.padded_shape[0] * self.padded_shape[1] // 2
            n_scales = n_packed * 2 // block
            if values.numel() != n_packed:
                values = F.pad(values, (0, self.padded_shape[1] // 2 - values.shape[1],
                                        0, self.padded_shape[0] - values.shape[0]))
            if scale_factors.ndim > 1:  # row-major 2-D scales: pad with zeros, then block
                sf = scale_factors.view(torch.uint8) if scale_factors.dtype != torch.uint8 else scale_factors
                if sf.numel() != n_scales:
                    sf = F.pad(sf, (0, self.padded_shape[1] // block - sf.shape[1],
                                    0, self.padded_shape[0] - sf.shape[0]))
                scale_factors = to_blocked(sf).contiguous().view(torch.float8_e4m3fn)
            if values.numel() != n_packed:
                raise ValueError(f"Expected {n_packed} e2m1 values, got {values.numel()}")
            if scale_factors.numel() != n_scales:
                raise ValueError(f"Expected {n_scales} scale factors, got {scale_factors.numel()}")
        self.values = values
        self.scale_factors = scale_factors
        self.amax = amax

    def dequantize(self, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        """``((e2m1 * e4m3) * amax) / (e2m1_max * e4m3_max)`` cast to ``dtype``, sliced to the
        original shape (HIP kernel)."""
        return _native.dequantize(self.values, self.scale_factors, self.amax, self.scale_rule.value,
                                  self.padded_shape, self.original_shape, dtype)

    # the reference also exposes the Triton variant under this name
    dequantize_triton = dequantize

    @property
    def device(self) -> torch.device:
        return self.values.device

    def __repr__(self) -> str:
        return (f"QuantizedTensor(shape={self.original_shape}, padded={self.padded_shape}, "
                f"rule={self.scale_rule.value}, device={self.values.device})")
