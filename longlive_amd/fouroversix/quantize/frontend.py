"""quantize_to_fp4 front end (mirror of fouroversix/src/fouroversix/quantize/frontend.py:19-122).

The reference picks among CUDA / Triton / PyTorch back ends; here every request is served by the
gfx950 HIP quantizer, and requests it does not implement raise ``ValueError`` exactly where the
reference raises when no back end supports the parameters."""
from __future__ import annotations

import torch

from ... import _native
from ..utils import DataType, RoundStyle
from .config import QuantizationConfig
from .quantized_tensor import QuantizedTensor


def _unsupported(x: torch.Tensor, config: QuantizationConfig) -> str | None:
    if x.ndim != 2:
        return "input must be 2-D"
    if config.dtype != DataType.nvfp4:
        return f"dtype {config.dtype.value} (NVFP4 only)"
    if config.round_style != RoundStyle.nearest:
        return "stochastic rounding"
    if config.rht:
        return "random Hadamard transform"
    if config.block_scale_2d:
        return "2-D block scaling"
    if config.transpose:
        return "transposed output"
    return None


def quantize_to_fp4(x: torch.Tensor, config: QuantizationConfig | None = None, *,
                    amax=None) -> QuantizedTensor:
    """Quantize a 2-D bfloat16 GPU tensor to NVFP4.

    Default configuration: block 16 along the last axis, e4m3 block scales, fp32 tensor amax,
    round-to-nearest, four-over-six selection with the mse rule.  The packed bytes equal those of
    the reference's PyTorch back end.  ``amax`` (an extension) is the amax ticket (``_native.amax_ticket``)
    that the kernel which produced ``x`` was given; the reduction pass over ``x`` is then skipped.
    """
    if config is None:
        config = QuantizationConfig()
    why = _unsupported(x, config)
    if why is not None:
        backend = config.backend.value if config.backend is not None else "hip"
        raise ValueError(f"Backend {backend} does not support the given parameters: {why}")
    values, scales, amax = _native.quantize(x, config.scale_rule.value, amax=amax)
    return QuantizedTensor(values, scales, amax, config.dtype, tuple(x.shape), config.scale_rule,
                           _native.padded_shape(tuple(x.shape)))
