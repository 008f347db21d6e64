"""fp4_matmul front end (mirror of fouroversix/src/fouroversix/matmul/frontend.py:14-115)."""
from __future__ import annotations

import torch

from ... import _native
from ..quantize import QuantizationConfig, QuantizedTensor, quantize_to_fp4
from ..utils import DataType, MatmulBackend


def fp4_matmul(
    input: torch.Tensor | QuantizedTensor,
    other: torch.Tensor | QuantizedTensor,
    *,
    backend: MatmulBackend | None = None,
    input_config: QuantizationConfig | None = None,
    other_config: QuantizationConfig | None = None,
    out_dtype: DataType = DataType.bfloat16,
    bias: torch.Tensor | None = None,
    activation: str | None = None,
    residual: torch.Tensor | None = None,
    gate: torch.Tensor | None = None,
    gate_rows: int = 0,
    amax_out=None,
) -> torch.Tensor:
    """``input @ other.T`` of two NVFP4 tensors with fp32 accumulation (W4A4 GEMM).

    High-precision operands are quantized first with ``input_config`` / ``other_config``.
    ``backend`` is accepted for compatibility; the gfx950 kernel always runs.  ``bias`` (bfloat16
    [N], an extension) is added to the bfloat16 result inside the kernel epilogue; ``activation``
    (``"gelu_tanh"``, an extension) is then applied to that bfloat16 value, also in the epilogue.
    ``residual`` (bfloat16 [M, N]) with an optional ``gate`` (bfloat16 [G, N], row ``m // gate_rows``)
    makes the result ``residual + y * gate`` (each step rounded to bfloat16 like the separate
    operations); ``amax_out`` (an amax ticket, ``_native.amax_ticket``) receives the absolute maximum of
    the result.  All of these are extensions.
    """
    if isinstance(backend, str):
        backend = MatmulBackend(backend)
    if isinstance(out_dtype, str):
        out_dtype = DataType(out_dtype)
    if isinstance(input, torch.Tensor):
        input = quantize_to_fp4(input, input_config or QuantizationConfig())
    if isinstance(other, torch.Tensor):
        other = quantize_to_fp4(other, other_config or QuantizationConfig())
    if input.dtype != other.dtype:
        raise ValueError("Both inputs must have the same dtype")
    if input.original_shape[1] != other.original_shape[1]:
        raise ValueError(
            "The first input must be in row-major layout, the second input must be in column-major "
            "layout, and both inputs must have the same inner dimension")
    if out_dtype != DataType.bfloat16:
        raise ValueError(f"Backend hip does not support the given parameters: out_dtype {out_dtype.value}")
    return _native.gemm(
        input.values, input.scale_factors, other.values, other.scale_factors,
        input.original_shape[0], other.original_shape[0],
        amax_a=input.amax, amax_b=other.amax,
        denom_a=float(input.scale_rule.max_allowed_e2m1_value() * input.scale_rule.max_allowed_e4m3_value()),
        denom_b=float(other.scale_rule.max_allowed_e2m1_value() * other.scale_rule.max_allowed_e4m3_value()),
        bias=bias,
        activation=activation,
        residual=residual,
        gate=gate,
        gate_rows=gate_rows,
        amax_out=amax_out,
    )
