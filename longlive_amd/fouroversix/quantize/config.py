"""QuantizationConfig (mirror of fouroversix/src/fouroversix/quantize/config.py:7-50)."""
from __future__ import annotations

from dataclasses import dataclass

from ..utils import DataType, QuantizeBackend, RoundStyle, ScaleRule


@dataclass
class QuantizationConfig:
    """Options of :func:`quantize_to_fp4`.  Defaults: NVFP4, nearest rounding, four-over-six with
    the mse rule, 1-D block scaling.  ``rht``, ``block_scale_2d``, ``transpose``, stochastic
    rounding and MXFP4 are training features and are rejected by the front end."""

    backend: QuantizeBackend | None = None
    block_scale_2d: bool = False
    dtype: DataType = DataType.nvfp4
    rht: bool = False
    round_style: RoundStyle = RoundStyle.nearest
    scale_rule: ScaleRule = ScaleRule.mse
    transpose: bool = False

    def __post_init__(self) -> None:
        if isinstance(self.backend, str):
            self.backend = QuantizeBackend(self.backend)
        if isinstance(self.dtype, str):
            self.dtype = DataType(self.dtype)
        if isinstance(self.round_style, str):
            self.round_style = RoundStyle(self.round_style)
        if isinstance(self.scale_rule, str):
            self.scale_rule = ScaleRule(self.scale_rule)
