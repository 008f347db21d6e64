"""Drop-in mirror of the reference's ``fouroversix`` package surface
(fouroversix/src/fouroversix/__init__.py:3-33) backed by the gfx950 kernels."""
from . import utils  # noqa: F401
from .matmul import fp4_matmul
from .model import (FourOverSixLinear, ModelQuantizationConfig, ModuleQuantizationConfig, QuantizedModule,
                    quantize_model)
from .quantize import QuantizationConfig, QuantizedTensor, quantize_to_fp4
from .utils import DataType, MatmulBackend, QuantizeBackend, RoundStyle, ScaleRule

__version__ = "0.1.0+gfx950"

__all__ = [
    "DataType", "FourOverSixLinear", "MatmulBackend", "ModelQuantizationConfig", "ModuleQuantizationConfig",
    "QuantizationConfig", "QuantizeBackend", "QuantizedModule", "QuantizedTensor", "RoundStyle", "ScaleRule",
    "fp4_matmul", "quantize_model", "quantize_to_fp4",
]
