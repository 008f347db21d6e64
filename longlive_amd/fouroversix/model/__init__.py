from .config import ModelQuantizationConfig, ModuleQuantizationConfig
from .modules import FourOverSixLinear
from .quantize import QuantizedModule, quantize_model
from . import config, modules, quantize  # noqa: F401

__all__ = ["FourOverSixLinear", "ModelQuantizationConfig", "ModuleQuantizationConfig", "QuantizedModule",
           "quantize_model"]
