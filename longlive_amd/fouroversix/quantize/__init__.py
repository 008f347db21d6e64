from .config import QuantizationConfig
from .frontend import quantize_to_fp4
from .quantized_tensor import QuantizedTensor
from . import quantized_tensor, utils  # noqa: F401

__all__ = ["QuantizationConfig", "QuantizedTensor", "quantize_to_fp4"]
