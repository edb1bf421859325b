from .config import ModelQuantizationConfig, ModuleQuantizationConfig
from .linear import FourOverSixLinear, fp4_linear
from .quantize import QuantizedModule, quantize_model

__all__ = [
    "FourOverSixLinear",
    "ModelQuantizationConfig",
    "ModuleQuantizationConfig",
    "QuantizedModule",
    "fp4_linear",
    "quantize_model",
]
