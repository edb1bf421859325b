"""MI355X (gfx950) implementation of the fouroversix quantize + FP4-matmul path.

Public names follow the reference package (``src/fouroversix/__init__.py:22-40``):
``quantize``, ``dequantize``, ``quantized_matmul``, ``quantize_model`` and their config /
container types.  Everything runs in hand-written HIP kernels behind a C ABI
(``include/fouroversix_hip.h``); there is no CPU or eager fallback.
"""

from .matmul import quantized_matmul
from .model import (
    FourOverSixLinear,
    ModelQuantizationConfig,
    ModuleQuantizationConfig,
    QuantizedModule,
    quantize_model,
)
from .quantize import QuantizationConfig, QuantizedTensor, dequantize, quantize
from .utils import DataType, MatmulBackend, QuantizeBackend, RoundStyle, ScaleRule

__version__ = "0.1.0"

__all__ = [
    "DataType",
    "FourOverSixLinear",
    "MatmulBackend",
    "ModelQuantizationConfig",
    "ModuleQuantizationConfig",
    "QuantizationConfig",
    "QuantizeBackend",
    "QuantizedModule",
    "QuantizedTensor",
    "RoundStyle",
    "ScaleRule",
    "dequantize",
    "quantize",
    "quantize_model",
    "quantized_matmul",
]
