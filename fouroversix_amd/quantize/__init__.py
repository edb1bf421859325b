from .config import QuantizationConfig
from .frontend import can_quantize, dequantize, quantize
from .layout import from_blocked, get_rht_matrix, to_blocked
from .quantized_tensor import QuantizedTensor

__all__ = [
    "QuantizationConfig",
    "QuantizedTensor",
    "can_quantize",
    "dequantize",
    "from_blocked",
    "get_rht_matrix",
    "quantize",
    "to_blocked",
]
