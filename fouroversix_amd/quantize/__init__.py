from .config import QuantizationConfig
from .frontend import attach_known_amax, can_quantize, dequantize, known_amax, quantize
from .layout import from_blocked, get_rht_matrix, to_blocked
from .quantized_tensor import QuantizedTensor

__all__ = [
    "QuantizationConfig",
    "QuantizedTensor",
    "attach_known_amax",
    "can_quantize",
    "dequantize",
    "from_blocked",
    "get_rht_matrix",
    "known_amax",
    "quantize",
    "to_blocked",
]
