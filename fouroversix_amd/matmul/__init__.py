from .frontend import quantized_matmul

__all__ = ["quantized_matmul"]
