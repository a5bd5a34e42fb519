from .cast import compose_minifloat_component, extract_minifloat_component, quantize_dequantize
from .linear import minifloat_linear
from .matmul import minifloat_matmul

__all__ = [
    "extract_minifloat_component",
    "compose_minifloat_component",
    "quantize_dequantize",
    "minifloat_linear",
    "minifloat_matmul",
]
