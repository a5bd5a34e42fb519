from .cast import compose_minifloat_component, extract_minifloat_component, quantize_dequantize
from .linear import gemm_weight_eligible, minifloat_linear, narrow_weight_codes
from .matmul import minifloat_matmul

__all__ = [
    "extract_minifloat_component",
    "compose_minifloat_component",
    "quantize_dequantize",
    "minifloat_linear",
    "minifloat_matmul",
]
