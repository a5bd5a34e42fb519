from .cast import (
    compose_mxfp_tensor,
    extract_mxfp_components,
    extract_mxfp_tensor,
    flatten_for_quantize,
    permute_for_dequantize,
    quantize_dequantize,
)
from .linear import mxfp_linear, parse_mxfp_linear_type
from .matmul import mxfp_matmul

__all__ = [
    "extract_mxfp_components",
    "extract_mxfp_tensor",
    "compose_mxfp_tensor",
    "quantize_dequantize",
    "flatten_for_quantize",
    "permute_for_dequantize",
    "mxfp_linear",
    "parse_mxfp_linear_type",
    "mxfp_matmul",
]
