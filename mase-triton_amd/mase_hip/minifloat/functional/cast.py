"""Public minifloat casts (API of src/mase_triton/minifloat/functional/cast.py:10-90)."""
from __future__ import annotations

import torch
from torch import Tensor

from ...utils.meta import device_str, dtype_str, shape_tuple
from .. import kernels
from ..meta import MinifloatMeta, MinifloatTensorMeta


def extract_minifloat_component(tensor: Tensor, minifloat_meta: MinifloatMeta) -> tuple[Tensor, MinifloatTensorMeta]:
    """Quantise ``tensor``: returns ``(uint16 codes, tensor_meta)``.

    The reference widens to float32 before its kernel (:27); the HIP kernel reads float16 and
    bfloat16 directly, which yields the same codes with half the read traffic.
    """
    tensor_meta = MinifloatTensorMeta(
        device=device_str(tensor.device), dtype=dtype_str(tensor.dtype), shape=shape_tuple(tensor.shape),
        meta=minifloat_meta)
    return kernels.extract_minifloat_component(tensor, minifloat_meta), tensor_meta


def compose_minifloat_component(element: Tensor, tensor_meta: MinifloatTensorMeta,
                                output_dtype: torch.dtype | None = None) -> Tensor:
    """Dequantise codes; ``output_dtype`` defaults to the dtype recorded at extraction."""
    if output_dtype is None:
        output_dtype = getattr(torch, tensor_meta.dtype)
    return kernels.compose_minifloat_component(element, tensor_meta.meta, output_dtype=output_dtype)


def quantize_dequantize(tensor: Tensor, minifloat_meta: MinifloatMeta, output_dtype: torch.dtype | None = None) -> Tensor:
    """Round ``tensor`` to the minifloat grid (fused single-pass kernel)."""
    return kernels.quantize_dequantize(tensor, minifloat_meta, tensor.dtype if output_dtype is None else output_dtype)
