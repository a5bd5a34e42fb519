"""Minifloat-quantised matmul (API of src/mase_triton/minifloat/functional/matmul.py:10-35)."""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from ..meta import MinifloatMeta
from .cast import quantize_dequantize


def minifloat_matmul(
    input: Tensor,
    other: Tensor,
    input_meta: MinifloatMeta | None,
    other_meta: MinifloatMeta | None,
    func_type: Literal["XW", "XqW", "XWq", "XqWq"],
    backend: Literal["separate", "fused"],
) -> Tensor:
    if backend not in ("separate", "fused"):
        raise NotImplementedError(f"backend {backend!r} not implemented")
    if "Xq" in func_type:
        assert input_meta is not None
        input = quantize_dequantize(input, input_meta)
    if "Wq" in func_type:
        assert other_meta is not None
        other = quantize_dequantize(other, other_meta)
    return torch.matmul(input, other)
