"""Minifloat-quantised linear (API of src/mase_triton/minifloat/functional/linear.py:108-171).

``layer_type`` spells which operands are quantised: X or Xq, W or Wq, B or Bq.  Activations
are quantise-dequantised on the fly; weights and biases arrive as uint16 codes.  Both backends
dequantise and call the dense GEMM; "fused" uses the single-pass QDQ kernel for activations
(the reference raises NotImplementedError for it).
"""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from ..meta import MinifloatMeta, MinifloatTensorMeta
from .cast import compose_minifloat_component, extract_minifloat_component, quantize_dequantize

_LAYER_TYPES = ("XWB", "XWBq", "XWqB", "XWqBq", "XqWB", "XqWBq", "XqWqB", "XqWqBq")


def _check_backend(backend: str) -> None:
    if backend not in ("separate", "fused"):
        raise NotImplementedError(f"backend {backend!r} not implemented")


def minifloat_linear(
    x: Tensor,
    x_meta: MinifloatMeta | None,
    w: Tensor | None,
    w_element: Tensor | None,
    w_tensor_meta: MinifloatTensorMeta | None,
    b: Tensor | None,
    b_element: Tensor | None,
    b_tensor_meta: MinifloatTensorMeta | None,
    layer_type: Literal["XWB", "XWBq", "XWqB", "XWqBq", "XqWB", "XqWBq", "XqWqB", "XqWqBq"],
    backend: Literal["separate", "fused"],
) -> Tensor:
    if layer_type not in _LAYER_TYPES:
        raise NotImplementedError(f"Layer type {layer_type} not implemented")
    _check_backend(backend)
    if layer_type.startswith("Xq"):
        if backend == "fused":
            x = quantize_dequantize(x, x_meta)
        else:
            x_element, x_tensor_meta = extract_minifloat_component(x, x_meta)
            x = compose_minifloat_component(x_element, x_tensor_meta)
    if "Wq" in layer_type:
        w = compose_minifloat_component(w_element, w_tensor_meta)
    if layer_type.endswith("Bq"):
        # as in the reference (:22-25, :49-52): the quantised bias is used only when a dense `b`
        # is passed as well; with b=None (what MinifloatLinearPTQ passes) no bias is added
        b = compose_minifloat_component(b_element, b_tensor_meta) if b is not None else None
    return torch.nn.functional.linear(x, w, b)
