"""MXFP matmul (API of src/mase_triton/mxfp/functional/matmul.py:10-35): ``input @ other`` with
``input`` quantised along its last axis and ``other`` along its second-to-last axis (the
contraction axis of both)."""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from ..meta import MXFPMeta
from .cast import compose_mxfp_tensor, extract_mxfp_components, quantize_dequantize


def mxfp_matmul(
    input: Tensor,
    other: Tensor,
    input_meta: MXFPMeta | None,
    other_meta: MXFPMeta | None,
    func_type: Literal["XW", "XqW", "XWq", "XqWq"],
    backend: Literal["separate", "fused"],
) -> Tensor:
    if backend not in ("separate", "fused"):
        raise NotImplementedError(f"backend {backend!r} not implemented")
    fused = backend == "fused"
    if "Xq" in func_type:
        assert input_meta is not None
        if fused:
            input = quantize_dequantize(input, block_dim=-1, mxfp_meta=input_meta)
        else:
            sc, el, tm = extract_mxfp_components(input, block_dim=-1, mxfp_meta=input_meta)
            input = compose_mxfp_tensor(sc, el, tm)
    if "Wq" in func_type:
        assert other_meta is not None
        if fused:
            other = quantize_dequantize(other, block_dim=-2, mxfp_meta=other_meta)
        else:
            sc, el, tm = extract_mxfp_components(other, block_dim=-2, mxfp_meta=other_meta)
            other = compose_mxfp_tensor(sc, el, tm)
    return torch.matmul(input, other)
