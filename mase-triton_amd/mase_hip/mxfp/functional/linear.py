"""MXFP linear (API of src/mase_triton/mxfp/functional/linear.py:10-210).

``layer_type`` spells which operands are quantised: X or Xq (activations, quantised on the fly
along the last axis), W or Wq (weights, given as MXFP components blocked along in_features),
B or Bq (bias).

backend="separate" follows the reference literally: dequantise every operand to a dense tensor,
then ``torch.nn.functional.linear``.
backend="fused" (NotImplementedError in the reference, :31-32) never builds the dense weight:
activations go through the single-pass QDQ kernel and the GEMM composes the MXFP weight tiles
to bf16 in registers on their way to the MFMA units (fp32 accumulation).  Every MXFP value has
at most four significant bits, so bf16 operands are exact and the result differs from
"separate" only by the summation order.
backend="auto" (not in the reference) is "fused" up to ``AUTO_DENSE_FROM_ROWS`` rows of x and, from there on, the
single-pass QDQ of x, ONE compose of W to bf16 in HBM and the library's dense GEMM: the fused kernel composes every W
element once per 512 rows of x, and on this power-limited chip that in-loop work costs more than writing W out once when
there are thousands of rows (measured cross-over between 2048 and 4096 rows for N x K = 14336 x 4096 and 4096 x 14336).
It needs N * K * 2 bytes of temporary memory per call.
"""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from .. import kernels
from ..meta import MXFPMeta, MXFPTensorMeta
from .cast import compose_mxfp_tensor, extract_mxfp_components, quantize_dequantize

_LAYER_TYPES = ("XWB", "XWBq", "XWqB", "XWqBq", "XqWB", "XqWBq", "XqWqB", "XqWqBq")
_GEMM_DTYPES = (torch.bfloat16, torch.float32)
AUTO_DENSE_FROM_ROWS = 3072


def parse_mxfp_linear_type(x_meta: MXFPMeta | None, w_tensor_meta: MXFPTensorMeta | None,
                           b_tensor_meta: MXFPTensorMeta | None) -> str:
    """Layer-type string from which metas are present."""
    return ("X" if x_meta is None else "Xq") + ("W" if w_tensor_meta is None else "Wq") + (
        "B" if b_tensor_meta is None else "Bq")


def _dense_bias(b, b_scales, b_elements, b_tensor_meta, layer_type):
    if not layer_type.endswith("Bq"):
        return b
    # as in the reference (:25-28, :56-59): the quantised bias is used only when a dense `b` is
    # passed too; with b=None (what MXFPLinearPTQ passes for "Bq" layers) no bias is added
    return compose_mxfp_tensor(b_scales, b_elements, b_tensor_meta) if b is not None else None


def _gemm_eligible(x: Tensor, quantised_x: bool, w_tensor_meta: MXFPTensorMeta, b: Tensor | None) -> bool:
    """The MFMA path computes on bf16 operands: exact for MXFP values, lossy for dense fp16/fp32
    activations, so a dense X must already be bf16."""
    if x.device.type != "cuda" or w_tensor_meta.meta.block_size != 32 or len(w_tensor_meta.shape) != 2:
        return False
    if not w_tensor_meta.meta.element_is_finite:
        return False  # the GEMM decodes the top exponent field as an ordinary binade, this format reads it as inf / NaN
    if w_tensor_meta.block_dim % 2 != 1 or w_tensor_meta.shape[1] % 32 != 0:
        return False
    if x.dtype not in _GEMM_DTYPES or getattr(torch, w_tensor_meta.dtype) != x.dtype:
        return False
    if not quantised_x and x.dtype != torch.bfloat16:
        return False
    return b is None or b.dtype in (torch.bfloat16, torch.float16, torch.float32)


def mxfp_linear(
    x: Tensor,
    x_meta: MXFPMeta | None,
    w: Tensor | None,
    w_scales: Tensor | None,
    w_elements: Tensor | None,
    w_tensor_meta: MXFPTensorMeta | None,
    b: Tensor | None,
    b_scales: Tensor | None,
    b_elements: Tensor | None,
    b_tensor_meta: MXFPTensorMeta | None,
    layer_type: Literal["XWB", "XWBq", "XWqB", "XWqBq", "XqWB", "XqWBq", "XqWqB", "XqWqBq"],
    backend: Literal["separate", "fused", "auto"],
) -> Tensor:
    if layer_type not in _LAYER_TYPES:
        raise NotImplementedError(f"Layer type {layer_type} not implemented")
    if backend not in ("separate", "fused", "auto"):
        raise NotImplementedError(f"backend {backend!r} not implemented")
    quantised_x = layer_type.startswith("Xq")
    quantised_w = "Wq" in layer_type
    bias = _dense_bias(b, b_scales, b_elements, b_tensor_meta, layer_type)

    if backend == "separate":
        if quantised_x:
            x_scales, x_elements, x_tensor_meta = extract_mxfp_components(x, block_dim=-1, mxfp_meta=x_meta)
            x = compose_mxfp_tensor(x_scales, x_elements, x_tensor_meta)
        if quantised_w:
            w = compose_mxfp_tensor(w_scales, w_elements, w_tensor_meta)
        return torch.nn.functional.linear(x, w, bias)

    # ---- fused (auto: only while the rows of x are few enough for the in-loop compose to pay)
    rows = x.numel() // x.shape[-1] if x.numel() else 0
    through_kernel = backend == "fused" or rows < AUTO_DENSE_FROM_ROWS
    if through_kernel and quantised_w and _gemm_eligible(x, quantised_x, w_tensor_meta, bias):
        out_features, in_features = w_tensor_meta.shape
        assert x.shape[-1] == in_features
        lead = x.shape[:-1]
        a = x.reshape(-1, in_features)
        if quantised_x:
            # MXFP values are exact in bf16 whatever x.dtype is
            a = kernels.quantize_dequantize(a.flatten(), x_meta, torch.bfloat16).view(-1, in_features)
        y = kernels.mxfp_gemm(a, None, None, None, w_scales, w_elements, w_tensor_meta.meta, bias,
                              a.shape[0], out_features, in_features, x.dtype)
        return y.view(*lead, out_features)
    if quantised_x:
        x = quantize_dequantize(x, block_dim=-1, mxfp_meta=x_meta)
    if quantised_w:
        w = compose_mxfp_tensor(w_scales, w_elements, w_tensor_meta)
    return torch.nn.functional.linear(x, w, bias)
