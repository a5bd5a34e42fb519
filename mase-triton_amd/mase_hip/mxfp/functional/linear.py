"""MXFP linear (API of src/mase_triton/mxfp/functional/linear.py:10-210).

``layer_type`` spells which operands are quantised: X or Xq (activations, quantised on the fly
along the last axis), W or Wq (weights, given as MXFP components blocked along in_features),
B or Bq (bias).

backend="separate" follows the reference literally: dequantise every operand to a dense tensor,
then ``torch.nn.functional.linear``.
backend="fused" (NotImplementedError in the reference, :31-32) never builds the dense weight.  It has two kernel
families and picks between them by format and shape:

* the block-scaled route (``fused_scaled`` forces it): x is quantised straight into FP8 bytes and E8M0 scales, the
  weight components are turned into the same form (once per layer when a layer calls, see ``w_operand``), and the GEMM
  feeds both to the block-scaled matrix instruction, which applies the scales itself.  Taken for quantised x and W in
  the element formats E4M3 / E3M2 / E2M3 / E2M1, bfloat16 x, K a multiple of 256, for the row counts of x that
  ``takes_scaled_route`` names;
* the bf16 route (``fused_bf16`` forces it): activations go through the single-pass QDQ kernel and the GEMM composes
  the MXFP weight tiles to bf16 in registers on their way to the bf16 matrix instruction.  Every MXFP value has at most
  four significant bits, so bf16 operands are exact.

Both accumulate in fp32 and differ from "separate" only by the summation order (and, on the block-scaled route, by
the re-encoding of E4M3 blocks that hold the code the matrix unit reads as NaN: at most 2^-14 of a block's largest
element, see include/mase_hip.h).
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
_BACKENDS = ("separate", "fused", "fused_bf16", "fused_scaled")
# Which row counts of x backend="fused" sends to the block-scaled kernels.  With the weight operand at hand (a layer keeps
# it): all of them.  Up to 64 rows the product is a read of W, which the block-scaled weight-streaming kernels do without
# touching the codes (N x K = 14336 x 4096: 15 / 15.6 / 19.2 us at 16 / 32 / 64 rows against 21 / 23 / 31 us on the bf16
# kernels; 4096 x 14336: 17.7 / 18.4 / 23.0 against 25.8 / 27.8 / 49.4); beyond, its 256 x 256 tiles, K split over workgroups where
# they are few, stay ahead (14336 x 4096: 33 / 44 / 45 us at 128 / 256 / 512 rows against 37 / 49 / 73).  When the operand has to
# be built inside the call (N * K bytes read and written, 25 us at that size) it pays from about 512 rows (71 against 73 us;
# 72 against 104 at 768).
SCALED_FROM_ROWS_UNPREPARED = 512


def takes_scaled_route(rows: int, prepared: bool) -> bool:
    """Does backend="fused" take the block-scaled kernels for this many rows of x (given that the operands qualify)?"""
    return rows >= (1 if prepared else SCALED_FROM_ROWS_UNPREPARED)


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


def _scaled_eligible(x: Tensor, x_meta: MXFPMeta | None, w_tensor_meta: MXFPTensorMeta, b: Tensor | None) -> bool:
    """Can the block-scaled matrix instruction take this product?"""
    if x_meta is None or x.device.type != "cuda" or x.dtype != torch.bfloat16 or len(w_tensor_meta.shape) != 2:
        return False
    if not (kernels.scaled_format_supported(x_meta) and kernels.scaled_format_supported(w_tensor_meta.meta)):
        return False
    if x_meta.round_mode != "rn" or w_tensor_meta.block_dim % 2 != 1 or getattr(torch, w_tensor_meta.dtype) != x.dtype:
        return False
    out_features, in_features = w_tensor_meta.shape
    if not kernels.scaled_shape_supported(out_features, in_features, x.dtype):
        return False
    return b is None or b.dtype in (torch.bfloat16, torch.float16, torch.float32)


def scaled_weight_operand(w_scales: Tensor, w_elements: Tensor, w_tensor_meta: MXFPTensorMeta) -> "kernels.ScaledOperand":
    """The weight components in the block-scaled GEMM's form (a copy: N * K bytes of codes and N * K / 32 of scales).
    A layer builds it once and passes it to ``mxfp_linear(..., w_operand=...)``."""
    out_features, in_features = w_tensor_meta.shape
    return kernels.scaled_operand_from_mxfp(w_scales, w_elements, w_tensor_meta.meta, out_features, in_features)


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
    backend: Literal["separate", "fused", "fused_bf16", "fused_scaled"],
    *,
    w_operand: "kernels.ScaledOperand | None" = None,
) -> Tensor:
    """``w_operand`` (not in the reference): the weight already in the block-scaled GEMM's form, from
    ``scaled_weight_operand``; without it the fused block-scaled route builds it inside the call."""
    if layer_type not in _LAYER_TYPES:
        raise NotImplementedError(f"Layer type {layer_type} not implemented")
    if backend not in _BACKENDS:
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

    # ---- fused
    rows = x.numel() // x.shape[-1] if x.numel() else 0
    if quantised_x and quantised_w and backend != "fused_bf16" and _scaled_eligible(x, x_meta, w_tensor_meta, bias):
        if backend == "fused_scaled" or takes_scaled_route(rows, w_operand is not None):
            out_features, in_features = w_tensor_meta.shape
            assert x.shape[-1] == in_features
            if w_operand is None:
                w_operand = scaled_weight_operand(w_scales, w_elements, w_tensor_meta)
            assert w_operand.rows == out_features and w_operand.K == in_features
            x2 = x.reshape(-1, in_features)
            if x2.is_contiguous() and x2.data_ptr() % 16 == 0 and x2.shape[0] > 0 and (bias is None or bias.is_contiguous()):
                # operand of x and product behind one call into the library (a decode-sized product is bound by the host)
                y = kernels.linear_scaled(x2, x_meta.element_exp_bits, x_meta.element_frac_bits, False, w_operand, bias)
            else:
                y = kernels.mxfp_gemm_scaled(kernels.scaled_operand_from_dense(x2, x_meta), w_operand, bias, x.dtype)
            return y.view(*x.shape[:-1], out_features)
    elif backend == "fused_scaled":
        raise NotImplementedError("backend 'fused_scaled' needs quantised bfloat16 x and W in E4M3 / E3M2 / E2M3 / E2M1 with in_features a "
                                  "multiple of 256 and out_features a multiple of 8")
    if quantised_w and _gemm_eligible(x, quantised_x, w_tensor_meta, bias):
        out_features, in_features = w_tensor_meta.shape
        assert x.shape[-1] == in_features
        lead = x.shape[:-1]
        a = x.reshape(-1, in_features)
        if quantised_x:
            # MXFP values are exact in bf16 whatever x.dtype is
            a = kernels.quantize_dequantize(a.flatten(), x_meta, torch.bfloat16).view(-1, in_features)
        if (w_operand is not None and a.dtype == torch.bfloat16 and w_operand.rows == out_features and w_operand.K == in_features
                and kernels.prepared_w_shape_supported(a.shape[0], out_features, in_features)):
            # a layer's kept weight operand: the large-tile bf16 kernel reads it with a cheaper compose and scale fetch
            return kernels.mxfp_gemm_prepared_w(a, w_operand, bias, x.dtype).view(*lead, out_features)
        y = kernels.mxfp_gemm(a, None, None, None, w_scales, w_elements, w_tensor_meta.meta, bias,
                              a.shape[0], out_features, in_features, x.dtype)
        return y.view(*lead, out_features)
    if quantised_x:
        x = quantize_dequantize(x, block_dim=-1, mxfp_meta=x_meta)
    if quantised_w:
        w = compose_mxfp_tensor(w_scales, w_elements, w_tensor_meta)
    return torch.nn.functional.linear(x, w, bias)
