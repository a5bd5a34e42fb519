"""Minifloat-quantised linear (API of src/mase_triton/minifloat/functional/linear.py:108-171).

``layer_type`` spells which operands are quantised: X or Xq, W or Wq, B or Bq.  Activations
are quantise-dequantised on the fly; weights and biases arrive as uint16 codes.

backend="separate" follows the reference literally: dequantise every operand, then
``torch.nn.functional.linear``.
backend="fused" (NotImplementedError in the reference, :127-128) uses the single-pass QDQ kernel
for activations and, when the weight format is one the MXFP GEMM decodes (at most 8 bits wide,
see ``_GEMM_WEIGHT_FORMATS``), never builds the dense weight: a minifloat code is an MXFP
element whose block scale is 2^0, so the codes are narrowed to one byte each and the GEMM
composes them to bf16 in registers on their way to the MFMA units.  Such values have at most
four significant bits, so the bf16 operands are exact and the result differs from "separate"
only by the summation order.  Other formats fall back to compose + dense GEMM.

With bfloat16 activations that are quantised too (XqWq), both formats among E4M3 / E3M2 / E2M3 /
E2M1 and round to nearest, "fused" takes the block-scaled matrix instruction instead, for the row
counts ``mxfp.functional.linear.takes_scaled_route`` names: x is rounded straight into code bytes
with unit scales, W's codes are put into the same form (once per layer when a layer calls), and
the GEMM multiplies the codes themselves at twice the bf16 rate.  The only difference in value is
the re-encoding of E4M3 blocks that hold the top code (see include/mase_hip.h).
``backend="fused_bf16"`` / ``"fused_scaled"`` (not in the reference) force one route or the other.
"""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from ...mxfp import kernels as mxfp_kernels
from ...mxfp.functional.linear import takes_scaled_route
from ...mxfp.meta import MXFPMeta
from .. import kernels
from ..meta import MinifloatMeta, MinifloatTensorMeta
from .cast import compose_minifloat_component, extract_minifloat_component, quantize_dequantize

_LAYER_TYPES = ("XWB", "XWBq", "XWqB", "XWqBq", "XqWB", "XqWBq", "XqWqB", "XqWqBq")


# (exp_bits, frac_bits) of the element formats the GEMM kernels are instantiated for
_GEMM_WEIGHT_FORMATS = ((4, 3), (5, 2), (2, 3), (3, 2), (2, 1))
_UNIT_SCALE = 127  # E8M0 code of 2^0


def narrow_weight_codes(w_element: Tensor, w_tensor_meta: MinifloatTensorMeta) -> tuple[Tensor, Tensor]:
    """uint16 minifloat codes [N, K] -> (uint8 unit scales [N*K/32], uint8 codes [N, K]) for the
    MXFP GEMM.  Only the low ``1 + exp_bits + frac_bits`` bits of a code carry meaning, as in
    the decode of the reference (src/mase_triton/minifloat/fake.py:97-123)."""
    assert w_element.dtype == torch.uint16
    codes = w_element.contiguous().view(torch.uint8).view(*w_element.shape, 2)[..., 0].contiguous()
    n_bits = w_tensor_meta.meta.n_bits
    if n_bits < 8:
        codes &= (1 << n_bits) - 1
    scales = torch.full((w_element.numel() // 32,), _UNIT_SCALE, dtype=torch.uint8, device=w_element.device)
    return scales, codes


def gemm_weight_eligible(w_tensor_meta: MinifloatTensorMeta) -> bool:
    """Can the MXFP GEMM decode this weight?  Finite-only format of a supported width, 2-D,
    in_features a multiple of the 32-element block."""
    m = w_tensor_meta.meta
    return (m.is_finite and (m.exp_bits, m.frac_bits) in _GEMM_WEIGHT_FORMATS
            and len(w_tensor_meta.shape) == 2 and w_tensor_meta.shape[1] % 32 == 0)


def _gemm_eligible(x: Tensor, x_meta: MinifloatMeta | None, w_tensor_meta: MinifloatTensorMeta,
                   b: Tensor | None) -> bool:
    """The MFMA path computes on bf16 operands: a dense X must already be bf16, a quantised X
    must be in a format bf16 holds exactly."""
    if x.device.type != "cuda" or not gemm_weight_eligible(w_tensor_meta):
        return False
    if x.dtype not in (torch.bfloat16, torch.float32) or getattr(torch, w_tensor_meta.dtype) != x.dtype:
        return False
    if x_meta is None:
        if x.dtype != torch.bfloat16:
            return False
    elif x_meta.exp_bits > 8 or x_meta.frac_bits > 7:
        return False
    return b is None or b.dtype in (torch.bfloat16, torch.float16, torch.float32)


def _scaled_format(meta: MinifloatMeta) -> bool:
    return meta.is_finite and meta.round_mode == "rn" and mxfp_kernels.scaled_element_format_supported(meta.exp_bits, meta.frac_bits)


def _scaled_eligible(x: Tensor, x_meta: MinifloatMeta | None, w_tensor_meta: MinifloatTensorMeta, b: Tensor | None) -> bool:
    """Can the block-scaled matrix instruction take this product?"""
    if x_meta is None or x.device.type != "cuda" or x.dtype != torch.bfloat16 or len(w_tensor_meta.shape) != 2:
        return False
    if not (_scaled_format(x_meta) and _scaled_format(w_tensor_meta.meta)) or getattr(torch, w_tensor_meta.dtype) != x.dtype:
        return False
    out_features, in_features = w_tensor_meta.shape
    if not mxfp_kernels.scaled_shape_supported(out_features, in_features, x.dtype):
        return False
    return b is None or b.dtype in (torch.bfloat16, torch.float16, torch.float32)


def scaled_weight_operand(w_element: Tensor, w_tensor_meta: MinifloatTensorMeta,
                          narrowed: tuple[Tensor, Tensor] | None = None) -> "mxfp_kernels.ScaledOperand":
    """The weight codes in the block-scaled GEMM's form (a copy: N * K bytes of codes, N * K / 32 of unit scales).
    A layer builds it once and passes it to ``minifloat_linear(..., _w_operand=...)``."""
    scales, codes = narrowed if narrowed is not None else narrow_weight_codes(w_element, w_tensor_meta)
    out_features, in_features = w_tensor_meta.shape
    wm = w_tensor_meta.meta
    as_mxfp = MXFPMeta(block_size=32, scale_exp_bits=8, element_exp_bits=wm.exp_bits, element_frac_bits=wm.frac_bits,
                       element_is_finite=True, round_mode="rn")
    return mxfp_kernels.scaled_operand_from_mxfp(scales, codes, as_mxfp, out_features, in_features)


_BACKENDS = ("separate", "fused", "fused_bf16", "fused_scaled")


def _check_backend(backend: str) -> None:
    if backend not in _BACKENDS:
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
    backend: Literal["separate", "fused", "fused_bf16", "fused_scaled"],
    _narrowed: tuple[Tensor, Tensor] | None = None,
    _w_operand: "mxfp_kernels.ScaledOperand | None" = None,
) -> Tensor:
    """``_narrowed`` and ``_w_operand`` (not in the reference's signature): the results of ``narrow_weight_codes`` and
    ``scaled_weight_operand`` for this weight, kept by a caller that applies the same weight many times."""
    if layer_type not in _LAYER_TYPES:
        raise NotImplementedError(f"Layer type {layer_type} not implemented")
    _check_backend(backend)
    quantised_x = layer_type.startswith("Xq")
    quantised_w = "Wq" in layer_type
    if layer_type.endswith("Bq"):
        # as in the reference (:22-25, :49-52): the quantised bias is used only when a dense `b`
        # is passed as well; with b=None (what MinifloatLinearPTQ passes) no bias is added
        b = compose_minifloat_component(b_element, b_tensor_meta) if b is not None else None

    fused = backend != "separate"
    if fused and backend != "fused_bf16" and quantised_x and quantised_w:
        ok = _scaled_eligible(x, x_meta, w_tensor_meta, b)
        if backend == "fused_scaled" and not ok:
            raise NotImplementedError("fused_scaled: this product does not fit the block-scaled GEMM (bfloat16 x, formats E4M3 / "
                                      "E3M2 / E2M3 / E2M1 rounded to nearest, K a multiple of 256 and at least 512, N of 8)")
        rows = x.numel() // x.shape[-1] if x.numel() else 0
        if ok and (backend == "fused_scaled" or takes_scaled_route(rows, _w_operand is not None)):
            if _w_operand is None:
                _w_operand = scaled_weight_operand(w_element, w_tensor_meta, _narrowed)
            x2 = x.reshape(-1, x.shape[-1])
            if x2.is_contiguous() and x2.data_ptr() % 16 == 0 and x2.shape[0] > 0 and (b is None or b.is_contiguous()):
                y = mxfp_kernels.linear_scaled(x2, x_meta.exp_bits, x_meta.frac_bits, True, _w_operand, b)
            else:
                a_op = mxfp_kernels.scaled_operand_from_dense_minifloat(x2, x_meta.exp_bits, x_meta.frac_bits)
                y = mxfp_kernels.mxfp_gemm_scaled(a_op, _w_operand, b, x.dtype)
            return y.view(*x.shape[:-1], w_tensor_meta.shape[0])
    elif backend == "fused_scaled":
        raise NotImplementedError("fused_scaled needs quantised activations and weights (XqWq layer types)")

    if fused and quantised_w and _gemm_eligible(x, x_meta if quantised_x else None, w_tensor_meta, b):
        if _narrowed is None:
            _narrowed = narrow_weight_codes(w_element, w_tensor_meta)
        return _fused_gemm(x, x_meta if quantised_x else None, _narrowed, w_tensor_meta, b)

    if quantised_x:
        if fused:
            x = quantize_dequantize(x, x_meta)
        else:
            x_element, x_tensor_meta = extract_minifloat_component(x, x_meta)
            x = compose_minifloat_component(x_element, x_tensor_meta)
    if quantised_w:
        w = compose_minifloat_component(w_element, w_tensor_meta)
    return torch.nn.functional.linear(x, w, b)


def _fused_gemm(x: Tensor, x_meta: MinifloatMeta | None, narrowed: tuple[Tensor, Tensor],
                w_tensor_meta: MinifloatTensorMeta, bias: Tensor | None) -> Tensor:
    out_features, in_features = w_tensor_meta.shape
    assert x.shape[-1] == in_features
    scales, codes = narrowed
    wm = w_tensor_meta.meta
    gemm_meta = MXFPMeta(block_size=32, scale_exp_bits=8, element_exp_bits=wm.exp_bits,
                         element_frac_bits=wm.frac_bits, element_is_finite=True, round_mode="rn")
    a = x.reshape(-1, in_features)
    if x_meta is not None:
        a = kernels.quantize_dequantize(a, x_meta, torch.bfloat16)
    y = mxfp_kernels.mxfp_gemm(a, None, None, None, scales, codes, gemm_meta, bias,
                               a.shape[0], out_features, in_features, x.dtype)
    return y.view(*x.shape[:-1], out_features)
