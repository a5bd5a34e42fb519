"""Minifloat-quantised matmul (API of src/mase_triton/minifloat/functional/matmul.py:10-35).

backend="separate" follows the reference: quantise-dequantise each quantised operand, then ``torch.matmul``.
backend="fused" (NotImplementedError in the reference, :21-22): when ``other`` is quantised to one of the one-byte formats
the GEMM kernels decode, it never becomes a dense tensor: its codes are extracted, laid out as [.., N, K] one byte each
and given unit block scales (a minifloat code is an MXFP element whose block scale is 2^0), and the dequant-fused GEMM
composes them to bf16 on their way to the MFMA units; leading batch axes, broadcast ones included, go into one batched
launch.  Such values have at most four significant bits, so the result differs from "separate" only by the order of the
fp32 additions.  Everything else (wider formats, formats with inf / NaN codes, a contraction axis that is not a multiple
of 32, a dense float32 ``input``) takes the single-pass quantise-dequantise kernels and ``torch.matmul``.
"""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from ...mxfp.functional.matmul import gemm_over_batches
from ...mxfp.meta import MXFPMeta
from .. import kernels
from ..meta import MinifloatMeta
from .cast import quantize_dequantize
from .linear import _GEMM_WEIGHT_FORMATS, _UNIT_SCALE


def _gemm_route(input: Tensor, other: Tensor, input_meta: MinifloatMeta | None, other_meta: MinifloatMeta) -> bool:
    if input.device.type != "cuda" or other.device != input.device or input.ndim < 2 or other.ndim < 2:
        return False
    if input.dtype != other.dtype or input.dtype not in (torch.bfloat16, torch.float32):
        return False
    if not other_meta.is_finite or (other_meta.exp_bits, other_meta.frac_bits) not in _GEMM_WEIGHT_FORMATS:
        return False
    if input_meta is None:
        if input.dtype != torch.bfloat16:
            return False        # the MFMA path would round a dense fp32 operand to bf16
    elif input_meta.exp_bits > 8 or input_meta.frac_bits > 7:
        return False            # bf16 would not hold the quantised values exactly
    K, N = other.shape[-2], other.shape[-1]
    if input.shape[-1] != K or K % 32 != 0 or input.numel() == 0 or other.numel() == 0:
        return False
    if other.ndim == 2:
        return True
    try:
        torch.broadcast_shapes(tuple(input.shape[:-2]), tuple(other.shape[:-2]))
    except RuntimeError:
        return False
    return (input.shape[-2] * N * input.element_size()) % 16 == 0   # every product's output 16-byte aligned


def _matmul_through_gemm(input: Tensor, other: Tensor, input_meta: MinifloatMeta | None, other_meta: MinifloatMeta) -> Tensor:
    K, N = other.shape[-2], other.shape[-1]
    a = input if input_meta is None else kernels.quantize_dequantize(input, input_meta, torch.bfloat16)
    codes16 = kernels.extract_minifloat_component(other, other_meta)                     # uint16 [.., K, N]
    codes = codes16.view(torch.int16).transpose(-1, -2).contiguous().view(torch.uint8)   # [.., N, 2 K]: low byte first
    codes = codes.view(*codes16.shape[:-2], N, K, 2)[..., 0].contiguous()                 # [.., N, K], one byte per code
    scales = torch.full((codes.numel() // 32,), _UNIT_SCALE, dtype=torch.uint8, device=codes.device)
    gemm_meta = MXFPMeta(block_size=32, scale_exp_bits=8, element_exp_bits=other_meta.exp_bits,
                         element_frac_bits=other_meta.frac_bits, element_is_finite=True, round_mode="rn")
    return gemm_over_batches(a.contiguous(), scales, codes, gemm_meta, tuple(other.shape[:-2]), N, input.dtype)


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
    quantised_input, quantised_other = "Xq" in func_type, "Wq" in func_type
    if quantised_input:
        assert input_meta is not None
    if quantised_other:
        assert other_meta is not None
    if backend == "fused" and quantised_other and _gemm_route(input, other, input_meta if quantised_input else None, other_meta):
        return _matmul_through_gemm(input, other, input_meta if quantised_input else None, other_meta)
    if quantised_input:
        input = quantize_dequantize(input, input_meta)
    if quantised_other:
        other = quantize_dequantize(other, other_meta)
    return torch.matmul(input, other)
