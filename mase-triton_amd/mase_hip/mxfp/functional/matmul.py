"""MXFP matmul (API of src/mase_triton/mxfp/functional/matmul.py:10-35): ``input @ other`` with
``input`` quantised along its last axis and ``other`` along its second-to-last axis (the
contraction axis of both).

backend="separate" follows the reference: extract + compose each quantised operand, then
``torch.matmul``.
backend="fused" (NotImplementedError in the reference, :21-22) quantises ``other`` in place
along its second-to-last axis (no transposed copy).  When ``other`` is quantised it stays in MXFP
form: its codes come out as [.., N, K], the layout the GEMM kernels read, and all leading batch
axes (broadcast ones included) go into ONE batched GEMM launch that composes the codes to bf16
on their way to the MFMA units.  A product of two quantised bfloat16 operands against ONE matrix
(``other`` without batch axes) with enough rows takes the block-scaled FP8 matrix instruction instead, as
``mxfp_linear`` does (functional/linear.py).  Everything else goes through the one-pass quantise-dequantise
kernels and ``torch.matmul``.
"""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from .. import kernels
from ..meta import MXFPMeta
from .cast import compose_mxfp_tensor, extract_mxfp_components, quantize_dequantize


def _gemm_route(input: Tensor, other: Tensor, quantised_input: bool, other_meta: MXFPMeta) -> bool:
    if input.device.type != "cuda" or other.device != input.device or input.ndim < 2 or other.ndim < 2:
        return False
    if input.dtype != other.dtype or input.dtype not in (torch.bfloat16, torch.float32):
        return False
    if not quantised_input and input.dtype != torch.bfloat16:
        return False  # the MFMA path would round a dense fp32 operand to bf16
    if input.shape[-1] != other.shape[-2] or input.numel() == 0 or other.numel() == 0:
        return False
    if not kernels.strided_blocks_supported(tuple(other.shape), -2, other_meta) or not other_meta.element_is_finite:
        return False
    if other.ndim == 2:
        return True
    try:
        torch.broadcast_shapes(tuple(input.shape[:-2]), tuple(other.shape[:-2]))
    except RuntimeError:
        return False
    M, N = input.shape[-2], other.shape[-1]
    return (M * N * input.element_size()) % 16 == 0       # every product's output 16-byte aligned


def _prod(shape) -> int:
    n = 1
    for d in shape:
        n *= d
    return n


def gemm_over_batches(a: Tensor, w_scales: Tensor, w_elements: Tensor, w_meta: MXFPMeta, w_batch: tuple, N: int,
                      output_dtype: torch.dtype) -> Tensor:
    """``a [*bi, M, K]`` (dense bfloat16, contiguous) against weights held as components in [*w_batch, N, K] order: one GEMM
    when the weight is a matrix, else ONE batched launch over the broadcast of the two batch shapes."""
    K = a.shape[-1]
    if len(w_batch) == 0:
        y = kernels.mxfp_gemm(a.view(-1, K), None, None, None, w_scales, w_elements, w_meta, None, a.numel() // K, N, K, output_dtype)
        return y.view(*a.shape[:-1], N)
    M = a.shape[-2]
    bi, bo = tuple(a.shape[:-2]), tuple(w_batch)
    batch = tuple(torch.broadcast_shapes(bi, bo))
    # an operand whose batch axes are all 1 is shared through a zero stride; one that is broadcast along some axes only
    # is expanded (a copy of that operand)
    if _prod(bi) == 1:
        a_stride = 0
    else:
        if bi != batch:
            a = a.expand(*batch, M, K).contiguous()
        a_stride = M * K
    if _prod(bo) == 1:
        w_stride = 0
    else:
        if bo != batch:
            w_scales = w_scales.view(*bo, N * K // 32).expand(*batch, N * K // 32).contiguous()
            w_elements = w_elements.view(*bo, N * K).expand(*batch, N * K).contiguous()
        w_stride = N * K
    y = kernels.mxfp_gemm_batched(a.reshape(-1), w_scales.reshape(-1), w_elements.reshape(-1), w_meta, _prod(batch), M, N, K,
                                  output_dtype, a_stride, w_stride)
    return y.view(*batch, M, N)


def _scaled_route(input: Tensor, other: Tensor, input_meta: MXFPMeta | None, other_meta: MXFPMeta) -> bool:
    """Both operands quantised, bfloat16, one weight matrix, formats and shape the block-scaled GEMM takes, and enough rows
    to pay for turning ``other``'s codes into its operand form inside the call."""
    from . import linear as L

    if input_meta is None or input.dtype != torch.bfloat16 or _prod(other.shape[:-2]) != 1:
        return False
    if not (kernels.scaled_format_supported(input_meta) and kernels.scaled_format_supported(other_meta)):
        return False
    if input_meta.round_mode != "rn" or other_meta.round_mode != "rn":
        return False
    K, N = other.shape[-2], other.shape[-1]
    return kernels.scaled_shape_supported(N, K, input.dtype) and L.takes_scaled_route(input.numel() // K, False)


def _matmul_through_gemm(input: Tensor, other: Tensor, input_meta: MXFPMeta | None, other_meta: MXFPMeta) -> Tensor:
    if _scaled_route(input, other, input_meta, other_meta):
        K, N = other.shape[-2], other.shape[-1]
        w_scales, w_elements = kernels.extract_mxfp_components_strided(other.reshape(K, N), -2, other_meta)   # [N, K] order
        w_op = kernels.scaled_operand_from_mxfp(w_scales, w_elements, other_meta, N, K)
        a_op = kernels.scaled_operand_from_dense(input.reshape(-1, K), input_meta)
        y = kernels.mxfp_gemm_scaled(a_op, w_op, None, input.dtype)
        lead = torch.broadcast_shapes(tuple(input.shape[:-2]), tuple(other.shape[:-2]))
        return y.view(*lead, input.shape[-2], N)
    a = input
    if input_meta is not None:
        # MXFP values are exact in bf16 whatever input.dtype is
        a = quantize_dequantize(input, block_dim=-1, mxfp_meta=input_meta, output_dtype=torch.bfloat16)
    w_scales, w_elements = kernels.extract_mxfp_components_strided(other, -2, other_meta)  # [.., N, K] order
    return gemm_over_batches(a.contiguous(), w_scales, w_elements, other_meta, tuple(other.shape[:-2]), other.shape[-1], input.dtype)


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
    quantised_input, quantised_other = "Xq" in func_type, "Wq" in func_type
    if quantised_input:
        assert input_meta is not None
    if quantised_other:
        assert other_meta is not None
    if fused and quantised_other and _gemm_route(input, other, quantised_input, other_meta):
        return _matmul_through_gemm(input, other, input_meta if quantised_input else None, other_meta)
    if quantised_input:
        if fused:
            input = quantize_dequantize(input, block_dim=-1, mxfp_meta=input_meta)
        else:
            sc, el, tm = extract_mxfp_components(input, block_dim=-1, mxfp_meta=input_meta)
            input = compose_mxfp_tensor(sc, el, tm)
    if quantised_other:
        if fused:
            other = quantize_dequantize(other, block_dim=-2, mxfp_meta=other_meta)
        else:
            sc, el, tm = extract_mxfp_components(other, block_dim=-2, mxfp_meta=other_meta)
            other = compose_mxfp_tensor(sc, el, tm)
    return torch.matmul(input, other)
