"""MXFP matmul (API of src/mase_triton/mxfp/functional/matmul.py:10-35): ``input @ other`` with
``input`` quantised along its last axis and ``other`` along its second-to-last axis (the
contraction axis of both).

backend="separate" follows the reference: extract + compose each quantised operand, then
``torch.matmul``.
backend="fused" (NotImplementedError in the reference, :21-22) quantises ``other`` in place
along its second-to-last axis (no transposed copy).  When ``other`` is quantised and either is a
matrix or has the batch shape of ``input`` with few batches, it stays in MXFP form: its codes
come out as [.., N, K], the layout the GEMM kernels read, and each batch is one GEMM launch that
composes the codes to bf16 on their way to the MFMA units.  Everything else goes through the
one-pass quantise-dequantise kernels and ``torch.matmul``.
"""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor

from .. import kernels
from ..meta import MXFPMeta
from .cast import compose_mxfp_tensor, extract_mxfp_components, quantize_dequantize

# more batches than this and one batched dense GEMM beats a launch per batch
_MAX_GEMM_BATCHES = 16


def _gemm_route(input: Tensor, other: Tensor, quantised_input: bool, other_meta: MXFPMeta) -> bool:
    if input.device.type != "cuda" or other.device != input.device or input.ndim < 2 or other.ndim < 2:
        return False
    if input.dtype != other.dtype or input.dtype not in (torch.bfloat16, torch.float32):
        return False
    if not quantised_input and input.dtype != torch.bfloat16:
        return False  # the MFMA path would round a dense fp32 operand to bf16
    if input.shape[-1] != other.shape[-2] or input.numel() == 0 or other.numel() == 0:
        return False
    if not kernels.strided_blocks_supported(tuple(other.shape), -2, other_meta):
        return False
    if other.ndim == 2:
        return True
    batches = 1
    for d in other.shape[:-2]:
        batches *= d
    return tuple(other.shape[:-2]) == tuple(input.shape[:-2]) and batches <= _MAX_GEMM_BATCHES


def _matmul_through_gemm(input: Tensor, other: Tensor, input_meta: MXFPMeta | None, other_meta: MXFPMeta) -> Tensor:
    K, N = other.shape[-2], other.shape[-1]
    a = input
    if input_meta is not None:
        # MXFP values are exact in bf16 whatever input.dtype is
        a = quantize_dequantize(input, block_dim=-1, mxfp_meta=input_meta, output_dtype=torch.bfloat16)
    a = a.contiguous()
    w_scales, w_elements = kernels.extract_mxfp_components_strided(other, -2, other_meta)  # [.., N, K] order
    if other.ndim == 2:
        y = kernels.mxfp_gemm(a.view(-1, K), None, None, None, w_scales, w_elements, other_meta, None,
                              a.numel() // K, N, K, input.dtype)
        return y.view(*input.shape[:-1], N)
    M = input.shape[-2]
    y = torch.empty(*input.shape[:-1], N, dtype=input.dtype, device=input.device)
    a3, y3 = a.view(-1, M, K), y.view(-1, M, N)
    sc3, el3 = w_scales.view(-1, N * K // 32), w_elements.view(-1, N * K)
    for b in range(a3.shape[0]):
        kernels.mxfp_gemm(a3[b], None, None, None, sc3[b], el3[b], other_meta, None, M, N, K, input.dtype, out=y3[b])
    return y


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
