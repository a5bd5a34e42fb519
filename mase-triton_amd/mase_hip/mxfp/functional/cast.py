"""Public MXFP casts (API of src/mase_triton/mxfp/functional/cast.py:11-129)."""
from __future__ import annotations

import torch
from torch import Tensor

from ...utils.meta import device_str, dtype_str, shape_tuple
from .. import kernels
from ..helpers import flatten_for_quantize, permute_for_dequantize
from ..meta import MXFPMeta, MXFPTensorMeta


def extract_mxfp_components(tensor: Tensor, block_dim: int, mxfp_meta: MXFPMeta) -> tuple[Tensor, Tensor, MXFPTensorMeta]:
    """Quantise ``tensor`` with blocks running along ``block_dim``.

    Returns ``(scales uint8 [n_blocks, 1], elements uint8 [n_blocks, block_size], tensor_meta)``.
    Blocks are consecutive runs of the tensor flattened with ``block_dim`` rotated last, so
    they are 1-D vectors and may straddle rows when that axis is not a multiple of the block.
    """
    ndim = tensor.ndim
    assert -ndim <= block_dim < ndim
    tensor_meta = MXFPTensorMeta(
        device=device_str(tensor.device), dtype=dtype_str(tensor.dtype), shape=shape_tuple(tensor.shape),
        block_dim=block_dim, meta=mxfp_meta)
    if tensor.device.type == "cuda" and kernels.strided_blocks_supported(tensor_meta.shape, block_dim, mxfp_meta):
        # blocks along an inner axis are read in place: same outputs as the permuted copy below
        scales, elements = kernels.extract_mxfp_components_strided(tensor, block_dim, mxfp_meta)
    else:
        scales, elements = kernels.extract_mxfp_components(flatten_for_quantize(tensor, block_dim), mxfp_meta=mxfp_meta)
    return scales, elements, tensor_meta


# name used by the reference's README for the same function
extract_mxfp_tensor = extract_mxfp_components


def compose_mxfp_tensor(scales: Tensor, elements: Tensor, tensor_meta: MXFPTensorMeta,
                        output_dtype: torch.dtype | None = None) -> Tensor:
    """Dequantise to the original shape; ``output_dtype`` defaults to the recorded dtype."""
    if output_dtype is None:
        output_dtype = getattr(torch, tensor_meta.dtype)
    flat = kernels.compose_mxfp_tensor(scales=scales, elements=elements, mxfp_meta=tensor_meta.meta,
                                       output_dtype=output_dtype)
    return permute_for_dequantize(flat, ori_shape=tensor_meta.shape, block_dim=tensor_meta.block_dim)


def quantize_dequantize(tensor: Tensor, block_dim: int, mxfp_meta: MXFPMeta,
                        output_dtype: torch.dtype | None = None) -> Tensor:
    """Round ``tensor`` to the MXFP grid; same values as compose(extract(tensor)), computed by
    one fused kernel without materialising scales or elements."""
    ndim = tensor.ndim
    assert -ndim <= block_dim < ndim
    if output_dtype is None:
        output_dtype = tensor.dtype
    if tensor.device.type == "cuda" and kernels.strided_blocks_supported(shape_tuple(tensor.shape), block_dim, mxfp_meta):
        # contiguous result in the tensor's own layout (the permuted-copy route returns the same
        # values as a transposed view)
        return kernels.quantize_dequantize_strided(tensor, block_dim, mxfp_meta, output_dtype)
    flat = kernels.quantize_dequantize(flatten_for_quantize(tensor, block_dim), mxfp_meta, output_dtype)
    return permute_for_dequantize(flat, ori_shape=shape_tuple(tensor.shape), block_dim=block_dim)
