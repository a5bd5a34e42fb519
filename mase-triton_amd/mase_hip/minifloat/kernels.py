"""GPU minifloat casts: tensor-level wrappers over the C ABI.

Same names and signatures as the reference's Triton wrappers
(src/mase_triton/minifloat/kernels/cast.py:148-170, 263-288); results are bit-identical to the
reference's PyTorch "fake" implementation (src/mase_triton/minifloat/fake.py), which the
reference's own Triton kernels are not.
"""
from __future__ import annotations

import torch
from torch import Tensor

from .. import _lib
from .meta import MinifloatMeta


def _fmt(meta: MinifloatMeta):
    return meta.exp_bits, meta.frac_bits, int(meta.is_finite)


def extract_minifloat_component(x: Tensor, minifloat_meta: MinifloatMeta) -> Tensor:
    """float tensor -> uint16 codes of the same shape."""
    _lib.require_gpu(x, "input tensor")
    x = _lib.dense(_lib.as_float_input(x))
    codes = torch.empty(x.shape, dtype=torch.uint16, device=x.device)
    with _lib.on_device(x.device):
        _lib.check(_lib.load().mase_hip_extract_minifloat(
            x.data_ptr(), _lib.dtype_code(x.dtype), codes.data_ptr(), x.numel(), *_fmt(minifloat_meta),
            _lib.round_code(minifloat_meta.round_mode), _lib.stream_ptr(x.device)))
    return codes


def compose_minifloat_component(elements: Tensor, minifloat_meta: MinifloatMeta, output_dtype: torch.dtype) -> Tensor:
    """uint16 codes -> tensor of ``output_dtype`` of the same shape."""
    assert elements.dtype == torch.uint16
    _lib.require_gpu(elements, "elements")
    elements = _lib.dense(elements)
    out = torch.empty(elements.shape, dtype=output_dtype, device=elements.device)
    with _lib.on_device(elements.device):
        _lib.check(_lib.load().mase_hip_compose_minifloat(
            elements.data_ptr(), out.data_ptr(), _lib.dtype_code(output_dtype), elements.numel(),
            *_fmt(minifloat_meta), _lib.stream_ptr(elements.device)))
    return out


def quantize_dequantize(x: Tensor, minifloat_meta: MinifloatMeta, output_dtype: torch.dtype) -> Tensor:
    """compose(extract(x)) in a single pass over memory; codes are never materialised."""
    _lib.require_gpu(x, "input tensor")
    x = _lib.dense(_lib.as_float_input(x))
    out = torch.empty(x.shape, dtype=output_dtype, device=x.device)
    with _lib.on_device(x.device):
        _lib.check(_lib.load().mase_hip_qdq_minifloat(
            x.data_ptr(), _lib.dtype_code(x.dtype), out.data_ptr(), _lib.dtype_code(output_dtype), x.numel(),
            *_fmt(minifloat_meta), _lib.round_code(minifloat_meta.round_mode), _lib.stream_ptr(x.device)))
    return out
