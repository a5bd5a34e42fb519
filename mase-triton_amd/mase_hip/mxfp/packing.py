"""Bit-packed storage form of MXFP element codes and a serialisable form of a quantised layer.

The reference keeps one byte per element code in memory and in ``state_dict`` and leaves the
tensor metas out of it (src/mase_triton/mxfp/layers.py:69-80), so a stored layer can only be
rebuilt by code that still knows its shapes and formats.  Here a layer exports to a plain dict
of tensors, strings and integers (loadable with ``torch.load(..., weights_only=True)``), with
4-bit codes stored two to a byte and 6-bit codes four to three bytes; importing restores the
reference's one-byte layout bit for bit.
"""
from __future__ import annotations

import torch
from torch import Tensor

from .. import _lib
from .meta import MXFPMeta, MXFPTensorMeta


def code_bits(mxfp_meta: MXFPMeta) -> int:
    """Significant bits of an element code: sign + exponent + fraction."""
    return 1 + mxfp_meta.element_exp_bits + mxfp_meta.element_frac_bits


def packed_nbytes(n_elements: int, mxfp_meta: MXFPMeta) -> int:
    return n_elements * code_bits(mxfp_meta) // 8


def pack_elements(elements: Tensor, mxfp_meta: MXFPMeta) -> Tensor:
    """uint8 codes (any shape, one per byte) -> flat uint8 bit stream, code i at bits
    [w*i, w*i + w) with w = ``code_bits``.  8-bit formats are returned flattened, unchanged."""
    assert elements.dtype == torch.uint8
    bits = code_bits(mxfp_meta)
    flat = elements.reshape(-1)
    if bits == 8:
        return flat.clone()
    _lib.require_gpu(elements, "elements")
    flat = _lib.dense(flat)
    n = flat.numel()
    assert n % 16 == 0, "element count must be a multiple of 16"
    packed = torch.empty(n * bits // 8, dtype=torch.uint8, device=flat.device)
    with _lib.on_device(flat.device):
        _lib.check(_lib.load().mase_hip_pack_codes(flat.data_ptr(), packed.data_ptr(), n, bits, _lib.stream_ptr(flat.device)))
    return packed


def unpack_elements(packed: Tensor, mxfp_meta: MXFPMeta, n_elements: int) -> Tensor:
    """Inverse of :func:`pack_elements`: uint8 [n / B, B], the layout of ``extract_mxfp_components``."""
    assert packed.dtype == torch.uint8 and packed.ndim == 1
    bits = code_bits(mxfp_meta)
    assert packed.numel() == n_elements * bits // 8
    B = mxfp_meta.block_size
    if bits == 8:
        return packed.clone().view(n_elements // B, B)
    _lib.require_gpu(packed, "packed elements")
    packed = _lib.dense(packed)
    assert n_elements % 16 == 0
    elements = torch.empty(n_elements, dtype=torch.uint8, device=packed.device)
    with _lib.on_device(packed.device):
        _lib.check(_lib.load().mase_hip_unpack_codes(packed.data_ptr(), elements.data_ptr(), n_elements, bits,
                                                     _lib.stream_ptr(packed.device)))
    return elements.view(n_elements // B, B)


# ----------------------------------------------------------------------------- plain-dict metas
def meta_to_dict(meta: MXFPMeta) -> dict:
    return {"block_size": meta.block_size, "scale_exp_bits": meta.scale_exp_bits,
            "element_exp_bits": meta.element_exp_bits, "element_frac_bits": meta.element_frac_bits,
            "element_is_finite": bool(meta.element_is_finite), "round_mode": meta.round_mode, "tag": meta.tag}


def meta_from_dict(d: dict) -> MXFPMeta:
    return MXFPMeta(block_size=int(d["block_size"]), scale_exp_bits=int(d["scale_exp_bits"]),
                    element_exp_bits=int(d["element_exp_bits"]), element_frac_bits=int(d["element_frac_bits"]),
                    element_is_finite=bool(d["element_is_finite"]), round_mode=str(d["round_mode"]), tag=str(d.get("tag", "")))


def tensor_meta_to_dict(tm: MXFPTensorMeta) -> dict:
    return {"device": tm.device, "dtype": tm.dtype, "shape": list(tm.shape), "block_dim": int(tm.block_dim),
            "meta": meta_to_dict(tm.meta)}


def tensor_meta_from_dict(d: dict, device=None) -> MXFPTensorMeta:
    return MXFPTensorMeta(device=d["device"] if device is None else device, dtype=d["dtype"], shape=tuple(d["shape"]),
                          block_dim=int(d["block_dim"]), meta=meta_from_dict(d["meta"]))


# ----------------------------------------------------------------------------- components <-> dict
def export_components(scales: Tensor, elements: Tensor, tensor_meta: MXFPTensorMeta) -> dict:
    """(scales, elements, tensor_meta) -> {"scales", "elements_packed", "tensor_meta"}."""
    return {"scales": scales.reshape(-1).clone(), "elements_packed": pack_elements(elements, tensor_meta.meta),
            "tensor_meta": tensor_meta_to_dict(tensor_meta)}


def import_components(d: dict, device=None) -> tuple[Tensor, Tensor, MXFPTensorMeta]:
    """Inverse of :func:`export_components`; tensors are moved to ``device`` when given."""
    tm = tensor_meta_from_dict(d["tensor_meta"], device=device)
    n = 1
    for s in tm.shape:
        n *= s
    scales, packed = d["scales"], d["elements_packed"]
    if device is not None:
        scales, packed = scales.to(device), packed.to(device)
    elements = unpack_elements(packed, tm.meta, n)
    return scales.view(-1, 1), elements, tm
