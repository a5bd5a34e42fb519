"""MXFP format descriptors (API of src/mase_triton/mxfp/meta.py:11-126).

An MXFP tensor is a flat run of blocks; each block of ``block_size`` elements shares one
8-bit power-of-two scale (biased by 127) and stores one minifloat code per element, one code
per byte whatever the element width.
"""
from __future__ import annotations

import functools
from dataclasses import dataclass
from typing import Literal

from ..minifloat.meta import MinifloatMeta
from ..utils.meta import device_str, dtype_str, shape_tuple

LEGAL_SCALE_EXP_BITS = (8,)
LEGAL_ELEMENT_EXP_FRAC_BITS = ((4, 3), (5, 2), (2, 3), (3, 2), (2, 1))


@dataclass(frozen=True)
class MXFPMeta:
    block_size: int
    scale_exp_bits: int
    element_exp_bits: int
    element_frac_bits: int
    element_is_finite: bool
    round_mode: Literal["rn", "ru", "rd", "rz"]
    tag: str = ""

    def __post_init__(self):
        assert self.scale_exp_bits in LEGAL_SCALE_EXP_BITS, (
            f"Invalid exponent bits: {self.scale_exp_bits}. Legal values are: {LEGAL_SCALE_EXP_BITS}.")
        pair = (self.element_exp_bits, self.element_frac_bits)
        assert pair in LEGAL_ELEMENT_EXP_FRAC_BITS, (
            f"Invalid element exponent and fraction bits: {pair[0]}, {pair[1]}. "
            f"Legal values are: {LEGAL_ELEMENT_EXP_FRAC_BITS}.")

    @functools.cached_property
    def element_meta(self) -> MinifloatMeta:
        """The minifloat format of one element."""
        return MinifloatMeta(exp_bits=self.element_exp_bits, frac_bits=self.element_frac_bits,
                             is_finite=self.element_is_finite, round_mode=self.round_mode)


@dataclass(frozen=True)
class MXFPTensorMeta:
    """What is needed to turn (scales, elements) back into the original tensor."""

    device: str
    dtype: str
    shape: tuple[int, ...]
    block_dim: int
    meta: MXFPMeta

    def __post_init__(self):
        object.__setattr__(self, "device", device_str(self.device))
        object.__setattr__(self, "dtype", dtype_str(self.dtype))
        object.__setattr__(self, "shape", shape_tuple(self.shape))

    def create(self, device=None, dtype=None, shape=None, block_dim: int | None = None,
               meta: MXFPMeta | None = None) -> "MXFPTensorMeta":
        """Copy with some fields replaced."""
        return MXFPTensorMeta(
            device=self.device if device is None else device,
            dtype=self.dtype if dtype is None else dtype,
            shape=self.shape if shape is None else shape,
            block_dim=self.block_dim if block_dim is None else block_dim,
            meta=self.meta if meta is None else meta,
        )


def _preset(exp_bits: int, frac_bits: int, tag: str) -> MXFPMeta:
    return MXFPMeta(block_size=32, scale_exp_bits=8, element_exp_bits=exp_bits, element_frac_bits=frac_bits,
                    element_is_finite=True, round_mode="rn", tag=tag)


MXFP8_E4M3_fn = _preset(4, 3, "MXFP8_E4M3_fn")
MXFP8_E5M2_fn = _preset(5, 2, "MXFP8_E5M2_fn")
OCP_MXFP6_E2M3 = _preset(2, 3, "OCP_MXFP6_E2M3")
OCP_MXFP6_E3M2 = _preset(3, 2, "OCP_MXFP6_E3M2")
OCP_MXFP4_E2M1 = _preset(2, 1, "OCP_MXFP4_E2M1")
