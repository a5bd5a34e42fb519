"""Minifloat format descriptors (API of src/mase_triton/minifloat/meta.py:48-124).

A format is ``1 + exp_bits + frac_bits`` wide.  ``is_finite=True`` (all "_fn" presets) means
the all-ones exponent is an ordinary binade: no code is spent on inf or NaN, so FP8_E4M3_fn
tops out at 480 and FP8_E5M2_fn at 114688.
"""
from __future__ import annotations

import functools
from dataclasses import dataclass
from typing import Literal

import torch

from ..utils.meta import device_str, dtype_str, shape_tuple


@dataclass(frozen=True)
class MinifloatMeta:
    exp_bits: int
    frac_bits: int
    is_finite: bool
    round_mode: Literal["rn", "rd", "ru", "rz"]
    tag: str = ""

    def __post_init__(self):
        assert self.exp_bits > 0
        assert self.frac_bits > 0
        assert self.exp_bits + self.frac_bits < 16  # codes travel as uint16

    @property
    def _bias(self) -> int:
        return 2 ** (self.exp_bits - 1) - 1

    @functools.cached_property
    def n_bits(self) -> int:
        return 1 + self.exp_bits + self.frac_bits

    @functools.cached_property
    def max_normal(self) -> float:
        top_field = 2 ** self.exp_bits - (1 if self.is_finite else 2)
        return 2.0 ** (top_field - self._bias) * (2.0 - 2.0 ** -self.frac_bits)

    @functools.cached_property
    def min_normal(self) -> float:
        return 2.0 ** (1 - self._bias)

    @functools.cached_property
    def max_subnormal(self) -> float:
        return 2.0 ** (1 - self._bias) * (1.0 - 2.0 ** -self.frac_bits)

    @functools.cached_property
    def min_subnormal(self) -> float:
        return 2.0 ** (1 - self._bias - self.frac_bits)


def _preset(exp_bits: int, frac_bits: int, tag: str) -> MinifloatMeta:
    return MinifloatMeta(exp_bits=exp_bits, frac_bits=frac_bits, is_finite=True, round_mode="rn", tag=tag)


FP8_E4M3_fn = _preset(4, 3, "FP8_E4M3_fn")
FP8_E5M2_fn = _preset(5, 2, "FP8_E5M2_fn")
FP6_E2M3_fn = _preset(2, 3, "FP6_E2M3_fn")
FP6_E3M2_fn = _preset(3, 2, "FP6_E3M2_fn")
FP4_E2M1_fn = _preset(2, 1, "FP4_E2M1_fn")


@dataclass
class MinifloatTensorMeta:
    """What is needed to turn stored codes back into the original tensor."""

    device: str
    dtype: str
    shape: tuple[int, ...]
    meta: MinifloatMeta

    def __post_init__(self):
        self.device = device_str(self.device)
        self.dtype = dtype_str(self.dtype)
        self.shape = shape_tuple(self.shape)

    def create(self, device=None, dtype=None, shape=None, meta: MinifloatMeta | None = None) -> "MinifloatTensorMeta":
        """Copy with some fields replaced."""
        return MinifloatTensorMeta(
            device=self.device if device is None else device,
            dtype=self.dtype if dtype is None else dtype,
            shape=self.shape if shape is None else shape,
            meta=self.meta if meta is None else meta,
        )
