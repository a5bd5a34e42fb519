"""Tensor-op restatement of the reference's CPU ("fake") path.  TEST INFRASTRUCTURE ONLY.

The same algorithm as ``mase_oracle.c`` but expressed, like the reference, as whole-tensor
torch operations in fp32/int32 (frexp, log2, floor, exp2, divide, round-half-even), so that
its cost profile on a CPU is that of the reference's own CPU path.  It serves two purposes:

* an independent cross-check of the integer restatement (tests compare the two and both
  against the golden vectors);
* the CPU baseline that the benchmark times beside each GPU figure.

Follows (paths relative to the reference checkout):
  minifloat_encode  <- src/mase_triton/minifloat/fake.py:7-78
  minifloat_decode  <- src/mase_triton/minifloat/fake.py:81-125
  mxfp_split        <- src/mase_triton/mxfp/fake.py:11-59
  mxfp_join         <- src/mase_triton/mxfp/fake.py:62-79
  mxfp_linear_xq_wq <- src/mase_triton/mxfp/functional/linear.py:36-64 ("separate" backend)
"""
from __future__ import annotations

import torch
from torch import Tensor

_I32 = torch.int32
_F32 = torch.float32


def _layout(exp_bits: int, frac_bits: int, is_finite: bool):
    bias = 2 ** (exp_bits - 1) - 1
    top_field = 2 ** exp_bits - (1 if is_finite else 2)
    return bias, top_field, top_field - bias, 2 ** frac_bits - 1


def minifloat_encode(x: Tensor, exp_bits: int, frac_bits: int, is_finite: bool = True,
                     round_mode: str = "rn") -> Tensor:
    bias, top_field, top_exp, top_frac = _layout(exp_bits, frac_bits, is_finite)
    v = x.to(_F32)
    negative = v < 0
    magnitude = v.abs()
    tiny = (magnitude.view(_I32) & 0x7F800000) == 0          # zero or fp32 subnormal
    mant, expo = torch.where(tiny, 0.0, v).abs().frexp()      # mant in [0.5, 1)
    mant, expo = mant * 2, expo - 1
    too_small, too_big = expo < -bias, expo > top_exp
    field = expo + bias
    bits = mant.view(_I32) & 0x7FFFFF
    if round_mode == "rz":
        frac = bits >> (23 - frac_bits)
    else:
        scaled = (bits >> 8).to(_F32) / float(1 << (15 - frac_bits))
        if round_mode == "rn":
            scaled = scaled.round()
        elif round_mode == "ru":
            scaled = scaled.ceil()
        elif round_mode == "rd":
            scaled = scaled.floor()
        else:
            raise ValueError(f"Unknown rounding mode: {round_mode}")
        frac = scaled.to(_I32)
    lowest_binade = (field == 0) & (frac != 0)
    frac = torch.where(lowest_binade, (frac | (1 << frac_bits)) >> 1, frac)
    for cond, f_val, e_val in ((too_small, 0, 0), (too_big, top_frac, top_field), (tiny, 0, 0)):
        frac = torch.where(cond, f_val, frac)
        field = torch.where(cond, e_val, field)
    if not is_finite:
        inf, nan = v.isinf(), v.isnan()
        frac = torch.where(nan, top_frac, torch.where(inf, 0, frac))
        field = torch.where(inf | nan, top_field, field)
    code = (field << frac_bits) | frac
    code = torch.where(negative, code + (1 << (exp_bits + frac_bits)), code)
    return code.to(torch.uint16)


def minifloat_decode(codes: Tensor, exp_bits: int, frac_bits: int, is_finite: bool,
                     output_dtype: torch.dtype) -> Tensor:
    assert codes.dtype == torch.uint16
    bias = 2 ** (exp_bits - 1) - 1
    c = codes.to(_I32)
    negative = (c & (1 << (exp_bits + frac_bits))) != 0
    c = c & 0x7FFF
    field = (c >> frac_bits) & (2 ** exp_bits - 1)
    frac = c & (2 ** frac_bits - 1)
    is_zero = (field == 0) & (frac == 0)
    is_sub = (field == 0) & (frac != 0)
    power = torch.exp2(torch.where(is_sub, field - bias + 1, field - bias))
    significand = frac.to(_F32) / float(1 << frac_bits)
    significand = torch.where(is_sub, significand, significand + 1.0)
    y = power * significand
    if not is_finite:
        top = field == (2 ** exp_bits - 1)
        y = torch.where(top & (frac == 0), float("inf"), y)
        y = torch.where(top & (frac != 0), float("nan"), y)
    y = torch.where(is_zero, 0.0, y)
    y = torch.where(negative, -y, y)
    return y.to(output_dtype)


def mxfp_split(x: Tensor, block_size: int, exp_bits: int, frac_bits: int,
               is_finite: bool = True, round_mode: str = "rn") -> tuple[Tensor, Tensor]:
    _, _, top_exp, _ = _layout(exp_bits, frac_bits, is_finite)
    v = x.float().flatten()
    assert v.numel() % block_size == 0
    v = v.reshape(-1, block_size)
    tiny = (v.view(_I32) & 0x7F800000) == 0
    shared = v.abs().max(dim=1, keepdim=True).values.log2().floor().to(_I32)
    shared -= top_exp
    shared = shared.clamp(-127, 128)
    scale_u8 = torch.where(tiny.all(dim=1, keepdim=True), 0, shared + 127).to(torch.uint8)
    quotient = torch.where(tiny, 0.0, v / torch.exp2(shared))
    elements = minifloat_encode(quotient, exp_bits, frac_bits, is_finite, round_mode)
    return scale_u8, elements.view(torch.uint16).to(torch.uint8)


def mxfp_join(scales: Tensor, elements: Tensor, exp_bits: int, frac_bits: int, is_finite: bool,
              output_dtype: torch.dtype) -> Tensor:
    assert scales.dtype == torch.uint8 and elements.dtype == torch.uint8
    factor = torch.exp2(scales.to(_I32) - 127)
    values = minifloat_decode(elements.to(torch.uint16), exp_bits, frac_bits, is_finite, _F32)
    return (values * factor).flatten().to(output_dtype)


def mxfp_qdq_lastdim(x: Tensor, block_size: int, exp_bits: int, frac_bits: int) -> Tensor:
    """quantize-dequantize with blocks along the last (contiguous) dimension."""
    sc, el = mxfp_split(x, block_size, exp_bits, frac_bits)
    return mxfp_join(sc, el, exp_bits, frac_bits, True, x.dtype).reshape(x.shape)


def mxfp_linear_xq_wq(x: Tensor, w_scales: Tensor, w_elements: Tensor, w_shape, w_dtype,
                      x_fmt: tuple[int, int], w_fmt: tuple[int, int], block_size: int = 32,
                      bias: Tensor | None = None) -> Tensor:
    x_dq = mxfp_qdq_lastdim(x, block_size, *x_fmt)
    w_dq = mxfp_join(w_scales, w_elements, w_fmt[0], w_fmt[1], True, w_dtype).reshape(w_shape)
    return torch.nn.functional.linear(x_dq, w_dq, bias)
