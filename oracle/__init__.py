"""CPU checker for the MXFP / minifloat path.  TEST INFRASTRUCTURE ONLY.

Two independent restatements of the reference's PyTorch "fake" path live here:

* ``mase_oracle.c``  - integer arithmetic in plain C (fast; loaded through ctypes below);
* ``torch_fake.py``  - the same algorithm as a sequence of torch tensor ops on CPU tensors,
  which is also what the CPU-baseline timing in the benchmark runs.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this package.
The shipped GPU path never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libmase_oracle.so")
_lib = None

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
ROUND_CODE = {"rn": 0, "ru": 1, "rd": 2, "rz": 3}


def build(force: bool = False) -> str:
    """Compile mase_oracle.c with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "mase_oracle.c"))
    ):
        subprocess.run(["make", "-s", "-C", _HERE, "-B"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        i32, i64, vp = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p
        _lib.orc_extract_minifloat.argtypes = [vp, i32, vp, i64, i32, i32, i32, i32]
        _lib.orc_compose_minifloat.argtypes = [vp, vp, i32, i64, i32, i32, i32]
        _lib.orc_qdq_minifloat.argtypes = [vp, i32, vp, i32, i64, i32, i32, i32, i32]
        _lib.orc_extract_mxfp.argtypes = [vp, i32, vp, vp, i64, i32, i32, i32, i32, i32]
        _lib.orc_compose_mxfp.argtypes = [vp, vp, vp, i32, i64, i32, i32, i32, i32]
        _lib.orc_qdq_mxfp.argtypes = [vp, i32, vp, i32, i64, i32, i32, i32, i32, i32]
        _lib.orc_matmul_nt_f32.argtypes = [vp, vp, vp, i64, i64, i64]
        for name in ("orc_extract_minifloat", "orc_compose_minifloat", "orc_qdq_minifloat",
                     "orc_extract_mxfp", "orc_compose_mxfp", "orc_qdq_mxfp", "orc_matmul_nt_f32"):
            getattr(_lib, name).restype = None
    return _lib


def _cpu(t: torch.Tensor) -> torch.Tensor:
    assert t.device.type == "cpu", "the checker runs on CPU tensors"
    return t.contiguous()


def extract_minifloat(x: torch.Tensor, exp_bits: int, frac_bits: int, is_finite: bool = True,
                      round_mode: str = "rn") -> torch.Tensor:
    x = _cpu(x)
    codes = torch.empty(x.shape, dtype=torch.uint16)
    lib().orc_extract_minifloat(x.data_ptr(), DTYPE_CODE[x.dtype], codes.data_ptr(), x.numel(),
                                exp_bits, frac_bits, int(is_finite), ROUND_CODE[round_mode])
    return codes


def compose_minifloat(codes: torch.Tensor, exp_bits: int, frac_bits: int, is_finite: bool,
                      output_dtype: torch.dtype) -> torch.Tensor:
    codes = _cpu(codes)
    assert codes.dtype == torch.uint16
    out = torch.empty(codes.shape, dtype=output_dtype)
    lib().orc_compose_minifloat(codes.data_ptr(), out.data_ptr(), DTYPE_CODE[output_dtype],
                                codes.numel(), exp_bits, frac_bits, int(is_finite))
    return out


def qdq_minifloat(x, exp_bits, frac_bits, is_finite=True, round_mode="rn", output_dtype=None):
    x = _cpu(x)
    output_dtype = output_dtype or x.dtype
    out = torch.empty(x.shape, dtype=output_dtype)
    lib().orc_qdq_minifloat(x.data_ptr(), DTYPE_CODE[x.dtype], out.data_ptr(),
                            DTYPE_CODE[output_dtype], x.numel(), exp_bits, frac_bits,
                            int(is_finite), ROUND_CODE[round_mode])
    return out


def extract_mxfp(x: torch.Tensor, block_size: int, exp_bits: int, frac_bits: int,
                 is_finite: bool = True, round_mode: str = "rn"):
    x = _cpu(x).flatten()
    n = x.numel()
    assert n % block_size == 0
    scales = torch.empty((n // block_size, 1), dtype=torch.uint8)
    elements = torch.empty((n // block_size, block_size), dtype=torch.uint8)
    lib().orc_extract_mxfp(x.data_ptr(), DTYPE_CODE[x.dtype], scales.data_ptr(),
                           elements.data_ptr(), n, block_size, exp_bits, frac_bits,
                           int(is_finite), ROUND_CODE[round_mode])
    return scales, elements


def compose_mxfp(scales: torch.Tensor, elements: torch.Tensor, block_size: int, exp_bits: int,
                 frac_bits: int, is_finite: bool, output_dtype: torch.dtype) -> torch.Tensor:
    scales, elements = _cpu(scales), _cpu(elements)
    assert scales.dtype == torch.uint8 and elements.dtype == torch.uint8
    n = elements.numel()
    out = torch.empty((n,), dtype=output_dtype)
    lib().orc_compose_mxfp(scales.data_ptr(), elements.data_ptr(), out.data_ptr(),
                           DTYPE_CODE[output_dtype], n, block_size, exp_bits, frac_bits,
                           int(is_finite))
    return out


def qdq_mxfp(x, block_size, exp_bits, frac_bits, is_finite=True, round_mode="rn",
             output_dtype=None):
    x = _cpu(x)
    output_dtype = output_dtype or x.dtype
    out = torch.empty(x.shape, dtype=output_dtype)
    lib().orc_qdq_mxfp(x.data_ptr(), DTYPE_CODE[x.dtype], out.data_ptr(),
                       DTYPE_CODE[output_dtype], x.numel(), block_size, exp_bits, frac_bits,
                       int(is_finite), ROUND_CODE[round_mode])
    return out


def matmul_nt(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """a [M,K] @ b[N,K]^T with float64 accumulation, fp32 result (small sizes only)."""
    a, b = _cpu(a.float()), _cpu(b.float())
    out = torch.empty((a.shape[0], b.shape[0]), dtype=torch.float32)
    lib().orc_matmul_nt_f32(a.data_ptr(), b.data_ptr(), out.data_ptr(), a.shape[0], b.shape[0],
                            a.shape[1])
    return out
