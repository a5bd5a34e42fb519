"""ctypes binding of lib/libmase_hip.so (declarations: include/mase_hip.h at the repo root)."""
from __future__ import annotations

import contextlib
import ctypes
import os

import torch

from .dtype import ROUND_MODE_TO_CODE, TORCH_DTYPE_TO_CODE

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmase_hip.so")
_lib = None

_i32, _i64, _vp = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p

SIGNATURES = {
    "mase_hip_abi_version": (_i32, []),
    "mase_hip_last_error": (ctypes.c_char_p, []),
    "mase_hip_extract_minifloat": (_i32, [_vp, _i32, _vp, _i64, _i32, _i32, _i32, _i32, _vp]),
    "mase_hip_compose_minifloat": (_i32, [_vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp]),
    "mase_hip_qdq_minifloat": (_i32, [_vp, _i32, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _vp]),
    "mase_hip_extract_mxfp": (_i32, [_vp, _i32, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
    "mase_hip_compose_mxfp": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _vp]),
    "mase_hip_qdq_mxfp": (_i32, [_vp, _i32, _vp, _i32, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
    "mase_hip_extract_mxfp_strided": (_i32, [_vp, _i32, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
    "mase_hip_qdq_mxfp_strided": (_i32, [_vp, _i32, _vp, _i32, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
    "mase_hip_pack_codes": (_i32, [_vp, _vp, _i64, _i32, _vp]),
    "mase_hip_unpack_codes": (_i32, [_vp, _vp, _i64, _i32, _vp]),
    "mase_hip_mxfp_gemm": (_i32, [_vp, _i32, _vp, _vp, _i32, _i32, _vp, _vp, _i32, _i32, _vp, _i32,
                                  _vp, _i32, _i64, _i64, _i64, _i32, _vp]),
    "mase_hip_mxfp_gemm_ws": (_i32, [_vp, _i32, _vp, _vp, _i32, _i32, _vp, _vp, _i32, _i32, _vp, _i32,
                                     _vp, _i32, _i64, _i64, _i64, _i32, _vp, _i64, _vp]),
    "mase_hip_mxfp_gemm_workspace_bytes": (_i64, [_i32, _i64, _i64, _i64]),
    "mase_hip_mxfp_gemm_batched": (_i32, [_vp, _i32, _vp, _vp, _i32, _i32, _vp, _i32, _i64, _i64, _i64, _i32,
                                          _i64, _i64, _i64, _i64, _vp]),
    "mase_hip_mxfp_gemm_static_ws": (_i32, [_vp, _i32, _vp, _vp, _i32, _i32, _vp, _vp, _i32, _i32, _vp, _i32,
                                            _vp, _i32, _i64, _i64, _i64, _i32, _vp]),
    "mase_hip_scaled_padded_rows": (_i64, [_i64]),
    "mase_hip_scaled_operand_from_dense": (_i32, [_vp, _i32, _i32, _i32, _i64, _i64, _vp, _vp, _vp]),
    "mase_hip_scaled_operand_from_dense_minifloat": (_i32, [_vp, _i32, _i32, _i32, _i64, _i64, _vp, _vp, _vp]),
    "mase_hip_scaled_operand_from_swiglu": (_i32, [_vp, _vp, _i32, _i64, _i32, _i32, _i64, _i64, _vp, _vp, _vp]),
    "mase_hip_scaled_operand_from_mxfp": (_i32, [_vp, _vp, _i32, _i32, _i64, _i64, _vp, _vp, _vp]),
    "mase_hip_mxfp_gemm_scaled": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _vp, _i32, _i64, _i64, _i64, _vp]),
    "mase_hip_mxfp_gemm_scaled_ws": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _vp, _i32, _i64, _i64, _i64, _vp, _i64, _vp]),
    "mase_hip_mxfp_gemm_scaled_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "mase_hip_mxfp_linear_scaled_scratch_bytes": (_i64, [_i64, _i64, _i64]),
    "mase_hip_mxfp_linear_scaled": (_i32, [_vp, _i32, _i32, _i32, _i32, _vp, _vp, _vp, _i32, _vp, _i32, _i64, _i64, _i64, _vp, _i64, _vp]),
    "mase_hip_mxfp_gemm_prepared_w": (_i32, [_vp, _i32, _vp, _vp, _vp, _i32, _vp, _i32, _i64, _i64, _i64, _vp]),
}


def library_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load the HIP library; raises if it has not been built (there is no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_PATH} is missing: build it with `python mase-triton_amd/build.py` "
                "(mase_hip has no other implementation to fall back to)")
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


class MaseHipError(RuntimeError):
    pass


def check(rc: int) -> None:
    if rc == 0:
        return
    msg = load().mase_hip_last_error().decode()
    if rc == -1:
        raise ValueError(f"mase_hip: invalid argument: {msg}")
    if rc == -2:
        raise NotImplementedError(f"mase_hip: unsupported: {msg}")
    raise MaseHipError(f"mase_hip: HIP error: {msg}")


def require_gpu(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(
            f"mase_hip: {what} is on {t.device}; this package only runs HIP kernels on a GPU "
            "and has no CPU implementation")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return TORCH_DTYPE_TO_CODE[dtype]
    except KeyError:
        raise TypeError(f"mase_hip: unsupported dtype {dtype}; use float32, float16 or bfloat16") from None


def round_code(mode: str) -> int:
    try:
        return ROUND_MODE_TO_CODE[mode]
    except KeyError:
        raise ValueError(f"Unknown rounding mode: {mode}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device: torch.device) -> int:
    """hipStream_t of torch's current stream on ``device`` (the raw getter costs a fraction of building a Stream object)."""
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


_NO_SWITCH = contextlib.nullcontext()


def on_device(device: torch.device):
    """Context in which ``device`` is the current HIP device; nothing to do (and nothing paid) when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


# how often dense() had to copy an operand because its storage was not 16-byte aligned (a full extra pass over it)
realignment_copies = 0


def dense(t: torch.Tensor) -> torch.Tensor:
    """Contiguous and 16-byte aligned (what the vector kernels assume).  A misaligned operand (a view that starts at an odd
    offset of its storage) is copied: counted in ``realignment_copies``, and the first one is reported with a warning."""
    global realignment_copies
    t = t.contiguous()
    if t.data_ptr() % 16:
        if realignment_copies == 0:
            import warnings

            warnings.warn("mase_hip: an operand is not 16-byte aligned and is copied before the kernel runs (further copies are "
                          "counted in mase_hip._lib.realignment_copies without a warning)", RuntimeWarning, stacklevel=3)
        realignment_copies += 1
        t = t.clone()
    return t


def as_float_input(t: torch.Tensor) -> torch.Tensor:
    """Kernels read float32 / float16 / bfloat16; anything else is widened to float32 first,
    as the reference's fake path does with ``.float()``."""
    return t if t.dtype in TORCH_DTYPE_TO_CODE else t.to(torch.float32)
