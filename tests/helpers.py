"""Shared test helpers: bit-pattern views, NaN-aware comparison, golden-file access."""
from __future__ import annotations

import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

TORCH_DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
PRESETS = {  # tag -> (exp_bits, frac_bits)
    "MXFP8_E4M3_fn": (4, 3),
    "MXFP8_E5M2_fn": (5, 2),
    "OCP_MXFP6_E2M3": (2, 3),
    "OCP_MXFP6_E3M2": (3, 2),
    "OCP_MXFP4_E2M1": (2, 1),
}


def golden(name: str):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def from_bits(a: np.ndarray, dtype_name: str) -> torch.Tensor:
    signed = a.view(np.int32 if dtype_name == "float32" else np.int16)
    return torch.from_numpy(signed.copy()).view(TORCH_DT[dtype_name])


def bits_of(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy().view(np.uint32)
    if t.dtype in (torch.bfloat16, torch.float16, torch.uint16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.uint8:
        return t.numpy()
    raise TypeError(t.dtype)


def codes_tensor(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.uint16)


def _nan_mask(bits: np.ndarray, dtype_name: str) -> np.ndarray:
    if dtype_name == "float32":
        return (bits & 0x7FFFFFFF) > 0x7F800000
    if dtype_name == "bfloat16":
        return (bits & 0x7FFF) > 0x7F80
    return (bits & 0x7FFF) > 0x7C00


def mismatches(got_bits: np.ndarray, want_bits: np.ndarray, dtype_name: str) -> np.ndarray:
    """Indices where the bit patterns differ, treating any NaN as equal to any NaN (NaN sign
    and payload are not stable even between torch's own CPU code paths)."""
    got_bits, want_bits = got_bits.reshape(-1), want_bits.reshape(-1)
    same = (got_bits == want_bits) | (_nan_mask(got_bits, dtype_name) & _nan_mask(want_bits, dtype_name))
    return np.nonzero(~same)[0]


def assert_bits_equal(got: torch.Tensor, want, dtype_name: str | None = None, what: str = ""):
    dtype_name = dtype_name or str(got.dtype).removeprefix("torch.")
    gb = bits_of(got)
    wb = want if isinstance(want, np.ndarray) else bits_of(want)
    assert gb.size == wb.size, f"{what}: size {gb.size} != {wb.size}"
    bad = mismatches(gb, wb, dtype_name)
    if bad.size:
        show = [(int(i), hex(int(gb.reshape(-1)[i])), hex(int(wb.reshape(-1)[i]))) for i in bad[:8]]
        raise AssertionError(f"{what}: {bad.size} of {gb.size} differ; first (index, got, want): {show}")


def assert_int_equal(got: torch.Tensor, want, what: str = ""):
    g = bits_of(got).reshape(-1)
    w = (want if isinstance(want, np.ndarray) else bits_of(want)).reshape(-1)
    assert g.size == w.size, f"{what}: size {g.size} != {w.size}"
    bad = np.nonzero(g != w)[0]
    if bad.size:
        show = [(int(i), hex(int(g[i])), hex(int(w[i]))) for i in bad[:8]]
        raise AssertionError(f"{what}: {bad.size} of {g.size} differ; first (index, got, want): {show}")


def parse_cfg_key(key: str):
    """'e4m3_fin_rn' -> (4, 3, True, 'rn')"""
    em, fin, rnd = key.split("_")
    e, m = em[1:].split("m")
    return int(e), int(m), fin == "fin", rnd
