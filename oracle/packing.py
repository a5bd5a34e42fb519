"""CPU checker for the bit-packed storage form of element codes.  TEST INFRASTRUCTURE ONLY.

The packed form is a little-endian bit stream: code i occupies bits [w*i, w*i + w) of the
buffer.  Restated here bit by bit with numpy (expand every code to its w bits, least
significant first, concatenate, regroup into bytes), independently of the word-level shifts the
HIP kernels use.  The reference has no packed form (it stores one byte per code,
src/mase_triton/mxfp/layers.py:69-80); what pins this checker is the definition above, the
hand-computed vectors in tests/test_oracle_golden.py and the round trip.
"""
from __future__ import annotations

import numpy as np


def pack_codes(codes: np.ndarray, bits: int) -> np.ndarray:
    codes = np.asarray(codes, dtype=np.uint8).reshape(-1)
    assert (codes.size * bits) % 8 == 0
    stream = ((codes[:, None] >> np.arange(bits, dtype=np.uint8)[None, :]) & 1).astype(np.uint8).reshape(-1)
    return np.packbits(stream, bitorder="little")


def unpack_codes(packed: np.ndarray, bits: int, n: int) -> np.ndarray:
    packed = np.asarray(packed, dtype=np.uint8).reshape(-1)
    assert packed.size * 8 == n * bits
    stream = np.unpackbits(packed, bitorder="little").reshape(n, bits).astype(np.uint16)
    return (stream << np.arange(bits, dtype=np.uint16)[None, :]).sum(axis=1).astype(np.uint8)
