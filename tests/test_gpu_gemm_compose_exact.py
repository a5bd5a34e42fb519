"""The GEMM's in-register compose, bit for bit.

The other GEMM tests hold the product to a relative Frobenius error, which a wrong low bit in the
composed weights would pass.  Here A selects single columns of W (rows of an identity matrix), so
y[m, n] = W_dq[n, m % K] with nothing to round: every kernel of the dispatch must reproduce the
reference's compose table (tests/golden/mxfp_compose_table.npz, written from the reference's own
compose_mxfp_tensor: every scale byte x every code) exactly.  Rows of W hold one scale each, every
code of the format, so all (scale, code) pairs pass through every kernel.
"""
import numpy as np
import pytest
import torch

from helpers import PRESETS, bits_of, golden, mismatches

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def mh():
    import mase_hip.mxfp.kernels as mxk
    from mase_hip import _lib
    from mase_hip.mxfp import meta

    _lib.load()

    class NS:
        pass

    ns = NS()
    ns.mxk, ns.meta = mxk, meta
    return ns


def expected_bits(table_bits: np.ndarray, dtype_name: str, scales: np.ndarray, codes: np.ndarray, M: int, K: int, off: int) -> np.ndarray:
    """y[m, n] for A[m, k] = (k == (m + off) % K): the selected value, +0 for a selected -0 (the sum starts from +0), and NaN
    wherever another element of the row is inf or NaN (0 * inf)."""
    w_bits = table_bits[scales[:, None], codes[None, :]]              # [N, K]
    if dtype_name == "float32":
        exp_all, frac_mask, sign, nan = 0x7F800000, 0x007FFFFF, 0x80000000, 0x7FC00000
    else:
        exp_all, frac_mask, sign, nan = 0x7F80, 0x007F, 0x8000, 0x7FC0
    nonfinite = (w_bits & exp_all) == exp_all                          # [N, K]
    n_bad = nonfinite.sum(axis=1)                                      # per row of W
    sel = (np.arange(M) + off) % K
    y = w_bits[:, sel].T.copy()                                        # [M, N]
    y[y == sign] = 0
    others_bad = (n_bad[None, :] - nonfinite[:, sel].T.astype(np.int64)) > 0
    y[others_bad] = nan
    return y


# (M, N, K): few rows on the 16-row and 32-row weight-streaming kernels, then 128 x 128, 256 x 128 and 512 x 128 tiles (the
# last with scales fetched 4 and 16 bytes at a time)
SHAPES = [(16, 256, 256), (64, 512, 256), (128, 256, 256), (256, 256, 256), (512, 8448, 256), (1024, 8448, 256), (1024, 8448, 512)]


@pytest.mark.parametrize("w_tag", list(PRESETS))
@pytest.mark.parametrize("MNK", SHAPES)
@pytest.mark.parametrize("odt", [torch.bfloat16, torch.float32])
def test_gemm_reproduces_the_compose_table(mh, w_tag, MNK, odt):
    M, N, K = MNK
    if odt == torch.float32 and (M not in (16, 256, 1024) or K != 256):
        pytest.skip("fp32 output: one shape per kernel family is enough")
    e, m = PRESETS[w_tag]
    n_codes = 1 << (1 + e + m)
    # the product is formed from bf16 operands: the composed weights are the reference's bf16 table whatever the output type
    table = golden("mxfp_compose_table.npz")[f"bfloat16_{w_tag}"]      # [scale, code] -> bf16 bits
    scales = (np.arange(N) * 37 % 256).astype(np.int64)                # every scale byte, spread over the rows
    codes = (np.arange(K) % n_codes).astype(np.int64)
    w_sc = torch.from_numpy(np.repeat(scales.astype(np.uint8)[:, None], K // 32, axis=1).copy())
    w_el = torch.from_numpy(np.repeat(codes.astype(np.uint8)[None, :], N, axis=0).copy())
    w_sc, w_el = w_sc.to(DEV), w_el.to(DEV)
    name = "float32" if odt == torch.float32 else "bfloat16"
    for off in range(0, K, M):   # few rows: several products, so that every column of W is selected once
        a = torch.zeros(M, K, dtype=torch.bfloat16)
        a[torch.arange(M), (torch.arange(M) + off) % K] = 1.0
        y = mh.mxk.mxfp_gemm(a.to(DEV), None, None, None, w_sc, w_el, getattr(mh.meta, w_tag), None, M, N, K, odt, split_k=False)
        torch.cuda.synchronize()
        want = expected_bits(table, "bfloat16", scales, codes, M, K, off)
        if odt == torch.float32:
            want = want.astype(np.uint32) << 16
        bad = mismatches(bits_of(y), want, name)
        if bad.size:
            i = bad[:8]
            rows, cols = i // N, i % N
            show = [(int(r), int(c), int(scales[c]), hex(int(codes[(r + off) % K])), hex(int(bits_of(y).reshape(-1)[j])),
                     hex(int(want.reshape(-1)[j]))) for r, c, j in zip(rows, cols, i)]
            raise AssertionError(f"offset {off}: {bad.size} of {M * N} differ; first (m, n, scale, code, got, want): {show}")
