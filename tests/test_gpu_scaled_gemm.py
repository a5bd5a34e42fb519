"""GPU parity tests for the block-scaled route of the MXFP GEMM: operands kept as FP8 bytes and E8M0 scales up to the
matrix unit (mase_hip_scaled_operand_from_dense / _from_mxfp, mase_hip_mxfp_gemm_scaled).

What is checked, against the CPU checker's components of the same inputs:
  * the prepared operand holds the reference's values: bit for bit in the formats that are embedded into E4M3 bytes,
    and for E4M3 itself in every block that does not hold the code S.1111.111; blocks that do are stored one scale
    step up with halved codes, by a rule restated here on integers, and no element moves by more than 2^-14 of its
    block's largest;
  * the product against float64 dequantise-then-matmul of the checker's values: relative Frobenius error <= 1e-3 for
    16-bit outputs (compared with the reference rounded to that type) and 1e-4 for fp32 outputs (measured 1 - 2e-5:
    the matrix unit adds a block's 32 products with fewer bits than a chain of fp32 FMAs keeps);
  * identity times W returns W's dequantised values exactly;
  * inf / NaN blocks poison exactly the rows (columns) they poison in dequantise-then-matmul;
  * the operand formed from silu(gate) * up inside the kernel equals the one built from torch's two bf16 operations.
"""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import PRESETS

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32_TOL = 1e-4
SCALED_TAGS = ["MXFP8_E4M3_fn", "OCP_MXFP6_E3M2", "OCP_MXFP6_E2M3", "OCP_MXFP4_E2M1"]


def rel_fro(y, y_ref):
    y, y_ref = y.double().cpu(), y_ref.double().cpu()
    return ((y - y_ref).norm() / y_ref.norm()).item()


@pytest.fixture(scope="module")
def mh():
    import mase_hip.mxfp.functional as F
    import mase_hip.mxfp.kernels as mxk
    from mase_hip import _lib
    from mase_hip.mxfp import meta
    from mase_hip.mxfp.layers import MXFPLinearPTQ

    _lib.load()

    class NS:
        pass

    ns = NS()
    ns.F, ns.mxk, ns.meta, ns.MXFPLinearPTQ = F, mxk, meta, MXFPLinearPTQ
    return ns


# ---------------------------------------------------------------- the prepared operand, decoded on the CPU
def decode_e4m3(codes: np.ndarray) -> np.ndarray:
    """OCP E4M3 bytes (no NaN code expected) -> float64."""
    c = codes.astype(np.int64)
    s, e, m = c >> 7, (c >> 3) & 15, c & 7
    v = np.where(e == 0, m / 8.0 * 2.0 ** -6, (1 + m / 8.0) * 2.0 ** (e - 7.0))
    return np.where(s == 1, -v, v)


def decode_fmt(codes: np.ndarray, E: int, M: int) -> np.ndarray:
    """Codes of the reference's finite (E, M) format -> float64 (minifloat/fake.py:97-123)."""
    c = codes.astype(np.int64)
    bias = (1 << (E - 1)) - 1
    s, e, m = (c >> (E + M)) & 1, (c >> M) & ((1 << E) - 1), c & ((1 << M) - 1)
    v = np.where(e == 0, m / float(1 << M) * 2.0 ** (1 - bias), (1 + m / float(1 << M)) * 2.0 ** (e.astype(np.float64) - bias))
    return np.where(s == 1, -v, v)


def operand_arrays(op):
    """(codes [rows, K] uint8, scales [rows, K/32] uint8) of a ScaledOperand, padding rows dropped."""
    codes = op.codes[: op.rows].cpu().numpy()
    sc = op.scales.cpu().numpy().view(np.uint32)                      # [K/128, rows_pad]
    by = np.stack([(sc >> (8 * b)) & 0xFF for b in range(4)], axis=-1)  # [K/128, rows_pad, 4]
    scales = by.transpose(1, 0, 2).reshape(sc.shape[1], -1)[: op.rows].astype(np.uint8)
    return codes, scales


def halved(codes: np.ndarray) -> np.ndarray:
    """The documented re-encoding of an E4M3 block one scale step up."""
    c = codes.astype(np.int64)
    sign, mag = c & 0x80, c & 0x7F
    small = mag // 2 + ((mag & 1) & ((mag // 2) & 1))   # below 16 the magnitude is linear in the value: halve, ties to even
    return (sign | np.where(mag >= 16, mag - 8, small)).astype(np.uint8)


def mixed_inputs(rows, K, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, K, generator=g)
    x[rows // 3] *= torch.exp2(torch.randint(-20, 20, (K,), generator=g).float())   # wide range inside blocks
    x[rows // 2, : K // 2] = 0.0                                                     # all-zero blocks
    x[rows // 2 + 1] *= 2.0 ** -130                                                  # flushed inputs
    x = x.to(torch.bfloat16)
    x[1, 5] = float("inf")
    x[2, 40] = float("-inf")
    x[3, 70] = float("nan")
    return x


def expected_operand(x: torch.Tensor, E: int, M: int):
    """What the prepared operand must hold, from the checker's components."""
    rows, K = x.shape
    sc, el = oracle.extract_mxfp(x, 32, E, M)
    sc = sc.numpy().reshape(rows, K // 32).astype(np.int64)
    el = el.numpy().reshape(rows, K // 32, 32)
    if (E, M) == (4, 3):
        top = ((el & 0x7F) == 0x7F).any(axis=2) & (sc < 254)
        codes = np.where(top[..., None], halved(el), el)
        scales = sc + top
    else:
        codes, scales = None, sc
    return sc, el, codes, scales


@pytest.mark.parametrize("tag", SCALED_TAGS)
def test_operand_from_dense_holds_the_reference_values(mh, tag):
    E, M = PRESETS[tag]
    rows, K = 300, 1024
    x = mixed_inputs(rows, K, seed=E * 10 + M)
    op = mh.mxk.scaled_operand_from_dense(x.to(DEV), getattr(mh.meta, tag))
    assert op.codes.shape == (512, K) and op.scales.shape == (K // 128, 512)
    codes, scales = operand_arrays(op)
    codes = codes.reshape(rows, K // 32, 32)
    ref_sc, ref_el, want_codes, want_scales = expected_operand(x, E, M)
    assert np.array_equal(scales, want_scales), "scale bytes"
    finite = ref_sc != 255
    got = decode_e4m3(codes) * 2.0 ** (scales[..., None].astype(np.float64) - 127)
    ref = decode_fmt(ref_el, E, M) * 2.0 ** (ref_sc[..., None].astype(np.float64) - 127)
    if (E, M) == (4, 3):
        assert np.array_equal(codes[finite], want_codes[finite]), "codes"
        assert not ((codes[finite] & 0x7F) == 0x7F).any(), "the NaN code must not appear"
        moved = np.abs(got - ref)[finite]
        assert (moved <= 2.0 ** -14 * np.abs(ref).max(axis=2, keepdims=True)[finite]).all()
        untouched = finite & (want_scales == ref_sc)
        assert np.array_equal(got[untouched], ref[untouched])
        assert (want_scales != ref_sc).sum() > 100, "the test data must hold blocks with the top code"
    else:
        assert np.array_equal(got[finite], ref[finite]), "embedded values"


@pytest.mark.parametrize("rows,K", [(260, 768), (300, 1536), (33, 640)])   # scale rows of 24 / 48 / 20 bytes: dword and 128-bit scale loads, ragged ends
@pytest.mark.parametrize("tag", SCALED_TAGS)
def test_operand_from_components_equals_from_dense(mh, tag, rows, K):
    E, M = PRESETS[tag]
    x = mixed_inputs(rows, K, seed=3)
    sc, el = oracle.extract_mxfp(x, 32, E, M)
    a = mh.mxk.scaled_operand_from_dense(x.to(DEV), getattr(mh.meta, tag))
    b = mh.mxk.scaled_operand_from_mxfp(sc.to(DEV), el.to(DEV), getattr(mh.meta, tag), rows, K)
    ca, sa = operand_arrays(a)
    cb, sb = operand_arrays(b)
    assert np.array_equal(sa, sb)
    assert np.array_equal(ca, cb)


def swiglu_inputs(rows, K, seed):
    g = torch.Generator().manual_seed(seed)
    t = (2.0 * torch.randn(rows, 2 * K, generator=g)).to(torch.bfloat16)
    t[0, :8] = torch.tensor([0.0, -0.0, 30.0, -30.0, 100.0, -100.0, 1e-30, -1e-30]).to(torch.bfloat16)
    t[1, 3] = float("inf")
    t[2, 4] = float("-inf")
    t[3, 5] = float("nan")
    t[4, K + 6] = float("inf")
    t[5, : 64] = 0.0
    return t


def test_swiglu_arithmetic_on_every_gate_value():
    """The operand kernel's silu(gate) * up (csrc/swiglu.h: hardware exp2 and reciprocal instead of the library's exp and
    division), run on its own through the test helper library.  The gate is bfloat16 and the SiLU is rounded to bfloat16
    before the product, so its 65536 inputs are all the cases there are: with up = 1 the output is that rounded SiLU, and
    it must be torch's, bit for bit, for every input (NaN for NaN).  Then 2^20 random pairs against torch's expression."""
    import ctypes

    path = os.path.join(ROOT, "mase-triton_amd", "mase_hip", "lib", "libmase_bench.so")
    assert os.path.exists(path), "libmase_bench.so is not built (python mase-triton_amd/build.py)"
    lib = ctypes.CDLL(path)
    lib.mase_bench_swiglu_bf16.restype = ctypes.c_int
    lib.mase_bench_swiglu_bf16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]

    def run(gate, up):
        out = torch.empty_like(gate)
        assert lib.mase_bench_swiglu_bf16(gate.data_ptr(), up.data_ptr(), out.data_ptr(), gate.numel(), torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        return out

    gate = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).to(DEV)
    got = run(gate, torch.ones_like(gate))
    want = torch.nn.functional.silu(gate)
    nan = want.isnan()
    assert torch.equal(got.isnan(), nan)
    assert torch.equal(got[~nan].view(torch.int16), want[~nan].view(torch.int16))
    g = torch.Generator().manual_seed(21)
    gate = (3.0 * torch.randn(1 << 20, generator=g)).to(torch.bfloat16).to(DEV)
    up = (torch.randn(1 << 20, generator=g) * torch.exp2(torch.randint(-8, 8, (1 << 20,), generator=g).float())).to(torch.bfloat16).to(DEV)
    assert torch.equal(run(gate, up).view(torch.int16), (torch.nn.functional.silu(gate) * up).view(torch.int16))


@pytest.mark.parametrize("tag", ["MXFP8_E4M3_fn", "OCP_MXFP4_E2M1"])
def test_operand_from_swiglu_equals_the_two_tensor_operations(mh, tag):
    """silu(gate) * up formed inside the operand kernel against the same expression as two tensor operations on the GPU
    (each rounding to bfloat16) followed by the dense operand kernel.  The kernel rounds at the same two places and its SiLU
    rounds to torch's bfloat16 value for every gate (the test above), so the operands must be equal."""
    rows, K = 300, 1024
    t = swiglu_inputs(rows, K, seed=11).to(DEV)
    gate, up = t[:, :K], t[:, K:]                      # views with row stride 2 K
    meta = getattr(mh.meta, tag)
    got = mh.mxk.scaled_operand_from_swiglu(gate, up, meta)
    h = torch.nn.functional.silu(gate) * up
    want = mh.mxk.scaled_operand_from_dense(h.contiguous(), meta)
    cg, sg = operand_arrays(got)
    cw, sw = operand_arrays(want)
    assert np.array_equal(sg, sw), "scale bytes"
    finite = np.repeat(sg != 255, 32, axis=1)     # (which element of an inf / NaN block carries the NaN code is the same too)
    assert np.array_equal(cg, cw), f"{(cg != cw).sum()} codes differ, {(cg != cw)[finite].sum()} of them in finite blocks"
    # separate tensors with their own (equal) row stride take the same kernel
    again = mh.mxk.scaled_operand_from_swiglu(gate.contiguous(), up.contiguous(), meta)
    ca, sa = operand_arrays(again)
    assert np.array_equal(ca, cg) and np.array_equal(sa, sg)


# ---------------------------------------------------------------- the product
def quantised(t: torch.Tensor, tag: str):
    E, M = PRESETS[tag]
    sc, el = oracle.extract_mxfp(t, 32, E, M)
    dq = oracle.compose_mxfp(sc, el, 32, E, M, True, torch.float32).view(t.shape)
    return sc, el, dq


@pytest.mark.parametrize("MNK", [(256, 256, 512), (300, 520, 768), (1024, 768, 1024), (1, 8, 512), (513, 264, 2048)])
@pytest.mark.parametrize("x_tag,w_tag", [("MXFP8_E4M3_fn", "MXFP8_E4M3_fn"), ("MXFP8_E4M3_fn", "OCP_MXFP6_E3M2"),
                                         ("OCP_MXFP6_E2M3", "OCP_MXFP4_E2M1"), ("OCP_MXFP4_E2M1", "OCP_MXFP6_E2M3")])
def test_scaled_gemm_vs_checker(mh, MNK, x_tag, w_tag):
    M, N, K = MNK
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    _, _, x_dq = quantised(x, x_tag)
    w_sc, w_el, w_dq = quantised(w, w_tag)
    y_ref = oracle.matmul_nt(x_dq, w_dq)
    a = mh.mxk.scaled_operand_from_dense(x.to(DEV), getattr(mh.meta, x_tag))
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), getattr(mh.meta, w_tag), N, K)
    y32 = mh.mxk.mxfp_gemm_scaled(a, wop, None, torch.float32)
    assert y32.shape == (M, N)
    assert rel_fro(y32, y_ref) <= F32_TOL
    y16 = mh.mxk.mxfp_gemm_scaled(a, wop, None, torch.bfloat16)
    assert rel_fro(y16, y_ref.to(torch.bfloat16)) <= 1e-3


@pytest.mark.parametrize("MNK", [(4200, 4808, 512), (2100, 9000, 768), (9000, 520, 512), (257, 65544, 512)])
def test_scaled_gemm_many_tiles(mh, MNK):
    """More 256 x 256 tiles than the GPU has compute units, in grids that the workgroups' walk order (patches of 4 x 8
    tiles per group of 32 workgroups) does not divide: every workgroup walks several tiles as one stream and the last
    patches are partial.  Every output element against the checker's product."""
    M, N, K = MNK
    g = torch.Generator().manual_seed(M ^ N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    _, _, x_dq = quantised(x, "MXFP8_E4M3_fn")
    w_sc, w_el, w_dq = quantised(w, "MXFP8_E4M3_fn")
    y_ref = x_dq.double() @ w_dq.double().t()      # the checker's dequantised operands, float64 product
    meta = mh.meta.MXFP8_E4M3_fn
    a = mh.mxk.scaled_operand_from_dense(x.to(DEV), meta)
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), meta, N, K)
    y = mh.mxk.mxfp_gemm_scaled(a, wop, None, torch.float32).cpu()
    assert rel_fro(y, y_ref) <= F32_TOL
    # no element may be far off on its own (a misplaced tile of a large output hides in a Frobenius norm)
    err = (y.double() - y_ref.double()).abs().view(-1)
    assert float(err.max()) <= 1e-3 * float(y_ref.double().abs().max())


@pytest.mark.parametrize("MNK", [(1, 4096, 4096), (7, 520, 1024), (16, 14336, 512), (17, 264, 2304), (32, 1032, 14336), (3, 8, 512),
                                 (17, 4104, 4096), (32, 14336, 4096), (33, 520, 768), (48, 4096, 3840), (49, 8, 512), (64, 4120, 4096),
                                 (24, 40, 4352), (64, 6160, 2048), (64, 4096, 14336), (40, 264, 8192), (17, 8, 4608)])
@pytest.mark.parametrize("x_tag,w_tag", [("MXFP8_E4M3_fn", "MXFP8_E4M3_fn"), ("MXFP8_E4M3_fn", "OCP_MXFP4_E2M1")])
def test_scaled_gemm_few_rows(mh, MNK, x_tag, w_tag):
    """Up to 64 rows of x: the weight-streaming kernels (a workgroup per 16 rows of W, its wavefronts taking the macro steps
    of K in turn and adding their partial sums through LDS; x in the wavefronts' registers, a K beyond 4096 cut into slices
    whose sums a second kernel adds (from 17 rows; the Python wrapper brings the room for them) or x streamed beside W (up to 16
    rows, and whenever there is no such room); the last row groups dealt in halves.  Row counts on both sides of the 16-row operand tiles, N that is not a
    multiple of 16, more and fewer row groups of W than the chip has CUs, K with fewer macro steps than a workgroup has
    wavefronts and with a count they do not divide; bias and every output type."""
    M, N, K = MNK
    g = torch.Generator().manual_seed(M * 7 + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    _, _, x_dq = quantised(x, x_tag)
    w_sc, w_el, w_dq = quantised(w, w_tag)
    y_ref = x_dq.double() @ w_dq.double().t()
    a = mh.mxk.scaled_operand_from_dense(x.to(DEV), getattr(mh.meta, x_tag))
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), getattr(mh.meta, w_tag), N, K)
    y32 = mh.mxk.mxfp_gemm_scaled(a, wop, None, torch.float32)
    assert y32.shape == (M, N)
    assert rel_fro(y32, y_ref) <= F32_TOL
    # without room for partial sums (the C entry point without a workspace): the kernels that need none
    assert rel_fro(mh.mxk.mxfp_gemm_scaled(a, wop, None, torch.float32, split_k=False), y_ref) <= F32_TOL
    err = (y32.cpu().double() - y_ref).abs().max()
    assert float(err) <= 1e-3 * float(y_ref.abs().max())
    y_b = y_ref + b.double()
    for odt in (torch.bfloat16, torch.float16):
        y16 = mh.mxk.mxfp_gemm_scaled(a, wop, b.to(DEV), odt)
        assert y16.dtype == odt and rel_fro(y16, y_b.to(odt)) <= 1e-3


def test_scaled_gemm_random_shapes(mh):
    """A seeded sweep over shapes on every route of the entry point (decode-sized kernel, lone tiles, K split, several
    tiles per workgroup): M 1 .. 700, N a multiple of 8 up to 1040, K a multiple of 256 up to 3072, format pairs in turn;
    every element of the fp32 result against a float64 product of the checker's dequantised operands."""
    import random

    rng = random.Random(1234)
    pairs = [("MXFP8_E4M3_fn", "MXFP8_E4M3_fn"), ("MXFP8_E4M3_fn", "OCP_MXFP6_E3M2"), ("OCP_MXFP6_E2M3", "OCP_MXFP4_E2M1")]
    for case in range(32):
        M = rng.choice([rng.randint(1, 32), rng.randint(17, 64), rng.randint(65, 300), rng.randint(301, 700)])
        N = 8 * rng.randint(1, 130)
        K = 256 * rng.randint(2, 12)
        x_tag, w_tag = pairs[case % len(pairs)]
        g = torch.Generator().manual_seed(case)
        x = (torch.randn(M, K, generator=g) * torch.exp2(torch.randint(-6, 6, (M, 1), generator=g).float())).to(torch.bfloat16)
        w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
        b = torch.randn(N, generator=g)
        _, _, x_dq = quantised(x, x_tag)
        w_sc, w_el, w_dq = quantised(w, w_tag)
        y_ref = x_dq.double() @ w_dq.double().t() + b.double()
        a = mh.mxk.scaled_operand_from_dense(x.to(DEV), getattr(mh.meta, x_tag))
        wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), getattr(mh.meta, w_tag), N, K)
        y = mh.mxk.mxfp_gemm_scaled(a, wop, b.to(DEV), torch.float32).cpu().double()
        assert y.shape == (M, N), (M, N, K)
        assert rel_fro(y, y_ref) <= F32_TOL, (M, N, K)
        assert float((y - y_ref).abs().max()) <= 1e-3 * float(y_ref.abs().max()), (M, N, K)


def test_scaled_gemm_bias_and_dtypes(mh):
    M, N, K = 300, 264, 512
    g = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    _, _, x_dq = quantised(x, "MXFP8_E4M3_fn")
    w_sc, w_el, w_dq = quantised(w, "MXFP8_E4M3_fn")
    meta = mh.meta.MXFP8_E4M3_fn
    a = mh.mxk.scaled_operand_from_dense(x.to(DEV), meta)
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), meta, N, K)
    for bdt in (torch.float32, torch.bfloat16, torch.float16):
        b = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(bdt)
        y_ref = oracle.matmul_nt(x_dq, w_dq) + b.float()
        for odt, tol in ((torch.float32, F32_TOL), (torch.bfloat16, 1e-3), (torch.float16, 1e-3)):
            y = mh.mxk.mxfp_gemm_scaled(a, wop, b.to(DEV), odt)
            assert y.dtype == odt
            assert rel_fro(y, y_ref.to(odt)) <= tol


@pytest.mark.parametrize("w_tag", SCALED_TAGS)
def test_identity_times_w_is_w(mh, w_tag):
    """x = identity: every output is one product, so the result must be W's dequantised values (rounded to bf16 the way
    the reference's compose rounds them); for E4M3 that includes the blocks that were re-encoded, except where a block
    holds both the top code and an odd code below 16.  Compared as values: a sign-only code composes to -0.0, and a
    product -0.0 added to the row's other products (+0.0) is +0.0 in any matmul."""
    E, M = PRESETS[w_tag]
    K = N = 512
    g = torch.Generator().manual_seed(9)
    w = (torch.randn(N, K, generator=g) * torch.exp2(torch.randint(-12, 12, (N, 1), generator=g).float())).to(torch.bfloat16)
    w_sc, w_el = oracle.extract_mxfp(w, 32, E, M)
    want = oracle.compose_mxfp(w_sc, w_el, 32, E, M, True, torch.bfloat16).view(N, K)
    x = torch.eye(K, dtype=torch.bfloat16)
    a = mh.mxk.scaled_operand_from_dense(x.to(DEV), mh.meta.MXFP8_E4M3_fn)
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), getattr(mh.meta, w_tag), N, K)
    y = mh.mxk.mxfp_gemm_scaled(a, wop, None, torch.bfloat16).cpu()   # y[k, n] = W[n, k]
    got = y.t().contiguous()
    if (E, M) == (4, 3):
        el = w_el.numpy().reshape(N, K // 32, 32)
        top = ((el & 0x7F) == 0x7F).any(axis=2)
        odd_small = (((el & 0x7F) < 16) & ((el & 1) == 1)).any(axis=2)
        inexact = torch.from_numpy(np.repeat(top & odd_small, 32, axis=1))
        assert top.sum() > 50
        assert torch.equal(got[~inexact].float(), want[~inexact].float())
        assert rel_fro(got, want) <= 1e-5
    else:
        assert torch.equal(got.float(), want.float())


def test_special_blocks_poison_the_same_outputs(mh):
    """inf / NaN in x or W: scale byte 255.  Dequantise-then-matmul turns the affected rows / columns into NaN (a zero
    code times 2^128 is NaN); so must the matrix unit."""
    M, N, K = 256, 256, 512
    g = torch.Generator().manual_seed(2)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    x[7, 100] = float("inf")
    x[200, 3] = float("nan")
    w[5, 40] = float("-inf")
    w[255, 511] = float("nan")
    _, _, x_dq = quantised(x, "MXFP8_E4M3_fn")
    w_sc, w_el, w_dq = quantised(w, "MXFP8_E4M3_fn")
    y_ref = x_dq.double() @ w_dq.double().t()
    meta = mh.meta.MXFP8_E4M3_fn
    a = mh.mxk.scaled_operand_from_dense(x.to(DEV), meta)
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), meta, N, K)
    y = mh.mxk.mxfp_gemm_scaled(a, wop, None, torch.float32).cpu()
    assert torch.equal(y.isnan(), y_ref.isnan())
    assert y.isnan().sum() == 2 * N + 2 * M - 4
    ok = ~y_ref.isnan()
    assert rel_fro(y[ok], y_ref[ok]) <= F32_TOL


@pytest.mark.parametrize("MNK", [(256, 256, 4096), (300, 520, 2048), (1024, 512, 14336), (700, 264, 7168)])
def test_scaled_gemm_k_split(mh, MNK):
    """Few tiles and a long K: the launcher splits K over several workgroups per tile (fp32 partial sums in a workspace,
    a second kernel adds them).  Against the checker and against the unsplit call (which it may equal bit for bit: products
    of two MXFP values have at most eight significant bits, and sums of a few thousand of them are often exact in fp32
    whatever the order)."""
    from mase_hip import _lib

    M, N, K = MNK
    need = _lib.load().mase_hip_mxfp_gemm_scaled_workspace_bytes(M, N, K)
    if need == 0:
        pytest.skip("this shape is not split on this device")
    assert need % (M * N * 4) == 0 and 2 <= need // (M * N * 4) <= 16
    g = torch.Generator().manual_seed(K + M)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    _, _, x_dq = quantised(x, "MXFP8_E4M3_fn")
    w_sc, w_el, w_dq = quantised(w, "OCP_MXFP6_E3M2")
    y_ref = oracle.matmul_nt(x_dq, w_dq) + b.float()
    a = mh.mxk.scaled_operand_from_dense(x.to(DEV), mh.meta.MXFP8_E4M3_fn)
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), mh.meta.OCP_MXFP6_E3M2, N, K)
    for odt, tol in ((torch.float32, F32_TOL), (torch.bfloat16, 1e-3)):
        y = mh.mxk.mxfp_gemm_scaled(a, wop, b.to(DEV), odt)
        y_one = mh.mxk.mxfp_gemm_scaled(a, wop, b.to(DEV), odt, split_k=False)
        assert rel_fro(y, y_ref.to(odt)) <= tol
        assert rel_fro(y, y_one) <= tol


# ---------------------------------------------------------------- the prepared weight on the bf16 kernel
@pytest.mark.parametrize("MNK", [(512, 256, 512), (1100, 384, 1024), (640, 128, 128)])
@pytest.mark.parametrize("w_tag", SCALED_TAGS)
def test_prepared_weight_on_the_bf16_kernel(mh, MNK, w_tag):
    """Dense bf16 A against the weight in prepared form (mase_hip_mxfp_gemm_prepared_w): against the float64 checker, and
    against mase_hip_mxfp_gemm on the components (which may pick another tile shape, i.e. another order of additions)."""
    M, N, K = MNK
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    _, _, x_dq = quantised(x, "MXFP8_E4M3_fn")
    w_sc, w_el, w_dq = quantised(w, w_tag)
    meta = getattr(mh.meta, w_tag)
    a = x_dq.to(torch.bfloat16).to(DEV)
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), meta, N, K)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    y_ref = oracle.matmul_nt(x_dq, w_dq) + b.float()
    for odt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-3)):
        y = mh.mxk.mxfp_gemm_prepared_w(a, wop, b.to(DEV), odt)
        assert y.shape == (M, N) and y.dtype == odt
        assert rel_fro(y, y_ref.to(odt)) <= tol
        y_comp = mh.mxk.mxfp_gemm(a, None, None, None, w_sc.to(DEV), w_el.to(DEV), meta, b.to(DEV), M, N, K, odt, split_k=False)
        assert rel_fro(y, y_comp) <= 2 * tol


def test_prepared_weight_special_blocks_and_refusals(mh):
    M, N, K = 512, 128, 256
    g = torch.Generator().manual_seed(8)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    w[5, 40] = float("inf")
    w[77, 255] = float("nan")
    w_sc, w_el, w_dq = quantised(w, "OCP_MXFP6_E3M2")
    meta = mh.meta.OCP_MXFP6_E3M2
    wop = mh.mxk.scaled_operand_from_mxfp(w_sc.to(DEV), w_el.to(DEV), meta, N, K)
    y = mh.mxk.mxfp_gemm_prepared_w(x.to(DEV), wop, None, torch.float32).cpu()
    y_ref = x.double() @ w_dq.double().t()
    assert torch.equal(y.isnan(), y_ref.isnan()) and y.isnan().sum() == 2 * M
    with pytest.raises(NotImplementedError):
        mh.mxk.mxfp_gemm_prepared_w(x[:256].to(DEV), wop, None, torch.float32)   # fewer than 512 rows


def test_weight_only_layer_keeps_the_prepared_weight(mh):
    """XWqB (dense bfloat16 activations): from 512 rows on the layer runs the bf16 kernel on its kept prepared weight."""
    lin = torch.nn.Linear(512, 256, bias=True, dtype=torch.bfloat16, device=DEV)
    wfmt = mh.meta.OCP_MXFP4_E2M1
    fused = mh.MXFPLinearPTQ.from_linear(lin, None, wfmt, None, "XWqB", "fused")
    sep = mh.MXFPLinearPTQ.from_linear(lin, None, wfmt, None, "XWqB", "separate")
    g = torch.Generator().manual_seed(3)
    small = torch.randn(64, 512, generator=g).to(torch.bfloat16).to(DEV)
    big = torch.randn(2, 300, 512, generator=g).to(torch.bfloat16).to(DEV)
    assert rel_fro(fused(small), sep(small)) <= 1e-3 and fused._scaled_w is None
    y = fused(big)
    assert fused._scaled_w is not None and y.shape == (2, 300, 256)
    assert rel_fro(y, sep(big)) <= 1e-3


def test_unsupported_shapes_are_refused(mh):
    meta = mh.meta.MXFP8_E4M3_fn
    x = torch.randn(64, 384).to(torch.bfloat16).to(DEV)
    a = mh.mxk.scaled_operand_from_dense(x, meta)   # K % 128 == 0: an operand can be built
    with pytest.raises(NotImplementedError):
        mh.mxk.mxfp_gemm_scaled(a, a, None, torch.bfloat16)   # K % 256 != 0
    with pytest.raises(NotImplementedError):
        mh.mxk.scaled_operand_from_dense(torch.randn(8, 96).to(torch.bfloat16).to(DEV), meta)
    x5 = torch.randn(8, 512).to(torch.bfloat16).to(DEV)
    with pytest.raises((NotImplementedError, AssertionError)):
        mh.mxk.scaled_operand_from_dense(x5, mh.meta.MXFP8_E5M2_fn)
