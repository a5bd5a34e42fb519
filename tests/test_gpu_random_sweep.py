"""Seeded random sweep of the cast kernels and the GEMM against the CPU checker: formats (any exponent / fraction
width, finite-only or not, four rounding modes), block sizes, element counts, dtypes in and out, value distributions
(wide dynamic range, raw random bit patterns, sparse, extreme scales, planted inf / NaN), layouts with the block
axis in the middle, and GEMM shapes across every kernel of the dispatch.  Bit-exact for the casts; the GEMM within the
stated tolerance (relative Frobenius error 1e-3 for 16-bit outputs, 1e-5 for fp32) of fp32 dequantize-then-matmul."""
import random

import pytest
import torch

import oracle
from helpers import assert_bits_equal, assert_int_equal

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
PRESETS = [(4, 3), (5, 2), (2, 3), (3, 2), (2, 1)]


def rand_tensor(rng, g, n, dt):
    kind = rng.randrange(5)
    if kind == 0:
        x = torch.randn(n, generator=g) * 10 ** rng.uniform(-6, 6)
    elif kind == 1:
        x = torch.randn(n, generator=g) * torch.exp2(torch.randint(-40, 40, (n,), generator=g).float())
    elif kind == 2:
        x = torch.randint(-2 ** 31, 2 ** 31 - 1, (n,), generator=g, dtype=torch.int64).to(torch.int32).view(torch.float32)
    elif kind == 3:
        x = torch.randn(n, generator=g)
        x[torch.rand(n, generator=g) < 0.3] = 0.0
    else:
        x = torch.randn(n, generator=g) * 2.0 ** rng.randrange(-130, 128)
    if rng.random() < 0.2 and n > 4:
        for v in (float("inf"), float("-inf"), float("nan")):
            x[rng.randrange(n)] = v
    return x.to(DT[dt])


@pytest.mark.parametrize("seed", [1, 2])
def test_random_casts_vs_checker(seed):
    import mase_hip.minifloat.kernels as mfk
    import mase_hip.mxfp.kernels as mxk
    from mase_hip.minifloat.meta import MinifloatMeta
    from mase_hip.mxfp.meta import MXFPMeta

    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    for _ in range(120):
        dt = rng.choice(list(DT))
        # minifloat, any format
        E = rng.randrange(1, 9)
        M = rng.randrange(1, 16 - E if E < 8 else 8)
        fin, rm = rng.random() < 0.7, rng.choice(["rn", "ru", "rd", "rz"])
        n = rng.choice([1, 7, 8, 100, 4097, 65536 + rng.randrange(100)])
        x = rand_tensor(rng, g, n, dt)
        meta = MinifloatMeta(E, M, fin, rm)
        what = f"{dt} E{E}M{M} finite={fin} {rm} n={n}"
        codes = mfk.extract_minifloat_component(x.to(DEV), meta)
        codes_w = oracle.extract_minifloat(x, E, M, fin, rm)
        assert_int_equal(codes, codes_w, "minifloat extract " + what)
        for odt in DT:
            w = oracle.compose_minifloat(codes_w, E, M, fin, DT[odt])
            assert_bits_equal(mfk.compose_minifloat_component(codes, meta, DT[odt]), w, odt, f"minifloat compose ->{odt} " + what)
            assert_bits_equal(mfk.quantize_dequantize(x.to(DEV), meta, DT[odt]), w, odt, f"minifloat qdq ->{odt} " + what)
        # MXFP, flat
        e, m = rng.choice(PRESETS)
        B = rng.choice([32, 32, 32, 16, 64, 8, 5, 128])
        nb = rng.choice([1, 3, 64, 1000, 4099])
        rm = rng.choice(["rn", "rn", "ru", "rd", "rz"])
        x = rand_tensor(rng, g, B * nb, dt)
        meta = MXFPMeta(B, 8, e, m, True, rm)
        what = f"{dt} e{e}m{m} B={B} {rm} blocks={nb}"
        sc_w, el_w = oracle.extract_mxfp(x, B, e, m, True, rm)
        sc, el = mxk.extract_mxfp_components(x.to(DEV), meta)
        assert_int_equal(sc, sc_w, "mxfp scales " + what)
        assert_int_equal(el, el_w, "mxfp elements " + what)
        for odt in DT:
            w = oracle.compose_mxfp(sc_w, el_w, B, e, m, True, DT[odt])
            assert_bits_equal(mxk.compose_mxfp_tensor(sc, el, meta, DT[odt]), w, odt, f"mxfp compose ->{odt} " + what)
            assert_bits_equal(mxk.quantize_dequantize(x.to(DEV), meta, DT[odt]), w, odt, f"mxfp qdq ->{odt} " + what)
        # MXFP, block axis in the middle, read in place
        K = 32 * rng.choice([1, 2, 4, 5, 8])
        inner, outer = rng.choice([1, 2, 6, 64, 128, 130, 256]), rng.choice([1, 2, 3])
        x = rand_tensor(rng, g, outer * K * inner, dt).view(outer, K, inner)
        meta = MXFPMeta(32, 8, e, m, True, rm)
        what = f"{dt} e{e}m{m} {rm} shape={tuple(x.shape)}"
        sc_w, el_w = oracle.extract_mxfp(x.permute(0, 2, 1).contiguous().flatten(), 32, e, m, True, rm)
        sc, el = mxk.extract_mxfp_components_strided(x.to(DEV), 1, meta)
        assert_int_equal(sc, sc_w, "in-place scales " + what)
        assert_int_equal(el, el_w, "in-place elements " + what)
        w = oracle.compose_mxfp(sc_w, el_w, 32, e, m, True, DT[dt]).view(outer, inner, K).permute(0, 2, 1).contiguous()
        assert_bits_equal(mxk.quantize_dequantize_strided(x.to(DEV), 1, meta, DT[dt]), w, dt, "in-place qdq " + what)


def test_random_gemm_shapes_vs_dequantize_then_matmul():
    import mase_hip.mxfp.kernels as mxk
    from mase_hip.mxfp.meta import MXFPMeta

    rng = random.Random(3)
    g = torch.Generator().manual_seed(3)
    for _ in range(100):
        M = rng.choice([1, 5, 16, 31, 64, 100, 128, 129, 200, 256, 257, 300, 384, 500, 512, 513, 700, 1024, 1500])
        N = rng.choice([32, 64, 96, 128, 256, 384, 640, 1024, 2048, 12288])
        K = rng.choice([32, 64, 96, 128, 192, 256, 384, 512, 1024, 1536, 2048, 4224])  # the longer ones get K split over workgroups
        e, m = rng.choice(PRESETS)
        odt = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
        x_dq = oracle.qdq_mxfp(x.flatten(), 32, 4, 3).view(M, K).to(DEV)
        sc_w, el_w = oracle.extract_mxfp(w, 32, e, m)
        w_dq = oracle.compose_mxfp(sc_w, el_w, 32, e, m, True, torch.bfloat16).view(N, K).to(DEV)
        b = torch.randn(N, generator=g).to(rng.choice([torch.bfloat16, torch.float32])).to(DEV) if rng.random() < 0.5 else None
        y = mxk.mxfp_gemm(x_dq, None, None, None, sc_w.to(DEV), el_w.to(DEV), MXFPMeta(32, 8, e, m, True, "rn"), b, M, N, K, odt)
        ref = x_dq.float() @ w_dq.float().T
        if b is not None:
            ref = ref + b.float()
        ref = ref.to(odt).double().cpu()
        err = ((y.double().cpu() - ref).norm() / ref.norm()).item()
        assert err <= (1e-5 if odt == torch.float32 else 1e-3), (M, N, K, e, m, odt, b is not None, err)
