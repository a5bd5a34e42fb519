"""GPU parity tests for the cast kernels, called through the package (ctypes -> C ABI -> HIP).

Bit-exact against (1) the vectors written by the reference's own "fake" path, (2) the CPU
checker on seeded inputs, at sizes up to the full benchmark configurations, and (3) size-free
properties.  NaN outputs compare equal to any NaN (payload/sign is unstable in torch itself).
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import PRESETS, assert_bits_equal, assert_int_equal, bits_of, codes_tensor, from_bits, golden, parse_cfg_key

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def mh():
    import mase_hip.minifloat.kernels as mfk
    import mase_hip.mxfp.kernels as mxk
    from mase_hip import _lib
    from mase_hip.minifloat.meta import MinifloatMeta
    from mase_hip.mxfp.meta import MXFPMeta

    _lib.load()

    class NS:
        pass

    ns = NS()
    ns.mfk, ns.mxk, ns.MinifloatMeta, ns.MXFPMeta = mfk, mxk, MinifloatMeta, MXFPMeta
    return ns


def mx_meta(mh, e, m, block=32, rnd="rn"):
    return mh.MXFPMeta(block_size=block, scale_exp_bits=8, element_exp_bits=e, element_frac_bits=m,
                       element_is_finite=True, round_mode=rnd)


# ----------------------------------------------------------------------------- golden vectors
def test_minifloat_extract_f32_vectors(mh):
    d = golden("minifloat_extract_f32.npz")
    x = from_bits(d["x_f32_bits"], "float32").to(DEV)
    for k in [k for k in d.files if k.startswith("codes_")]:
        e, m, fin, rnd = parse_cfg_key(k[len("codes_"):])
        meta = mh.MinifloatMeta(e, m, fin, rnd)
        assert_int_equal(mh.mfk.extract_minifloat_component(x, meta), d[k], k)


@pytest.mark.parametrize("dt", ["bfloat16", "float16"])
def test_minifloat_extract_every_16bit_pattern(mh, dt):
    d = golden("minifloat_extract_all16.npz")
    x = from_bits(np.arange(1 << 16, dtype=np.uint32).astype(np.uint16), dt).to(DEV)
    for k in [k for k in d.files if k.startswith(dt + "_")]:
        e, m, fin, rnd = parse_cfg_key(k[len(dt) + 1:])
        assert_int_equal(mh.mfk.extract_minifloat_component(x, mh.MinifloatMeta(e, m, fin, rnd)), d[k], k)


def test_minifloat_compose_whole_code_space(mh):
    d = golden("minifloat_compose.npz")
    for k in [k for k in d.files if k.startswith("codes_")]:
        em, fin = k[len("codes_"):].split("_")
        e, m = (int(v) for v in em[1:].split("m"))
        codes = codes_tensor(d[k]).to(DEV)
        meta = mh.MinifloatMeta(e, m, fin == "fin", "rn")
        for dt in ("float32", "bfloat16", "float16"):
            got = mh.mfk.compose_minifloat_component(codes, meta, getattr(torch, dt))
            assert_bits_equal(got, d[f"out_{dt}_{em}_{fin}"], dt, f"{k} {dt}")


@pytest.mark.parametrize("dt", ["bfloat16", "float16", "float32"])
def test_mxfp_block_vectors(mh, dt):
    d = golden(f"mxfp_blocks_{dt}.npz")
    x = from_bits(d["x_bits"], dt).to(DEV).flatten()
    for tag, (e, m) in PRESETS.items():
        meta = mx_meta(mh, e, m)
        sc, el = mh.mxk.extract_mxfp_components(x, meta)
        assert sc.shape == (x.numel() // 32, 1) and el.shape == (x.numel() // 32, 32)
        assert sc.dtype == torch.uint8 and el.dtype == torch.uint8
        assert_int_equal(sc, d["scales_" + tag], f"scales {dt} {tag}")
        assert_int_equal(el, d["elements_" + tag], f"elements {dt} {tag}")
        for odt in sorted({dt, "float32"}):
            want = d[f"dq_{odt}_{tag}"]
            assert_bits_equal(mh.mxk.compose_mxfp_tensor(sc, el, meta, getattr(torch, odt)), want, odt, f"dq {dt}->{odt} {tag}")
            assert_bits_equal(mh.mxk.quantize_dequantize(x, meta, getattr(torch, odt)), want, odt, f"qdq {dt}->{odt} {tag}")


def test_mxfp_other_block_sizes_and_round_modes(mh):
    d = golden("mxfp_blocks_misc.npz")
    for k in [k for k in d.files if k.startswith("scales_")]:
        _, dt, b, em, rnd = k.split("_")
        bs = int(b[1:])
        e, m = (int(v) for v in em[1:].split("m"))
        meta = mx_meta(mh, e, m, bs, rnd)
        x = from_bits(d[f"x_{dt}_b{bs}"], dt).to(DEV).flatten()
        sc, el = mh.mxk.extract_mxfp_components(x, meta)
        assert_int_equal(sc, d[k], f"scales {k}")
        assert_int_equal(el, d["elements_" + k[7:]], f"elements {k}")
        assert_bits_equal(mh.mxk.compose_mxfp_tensor(sc, el, meta, getattr(torch, dt)), d["dq_" + k[7:]], dt, f"dq {k}")
        assert_bits_equal(mh.mxk.quantize_dequantize(x, meta, getattr(torch, dt)), d["dq_" + k[7:]], dt, f"qdq {k}")


def test_mxfp_compose_every_scale_and_code(mh):
    d = golden("mxfp_compose_table.npz")
    sc = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(256, 1).to(DEV)
    el = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(1, 256).repeat(256, 1).to(DEV)
    for k in d.files:
        odt, tag = k.split("_", 1)
        e, m = PRESETS[tag]
        got = mh.mxk.compose_mxfp_tensor(sc, el, mx_meta(mh, e, m, 256), getattr(torch, odt))
        assert_bits_equal(got, d[k], odt, k)


def test_mxfp4_known_answers(mh):
    d = golden("mxfp4_known_answer.npz")
    meta = mx_meta(mh, 2, 1, 8)
    for dt in ("float32", "bfloat16", "float16"):
        x = from_bits(d[f"x_{dt}"], dt).to(DEV)
        sc, el = mh.mxk.extract_mxfp_components(x, meta)
        assert_int_equal(sc, d[f"scales_{dt}"], f"scales {dt}")
        assert_int_equal(el, d[f"elements_{dt}"], f"elements {dt}")
        y = mh.mxk.compose_mxfp_tensor(sc, el, meta, getattr(torch, dt))
        assert torch.equal(y, x)


# ----------------------------------------------------------------------------- seeded inputs vs the CPU checker
@pytest.mark.parametrize("dt", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 1000, 4099, 1 << 20])
def test_minifloat_random_vs_checker(mh, dt, n):
    g = torch.Generator().manual_seed(n + 11)
    x = (torch.randn(n, generator=g) * torch.exp2(torch.randint(-10, 10, (n,), generator=g).float())).to(getattr(torch, dt))
    xd = x.to(DEV)
    for (e, m, fin, rnd) in [(4, 3, True, "rn"), (5, 2, True, "rn"), (2, 1, True, "rn"), (3, 2, False, "ru"), (5, 10, True, "rz")]:
        meta = mh.MinifloatMeta(e, m, fin, rnd)
        want = oracle.extract_minifloat(x, e, m, fin, rnd)
        got = mh.mfk.extract_minifloat_component(xd, meta)
        assert got.shape == x.shape and got.dtype == torch.uint16
        assert_int_equal(got, want, f"codes {dt} n={n} e{e}m{m}")
        for odt in (torch.float32, torch.bfloat16, torch.float16):
            w = oracle.compose_minifloat(want, e, m, fin, odt)
            name = str(odt).removeprefix("torch.")
            assert_bits_equal(mh.mfk.compose_minifloat_component(got, meta, odt), w, name, f"dq {dt}->{name} n={n}")
            assert_bits_equal(mh.mfk.quantize_dequantize(xd, meta, odt), w, name, f"qdq {dt}->{name} n={n}")


@pytest.mark.parametrize("tag", list(PRESETS))
def test_mxfp_bf16_every_pattern_under_chosen_block_maxima(mh, tag):
    """Every bf16 bit pattern as an element of a block whose first element is a chosen value (exponent fields from the
    subnormal edge to the top, smallest and largest mantissa): elements above it become the block maximum themselves, the
    others land in every binade below it, inf / NaN patterns make special blocks.  Extract, compose and the fused pass
    against the checker, bit for bit: pins the packed 16-bit arithmetic of the bf16 kernels."""
    e, m = PRESETS[tag]
    pats = torch.arange(1 << 16, dtype=torch.int32)
    pats = torch.cat([pats, torch.zeros(31 * 2115 - (1 << 16), dtype=torch.int32)]).view(2115, 31)
    blocks = []
    for ef in (1, 2, 9, 60, 126, 127, 128, 140, 200, 253, 254):
        for mant in (0x00, 0x7F):
            first = torch.full((2115, 1), (ef << 7) | mant, dtype=torch.int32)
            blocks.append(torch.cat([first, pats], dim=1))
    bits = torch.cat(blocks).reshape(-1)
    x = bits.to(torch.int16).view(torch.bfloat16)
    xd = x.to(DEV)
    meta = mx_meta(mh, e, m)
    w_sc, w_el = oracle.extract_mxfp(x, 32, e, m)
    g_sc, g_el = mh.mxk.extract_mxfp_components(xd, meta)
    assert_int_equal(g_sc.flatten(), w_sc.flatten(), f"scales {tag}")
    assert_int_equal(g_el.flatten(), w_el.flatten(), f"elements {tag}")
    want = oracle.compose_mxfp(w_sc, w_el, 32, e, m, True, torch.bfloat16)
    assert_bits_equal(mh.mxk.compose_mxfp_tensor(g_sc, g_el, meta, torch.bfloat16), want, "bfloat16", f"compose {tag}")
    assert_bits_equal(mh.mxk.quantize_dequantize(xd, meta, torch.bfloat16), want, "bfloat16", f"qdq {tag}")


@pytest.mark.parametrize("tag", list(PRESETS))
def test_minifloat_every_fp32_class(mh, tag):
    """The code of an fp32 input depends on its sign, its exponent field and the top 15 bits of its mantissa only
    (the reference truncates the mantissa to 15 bits before it rounds): 2^24 classes.  One input of every class, the low
    8 mantissa bits filled from a hash of the class, through extract and the fused pass against the checker: pins the
    branch-free encode of the preset formats, ties, lost carries, the subnormal binade and saturation included."""
    e, m = PRESETS[tag]
    cls = torch.arange(1 << 24, dtype=torch.int64)
    low = (cls * 2654435761 >> 11) & 0xFF
    x = ((cls << 8) | low).to(torch.int32).view(torch.float32)   # classes with exponent field 255 are inf / NaN inputs
    xd = x.to(DEV)
    meta = mh.MinifloatMeta(e, m, True, "rn")
    want = oracle.extract_minifloat(x, e, m, True, "rn")
    assert_int_equal(mh.mfk.extract_minifloat_component(xd, meta), want, f"codes {tag}")
    assert_bits_equal(mh.mfk.quantize_dequantize(xd, meta, torch.float32), oracle.compose_minifloat(want, e, m, True, torch.float32),
                      "float32", f"qdq {tag}")


@pytest.mark.parametrize("dt", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("block,n_blocks", [(32, 1), (32, 5), (32, 1025), (32, 40000), (16, 77), (64, 33), (8, 3),
                                             (4, 10), (3, 7), (1, 5), (96, 9), (256, 17), (1024, 3)])
def test_mxfp_random_vs_checker(mh, dt, block, n_blocks):
    g = torch.Generator().manual_seed(block * 1000 + n_blocks)
    n = block * n_blocks
    x = torch.randn(n, generator=g) * torch.exp2(torch.randint(-30, 30, (n_blocks, 1), generator=g).float()).repeat(1, block).flatten()
    x[torch.rand(n, generator=g) < 0.01] = 0.0
    x = x.to(getattr(torch, dt))
    xd = x.to(DEV)
    for tag, (e, m) in PRESETS.items():
        meta = mx_meta(mh, e, m, block)
        sc_w, el_w = oracle.extract_mxfp(x, block, e, m)
        sc, el = mh.mxk.extract_mxfp_components(xd, meta)
        assert_int_equal(sc, sc_w, f"scales {dt} {tag} B={block}")
        assert_int_equal(el, el_w, f"elements {dt} {tag} B={block}")
        w = oracle.compose_mxfp(sc_w, el_w, block, e, m, True, x.dtype)
        assert_bits_equal(mh.mxk.compose_mxfp_tensor(sc, el, meta, x.dtype), w, dt, f"dq {dt} {tag} B={block}")
        assert_bits_equal(mh.mxk.quantize_dequantize(xd, meta, x.dtype), w, dt, f"qdq {dt} {tag} B={block}")


def test_unaligned_views(mh):
    """Slices that start at odd offsets (not 16-byte aligned) must still give the same bits."""
    g = torch.Generator().manual_seed(5)
    base = torch.randn(32 * 64 + 3, generator=g).to(torch.bfloat16)
    x = base[3:]
    xd = base.to(DEV)[3:]
    import warnings

    from mase_hip import _lib

    meta = mx_meta(mh, 4, 3)
    sc_w, el_w = oracle.extract_mxfp(x.clone(), 32, 4, 3)
    copies = _lib.realignment_copies
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)      # the first realignment copy of a process warns
        sc, el = mh.mxk.extract_mxfp_components(xd, meta)
        assert _lib.realignment_copies == copies + 1, "the copy that realigns the operand is counted"
        assert_int_equal(sc, sc_w, "scales")
        assert_int_equal(el, el_w, "elements")
        mm = mh.MinifloatMeta(4, 3, True, "rn")
        assert_int_equal(mh.mfk.extract_minifloat_component(xd, mm), oracle.extract_minifloat(x.clone(), 4, 3), "codes")
        assert _lib.realignment_copies == copies + 2


# ----------------------------------------------------------------------------- full-size configurations
def test_config_c1_full_size(mh):
    from workloads import make_c1

    x = make_c1()
    meta = mx_meta(mh, 4, 3)
    sc_w, el_w = oracle.extract_mxfp(x, 32, 4, 3)
    sc, el = mh.mxk.extract_mxfp_components(x.to(DEV).flatten(), meta)
    assert_int_equal(sc, sc_w, "c1 scales")
    assert_int_equal(el, el_w, "c1 elements")
    w = oracle.compose_mxfp(sc_w, el_w, 32, 4, 3, True, torch.bfloat16)
    assert_bits_equal(mh.mxk.compose_mxfp_tensor(sc, el, meta, torch.bfloat16), w, "bfloat16", "c1 dq")
    assert_bits_equal(mh.mxk.quantize_dequantize(x.to(DEV).flatten(), meta, torch.bfloat16), w, "bfloat16", "c1 qdq")


def test_config_c2_full_size(mh):
    from workloads import make_c2

    x = make_c2()
    xd = x.to(DEV)
    for e, m in ((4, 3), (5, 2)):
        meta = mh.MinifloatMeta(e, m, True, "rn")
        want = oracle.extract_minifloat(x, e, m)
        got = mh.mfk.extract_minifloat_component(xd, meta)
        assert_int_equal(got, want, f"c2 codes e{e}m{m}")
        w = oracle.compose_minifloat(want, e, m, True, torch.float32)
        assert_bits_equal(mh.mfk.compose_minifloat_component(got, meta, torch.float32), w, "float32", f"c2 dq e{e}m{m}")
        assert_bits_equal(mh.mfk.quantize_dequantize(xd, meta, torch.float32), w, "float32", f"c2 qdq e{e}m{m}")


def test_config_c3_full_size(mh):
    from workloads import make_c3

    x = make_c3()
    meta = mx_meta(mh, 2, 1)
    sc_w, el_w = oracle.extract_mxfp(x, 32, 2, 1)
    sc, el = mh.mxk.extract_mxfp_components(x.to(DEV).flatten(), meta)
    assert_int_equal(sc, sc_w, "c3 scales")
    assert_int_equal(el, el_w, "c3 elements")
    w = oracle.compose_mxfp(sc_w, el_w, 32, 2, 1, True, torch.bfloat16)
    assert_bits_equal(mh.mxk.compose_mxfp_tensor(sc, el, meta, torch.bfloat16), w, "bfloat16", "c3 dq")


# ----------------------------------------------------------------------------- size-free properties
@pytest.mark.parametrize("tag", list(PRESETS))
def test_power_of_two_and_sign_symmetry_full_size(mh, tag):
    """At the largest benchmark shape (14336 x 4096 bf16): multiplying the input by 2^k shifts every
    scale by k and leaves the element codes alone; negating it flips only the sign bit of the
    codes of non-zero quotients.  (Quantisation itself is NOT idempotent in this scheme: a lost
    mantissa carry can move a block maximum down a binade.)"""
    e, m = PRESETS[tag]
    meta = mx_meta(mh, e, m)
    sign = 1 << (e + m)
    g = torch.Generator(device=DEV).manual_seed(9)
    x = (torch.randn(14336 * 4096, generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    sc, el = mh.mxk.extract_mxfp_components(x, meta)
    sc2, el2 = mh.mxk.extract_mxfp_components(x * 2.0 ** 7, meta)
    assert torch.equal(sc2.int(), sc.int() + 7)
    assert torch.equal(el2, el)
    sc3, el3 = mh.mxk.extract_mxfp_components(-x, meta)
    assert torch.equal(sc3, sc)
    assert torch.equal(el3 & (sign - 1), el & (sign - 1))
    nonzero = (el & (sign - 1)) != 0
    assert torch.equal((el3 ^ el)[nonzero], torch.full_like(el, sign)[nonzero])
    # the round trip never increases a magnitude by more than one grid step of the top binade and
    # never loses more than half of it (the lost-carry case, 1.97 -> 1.0) plus one step
    y = mh.mxk.compose_mxfp_tensor(sc, el, meta, torch.float32).view(-1, 32)
    step = torch.exp2(sc.float() - 127 + ((1 << e) - 1 - ((1 << (e - 1)) - 1)) - m)
    xa, ya = x.float().view(-1, 32).abs(), y.abs()
    assert (ya <= xa + step).all()
    assert (ya >= xa / 2 - step).all()


def test_inplace_qdq(mh):
    from mase_hip import _lib

    x = torch.randn(1 << 16, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16).to(DEV)
    meta = mx_meta(mh, 4, 3)
    want = mh.mxk.quantize_dequantize(x, meta, torch.bfloat16)
    y = x.clone()
    _lib.check(_lib.load().mase_hip_qdq_mxfp(y.data_ptr(), 2, y.data_ptr(), 2, y.numel(), 32, 4, 3, 1, 0, _lib.stream_ptr(y.device)))
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))


def test_error_codes(mh):
    from mase_hip import _lib

    lib = _lib.load()
    x = torch.zeros(64, dtype=torch.bfloat16, device=DEV)
    sc = torch.zeros(2, dtype=torch.uint8, device=DEV)
    el = torch.zeros(64, dtype=torch.uint8, device=DEV)
    assert lib.mase_hip_extract_mxfp(x.data_ptr(), 2, sc.data_ptr(), el.data_ptr(), 63, 32, 4, 3, 1, 0, None) == -1
    assert b"multiple" in lib.mase_hip_last_error()
    assert lib.mase_hip_extract_mxfp(x.data_ptr(), 2, sc.data_ptr(), el.data_ptr(), 64, 32, 4, 4, 1, 0, None) == -1
    assert lib.mase_hip_extract_mxfp(x.data_ptr(), 7, sc.data_ptr(), el.data_ptr(), 64, 32, 4, 3, 1, 0, None) == -1
    assert lib.mase_hip_extract_minifloat(x.data_ptr(), 2, el.data_ptr(), 64, 9, 9, 1, 0, None) == -1
    with pytest.raises(ValueError):
        _lib.check(lib.mase_hip_extract_mxfp(None, 2, sc.data_ptr(), el.data_ptr(), 64, 32, 4, 3, 1, 0, None))
