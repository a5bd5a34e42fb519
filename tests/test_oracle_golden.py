"""CPU tests: the checker (oracle/) against the vectors written by the reference's own PyTorch
"fake" path (tests/golden/*.npz, produced by tests/golden/make_fixtures.py), against the
known-answer tests the reference holds, and against closed forms.  No GPU needed."""
import hashlib
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import (GOLDEN, PRESETS, assert_bits_equal, assert_int_equal, bits_of, codes_tensor, from_bits, golden,
                     parse_cfg_key)
from oracle import torch_fake


# ----------------------------------------------------------------------------- golden vectors
def test_minifloat_extract_f32_vectors():
    d = golden("minifloat_extract_f32.npz")
    x = from_bits(d["x_f32_bits"], "float32")
    keys = [k for k in d.files if k.startswith("codes_")]
    assert len(keys) >= 30
    for k in keys:
        e, m, fin, rnd = parse_cfg_key(k[len("codes_"):])
        assert_int_equal(oracle.extract_minifloat(x, e, m, fin, rnd), d[k], f"C {k}")
        assert_int_equal(torch_fake.minifloat_encode(x, e, m, fin, rnd), d[k], f"torch {k}")


@pytest.mark.parametrize("dt", ["bfloat16", "float16"])
def test_minifloat_extract_every_16bit_pattern(dt):
    d = golden("minifloat_extract_all16.npz")
    x = from_bits(np.arange(1 << 16, dtype=np.uint32).astype(np.uint16), dt)
    keys = [k for k in d.files if k.startswith(dt + "_")]
    assert len(keys) == 8
    for k in keys:
        e, m, fin, rnd = parse_cfg_key(k[len(dt) + 1:])
        assert_int_equal(oracle.extract_minifloat(x, e, m, fin, rnd), d[k], f"C {k}")
        assert_int_equal(torch_fake.minifloat_encode(x, e, m, fin, rnd), d[k], f"torch {k}")


def test_minifloat_compose_whole_code_space():
    d = golden("minifloat_compose.npz")
    for k in [k for k in d.files if k.startswith("codes_")]:
        em, fin = k[len("codes_"):].split("_")
        e, m = (int(v) for v in em[1:].split("m"))
        codes = codes_tensor(d[k])
        for dt in ("float32", "bfloat16", "float16"):
            want = d[f"out_{dt}_{em}_{fin}"]
            got = oracle.compose_minifloat(codes, e, m, fin == "fin", getattr(torch, dt))
            assert_bits_equal(got, want, dt, f"C {k} {dt}")
            if e + m <= 9:  # the tensor-op version is slow on the 64K-code formats
                got = torch_fake.minifloat_decode(codes, e, m, fin == "fin", getattr(torch, dt))
                assert_bits_equal(got, want, dt, f"torch {k} {dt}")


@pytest.mark.parametrize("dt", ["bfloat16", "float16", "float32"])
def test_mxfp_block_vectors(dt):
    d = golden(f"mxfp_blocks_{dt}.npz")
    x = from_bits(d["x_bits"], dt)
    for tag, (e, m) in PRESETS.items():
        sc, el = oracle.extract_mxfp(x, 32, e, m)
        assert_int_equal(sc, d["scales_" + tag], f"C scales {dt} {tag}")
        assert_int_equal(el, d["elements_" + tag], f"C elements {dt} {tag}")
        sc_t, el_t = torch_fake.mxfp_split(x, 32, e, m)
        assert_int_equal(sc_t, d["scales_" + tag], f"torch scales {dt} {tag}")
        assert_int_equal(el_t, d["elements_" + tag], f"torch elements {dt} {tag}")
        for odt in sorted({dt, "float32"}):
            want = d[f"dq_{odt}_{tag}"]
            got = oracle.compose_mxfp(sc, el, 32, e, m, True, getattr(torch, odt))
            assert_bits_equal(got, want, odt, f"C dq {dt}->{odt} {tag}")
            got = torch_fake.mxfp_join(sc, el, e, m, True, getattr(torch, odt))
            assert_bits_equal(got, want, odt, f"torch dq {dt}->{odt} {tag}")
            got = oracle.qdq_mxfp(x, 32, e, m, True, "rn", getattr(torch, odt))
            assert_bits_equal(got, want, odt, f"C qdq {dt}->{odt} {tag}")


def test_mxfp_other_block_sizes_and_round_modes():
    d = golden("mxfp_blocks_misc.npz")
    keys = [k for k in d.files if k.startswith("scales_")]
    assert len(keys) == 2 * 4 * 5
    for k in keys:
        _, dt, b, em, rnd = k.split("_")
        bs = int(b[1:])
        e, m = (int(v) for v in em[1:].split("m"))
        x = from_bits(d[f"x_{dt}_b{bs}"], dt)
        sc, el = oracle.extract_mxfp(x, bs, e, m, True, rnd)
        assert_int_equal(sc, d[k], f"scales {k}")
        assert_int_equal(el, d["elements_" + k[7:]], f"elements {k}")
        assert_bits_equal(oracle.compose_mxfp(sc, el, bs, e, m, True, getattr(torch, dt)), d["dq_" + k[7:]], dt, f"dq {k}")


def test_mxfp_compose_every_scale_and_code():
    d = golden("mxfp_compose_table.npz")
    sc = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(256, 1)
    el = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(1, 256).repeat(256, 1)
    assert len(d.files) == 15
    for k in d.files:
        odt, tag = k.split("_", 1)
        e, m = PRESETS[tag]
        assert_bits_equal(oracle.compose_mxfp(sc, el, 256, e, m, True, getattr(torch, odt)), d[k], odt, f"C {k}")
        assert_bits_equal(torch_fake.mxfp_join(sc, el, e, m, True, getattr(torch, odt)), d[k], odt, f"torch {k}")


# ----------------------------------------------------------------------------- reference's own known answers
def minifloat_value(code: int, exp_bits: int, frac_bits: int) -> float:
    """Closed form of a code's value (independent of the checker's decode)."""
    sign = -1.0 if code >> (exp_bits + frac_bits) & 1 else 1.0
    field = (code >> frac_bits) & ((1 << exp_bits) - 1)
    frac = code & ((1 << frac_bits) - 1)
    bias = (1 << (exp_bits - 1)) - 1
    if field == 0:
        return sign * frac * 2.0 ** (1 - bias - frac_bits)
    return sign * (1 + frac / (1 << frac_bits)) * 2.0 ** (field - bias)


def test_fp4_code_table():
    # the 16 FP4 E2M1 values (reference test/test_minifloat_fake.py:58-70)
    want = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]
    codes = torch.arange(16, dtype=torch.int32).to(torch.uint16)
    got = oracle.compose_minifloat(codes, 2, 1, True, torch.float32)
    assert got.tolist() == want
    assert [minifloat_value(c, 2, 1) for c in range(16)] == want


@pytest.mark.parametrize("e,m", [(4, 3), (5, 2), (2, 3), (3, 2), (2, 1), (3, 4), (5, 10), (8, 7)])
def test_compose_matches_closed_form(e, m):
    n = 1 << (e + m + 1)
    codes = torch.arange(n, dtype=torch.int32).to(torch.uint16)
    got = oracle.compose_minifloat(codes, e, m, True, torch.float32).double()
    want = torch.tensor([minifloat_value(c, e, m) for c in range(n)], dtype=torch.float64)
    # exact in fp32 except where the value needs fp32-subnormal rounding or overflows (8,7)
    ok = (want.abs() >= 2.0 ** -126) & (want.abs() < 2.0 ** 128) | (want == 0)
    assert torch.equal(got[ok], want[ok])


FORMAT_EXTREMA = {  # (max_normal, min_normal, max_subnormal, min_subnormal), test_minifloat_fake.py:43-55
    (2, 1): (6.0, 1.0, 0.5, 0.5),
    (2, 3): (7.5, 1.0, 0.875, 0.125),
    (3, 2): (28.0, 0.25, 0.1875, 0.0625),
    (4, 3): (480.0, 2.0 ** -6, 2.0 ** -6 * 0.875, 2.0 ** -9),
}


@pytest.mark.parametrize("fmt", list(FORMAT_EXTREMA))
def test_format_extrema_and_saturation(fmt):
    e, m = fmt
    max_normal, min_normal, max_sub, min_sub = FORMAT_EXTREMA[fmt]
    top = (1 << (e + m)) - 1
    vals = oracle.compose_minifloat(torch.tensor([top, 1 << m, (1 << m) - 1, 1], dtype=torch.int32).to(torch.uint16),
                                    e, m, True, torch.float32)
    assert vals.tolist() == [max_normal, min_normal, max_sub, min_sub]
    # 2 * max_normal saturates to max_normal (test_minifloat_fake.py:110-123)
    x = torch.full((8,), 2 * max_normal)
    c = oracle.extract_minifloat(x, e, m)
    assert (oracle.compose_minifloat(c, e, m, True, torch.float32) == max_normal).all()


@pytest.mark.parametrize("e,m", [(4, 3), (5, 2), (2, 3), (3, 2), (2, 1)])
def test_extract_inverts_compose_on_representable_values(e, m):
    """extract(compose(c)) == c for every code the format can reach: all normal codes and the
    subnormal codes of the top subnormal binade.  The other subnormal codes are unreachable in
    the reference's encoder: their values come back as the sign-only code (or 0)."""
    n = 1 << (e + m + 1)
    codes = torch.arange(n, dtype=torch.int32).to(torch.uint16)
    back = oracle.extract_minifloat(oracle.compose_minifloat(codes, e, m, True, torch.float32), e, m)
    field = (codes.int() >> m) & ((1 << e) - 1)
    frac = codes.int() & ((1 << m) - 1)
    # subnormal codes: only the top binade [2^-bias, 2^(1-bias)) is reachable, and its lowest value
    # (zero mantissa, frac == 2^(m-1)) encodes to zero by the reference's rule
    reachable = (field > 0) | (frac > (1 << (m - 1)))
    expect = torch.where(reachable, codes.int(), (codes.int() >> (e + m)) << (e + m))
    expect[1 << (e + m)] = 0  # -0.0 is not < 0: no sign code
    assert torch.equal(back.int(), expect)


@pytest.mark.parametrize("e,m", [(4, 3), (5, 2), (2, 3), (3, 2), (2, 1)])
def test_interior_rounding_is_nearest_even(e, m):
    """Away from carries, exponent edges and the 8 dropped mantissa bits the encoder must agree
    with exact round-to-nearest-even computed in rational arithmetic."""
    from fractions import Fraction

    rng = np.random.default_rng(7)
    bias = (1 << (e - 1)) - 1
    emax = (1 << e) - 1 - bias
    xs, want = [], []
    for _ in range(4000):
        ex = int(rng.integers(1 - bias, emax + 1))
        mant = int(rng.integers(0, 1 << 15)) << 8  # low 8 bits zero: no truncation effect
        val = Fraction((1 << 23) + mant, 1 << 23) * Fraction(2) ** ex
        scaled = Fraction(mant, 1 << (23 - m))
        q = int(scaled)
        rem = scaled - q
        q += rem > Fraction(1, 2) or (rem == Fraction(1, 2) and q & 1)
        if q == 1 << m:
            continue  # carry: the reference's OR quirk, pinned by the golden vectors instead
        xs.append(float(val))
        want.append(((ex + bias) << m) | q)
    x = torch.tensor(xs, dtype=torch.float32)
    assert oracle.extract_minifloat(x, e, m).int().tolist() == want


def test_mxfp4_known_answers():
    # reference test/test_mxfp_fake.py:157-216: exact round trip of {6,1,.5,0} * 2^-120, block 8
    d = golden("mxfp4_known_answer.npz")
    for dt in ("float32", "bfloat16", "float16"):
        x = from_bits(d[f"x_{dt}"], dt)
        sc, el = oracle.extract_mxfp(x, 8, 2, 1)
        assert_int_equal(sc, d[f"scales_{dt}"], f"scales {dt}")
        assert_int_equal(el, d[f"elements_{dt}"], f"elements {dt}")
        y = oracle.compose_mxfp(sc, el, 8, 2, 1, True, getattr(torch, dt))
        assert_bits_equal(y, d[f"dq_{dt}"], dt, f"dq {dt}")
        assert torch.equal(y, x)  # the property the reference asserts
    x = torch.tensor([1.0, 0.0, 0.5, 0.5, -0.5, -0.5, -0.5, -0.5] + [0.0] * 8) * 2.0 ** -120
    sc, el = oracle.extract_mxfp(x, 8, 2, 1)
    assert torch.equal(oracle.compose_mxfp(sc, el, 8, 2, 1, True, torch.float32), x)


@pytest.mark.parametrize("tag", list(PRESETS))
def test_subnormal_inputs_dequantise_to_zero(tag):
    # reference test/test_mxfp_fake.py:133-154
    e, m = PRESETS[tag]
    g = torch.Generator().manual_seed(0)
    w = torch.randint(0, 0x7F, (512,), dtype=torch.int32, generator=g).view(torch.float32)
    sc, el = oracle.extract_mxfp(w, 32, e, m)
    assert (oracle.compose_mxfp(sc, el, 32, e, m, True, torch.float32) == 0).all()


@pytest.mark.parametrize("tag,limit", [("MXFP8_E4M3_fn", 0.05), ("MXFP8_E5M2_fn", 0.1), ("OCP_MXFP6_E2M3", 0.1),
                                       ("OCP_MXFP6_E3M2", 0.1), ("OCP_MXFP4_E2M1", 0.25)])
def test_error_envelope(tag, limit):
    # reference test/test_mxfp_fake.py:55-94
    e, m = PRESETS[tag]
    w = torch.randn(512, generator=torch.Generator().manual_seed(1)) * 100.0
    w_dq = oracle.qdq_mxfp(w, 32, e, m)
    assert ((w - w_dq).abs().mean() / w.abs().mean()).item() < limit


def test_closed_form_scale_for_half_precision_inputs():
    """scale = clamp(e_max - emax_unb, -127, ..) + 127 from the block's largest exponent field."""
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(256, 32, generator=g) * torch.exp2(torch.randint(-40, 40, (256, 1), generator=g).float())).to(torch.bfloat16)
    for tag, (e, m) in PRESETS.items():
        emax_unb = (1 << e) - 1 - ((1 << (e - 1)) - 1)
        sc, _ = oracle.extract_mxfp(x, 32, e, m)
        field = (x.view(torch.int16).int() >> 7) & 0xFF
        want = (field.max(dim=1).values - emax_unb).clamp(min=0)
        assert torch.equal(sc.flatten().int(), want), tag


# ----------------------------------------------------------------------------- full-size configurations
def _sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def _hashes():
    out = {}
    with open(os.path.join(GOLDEN, "config_hashes.txt")) as f:
        for line in f:
            cfg, name, h = line.split()
            out[(cfg, name)] = h
    return out


def test_config_c1_hashes():
    from workloads import make_c1

    want = _hashes()
    x = make_c1()
    if _sha(bits_of(x)) != want[("c1", "input")]:
        pytest.skip("this torch build draws a different random stream than the one the hashes were made with")
    sc, el = oracle.extract_mxfp(x, 32, 4, 3)
    assert _sha(sc.numpy()) == want[("c1", "scales")]
    assert _sha(el.numpy()) == want[("c1", "elements")]
    assert _sha(bits_of(oracle.compose_mxfp(sc, el, 32, 4, 3, True, torch.bfloat16))) == want[("c1", "dq_bf16")]


def test_config_c2_hashes():
    from workloads import make_c2

    want = _hashes()
    x = make_c2()
    if _sha(bits_of(x)) != want[("c2", "input")]:
        pytest.skip("this torch build draws a different random stream than the one the hashes were made with")
    for e, m in ((4, 3), (5, 2)):
        c = oracle.extract_minifloat(x, e, m)
        assert _sha(bits_of(c)) == want[("c2", f"codes_e{e}m{m}")]
        assert _sha(bits_of(oracle.compose_minifloat(c, e, m, True, torch.float32))) == want[("c2", f"dq_f32_e{e}m{m}")]
        assert _sha(bits_of(oracle.qdq_minifloat(x, e, m))) == want[("c2", f"dq_f32_e{e}m{m}")]


def test_config_c3_hashes():
    from workloads import make_c3

    want = _hashes()
    x = make_c3()
    if _sha(bits_of(x)) != want[("c3", "input")]:
        pytest.skip("this torch build draws a different random stream than the one the hashes were made with")
    sc, el = oracle.extract_mxfp(x, 32, 2, 1)
    assert _sha(sc.numpy()) == want[("c3", "scales")]
    assert _sha(el.numpy()) == want[("c3", "elements")]
    yb = bits_of(oracle.compose_mxfp(sc, el, 32, 2, 1, True, torch.bfloat16)).copy()
    yb[(yb & 0x7FFF) > 0x7F80] = 0x7FC0
    assert _sha(yb) == want[("c3", "dq_bf16_nan_canonical")]


# ----------------------------------------------------------------------------- packed storage form of codes
def test_packed_codes_hand_computed_vectors():
    """Bit stream, least significant bit first: worked out by hand, not by the checker's formula."""
    from oracle import packing

    # 4-bit: codes 0x1, 0xF, 0x8, 0x3 -> bytes 0xF1, 0x38
    assert packing.pack_codes(np.array([0x1, 0xF, 0x8, 0x3], np.uint8), 4).tolist() == [0xF1, 0x38]
    # 6-bit: codes 1, 0, 0, 0 -> bit 0 set; codes 0, 1, 0, 0 -> bit 6; 0, 0, 1, 0 -> bit 12 (byte 1 bit 4); 0, 0, 0, 1 -> bit 18 (byte 2 bit 2)
    assert packing.pack_codes(np.array([1, 0, 0, 0], np.uint8), 6).tolist() == [0x01, 0x00, 0x00]
    assert packing.pack_codes(np.array([0, 1, 0, 0], np.uint8), 6).tolist() == [0x40, 0x00, 0x00]
    assert packing.pack_codes(np.array([0, 0, 1, 0], np.uint8), 6).tolist() == [0x00, 0x10, 0x00]
    assert packing.pack_codes(np.array([0, 0, 0, 1], np.uint8), 6).tolist() == [0x00, 0x00, 0x04]
    # 6-bit: 0x3F, 0x00, 0x3F, 0x00 -> bits 0-5 and 12-17: 0x3F, 0xF0, 0x03
    assert packing.pack_codes(np.array([0x3F, 0, 0x3F, 0], np.uint8), 6).tolist() == [0x3F, 0xF0, 0x03]
    # 6-bit: 0x2A (101010), 0x15 (010101), 0x2A, 0x15 -> 0b01101010, 0b10100101, 0b01010110 read LSB first
    assert packing.pack_codes(np.array([0x2A, 0x15, 0x2A, 0x15], np.uint8), 6).tolist() == [0x6A, 0xA5, 0x56]
    # bits above the code width are dropped
    assert packing.pack_codes(np.array([0xF1, 0x2F], np.uint8), 4).tolist() == [0xF1]


@pytest.mark.parametrize("bits", [4, 6])
def test_packed_codes_round_trip(bits):
    from oracle import packing

    rng = np.random.default_rng(bits)
    codes = rng.integers(0, 1 << bits, size=4096, dtype=np.uint8)
    packed = packing.pack_codes(codes, bits)
    assert packed.size == codes.size * bits // 8
    assert np.array_equal(packing.unpack_codes(packed, bits, codes.size), codes)
    # every code value at every position of a group
    every = np.tile(np.arange(1 << bits, dtype=np.uint8), 4)
    for shift in range(4):
        c = np.roll(every, shift)
        assert np.array_equal(packing.unpack_codes(packing.pack_codes(c, bits), bits, c.size), c)
