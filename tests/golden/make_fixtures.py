#!/usr/bin/env python3
"""Write the golden vectors under tests/golden/ from the reference's PyTorch "fake" path.

Run once, in a container that has the reference checkout:

    python tests/golden/make_fixtures.py [--ref /root/reference/src]

Only four reference functions are imported and called, the ones whose numerics no
reference-held test vector pins:

  * mase_triton.minifloat.fake.extract_minifloat_component   (minifloat/fake.py:7-78)
  * mase_triton.minifloat.fake.compose_minifloat_component   (minifloat/fake.py:81-125)
  * mase_triton.mxfp.fake.extract_mxfp_components            (mxfp/fake.py:11-59)
  * mase_triton.mxfp.fake.compose_mxfp_tensor                (mxfp/fake.py:62-79)

plus the two dataclasses they take (minifloat/meta.py:48, mxfp/meta.py:11).  Everything is
stored as raw bit patterns in compressed .npz files (loadable with allow_pickle=False):
inputs and the reference's outputs, nothing else.  The reference itself never leaves the
container; the tests read only these files.
"""
from __future__ import annotations

import argparse
import hashlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))

# (exp_bits, frac_bits, is_finite, round_mode) combinations pinned for the minifloat path.
PRESETS = [(4, 3), (5, 2), (2, 3), (3, 2), (2, 1)]
MINIFLOAT_CONFIGS = (
    [(e, m, True, "rn") for e, m in PRESETS]
    + [(e, m, True, r) for e, m in PRESETS for r in ("ru", "rd", "rz")]
    + [(e, m, False, "rn") for e, m in ((4, 3), (5, 2), (3, 2))]
    + [(8, 7, True, "rn"), (5, 10, True, "rn"), (5, 10, False, "rn"), (3, 4, True, "rn"),
       (6, 9, True, "rz"), (1, 1, True, "rn"), (1, 6, True, "rn"), (7, 1, True, "rn"),
       (7, 8, True, "rn")]
)
MXFP_FORMATS = {  # tag -> (exp_bits, frac_bits); block 32, 8-bit scale, rn, finite
    "MXFP8_E4M3_fn": (4, 3),
    "MXFP8_E5M2_fn": (5, 2),
    "OCP_MXFP6_E2M3": (2, 3),
    "OCP_MXFP6_E3M2": (3, 2),
    "OCP_MXFP4_E2M1": (2, 1),
}
TORCH_DT = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
NP_BITS = {"float32": np.uint32, "bfloat16": np.uint16, "float16": np.uint16}
TORCH_BITS = {"float32": torch.int32, "bfloat16": torch.int16, "float16": torch.int16}


def cfg_key(e, m, fin, rnd):
    return f"e{e}m{m}_{'fin' if fin else 'inf'}_{rnd}"


def bits_of(t: torch.Tensor) -> np.ndarray:
    """Raw bit pattern of a float tensor as an unsigned numpy array."""
    name = str(t.dtype).removeprefix("torch.")
    return t.contiguous().view(TORCH_BITS[name]).numpy().view(NP_BITS[name]).copy()


def from_bits(a: np.ndarray, name: str) -> torch.Tensor:
    signed = a.view(np.int32 if name == "float32" else np.int16)
    return torch.from_numpy(signed.copy()).view(TORCH_DT[name])


def u16(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


# --------------------------------------------------------------------------- inputs
def minifloat_fp32_inputs(rng: np.random.Generator) -> np.ndarray:
    """fp32 bit patterns: rounding ties +-1 at 15-bit and 23-bit granularity, carry edges,
    every binade edge of every pinned format, specials, and random bits."""
    out = []
    exps = sorted(set(list(range(-20, 20)) + [-126, -125, -100, -64, -63, -62, -33, -32, -31,
                                               31, 32, 33, 62, 63, 64, 100, 126, 127]))
    for m in (1, 2, 3, 4, 6, 7, 8, 9, 10):
        sh = 15 - m
        half = 1 << (sh - 1)
        rems = sorted({0, 1, half - 1, half, half + 1, (1 << sh) - 1} & set(range(1 << sh)))
        qs = range(1 << m) if m <= 4 else sorted({0, 1, 2, (1 << m) - 2, (1 << m) - 1,
                                                   (1 << (m - 1)) - 1, 1 << (m - 1)})
        for e in exps:
            for q in qs:
                for r in rems:
                    for low in (0, 1, 0x80, 0xFF):
                        f23 = (q << (23 - m)) | (r << 8) | low
                        bits = ((e + 127) << 23) | f23
                        out.append(bits)
                        out.append(bits | 0x80000000)
    special = [0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x007FFFFF, 0x807FFFFF,
               0x00400000, 0x80400000, 0x00800000, 0x80800000, 0x7F7FFFFF, 0xFF7FFFFF,
               0x7F800000, 0xFF800000, 0x7FC00000, 0xFFC00000, 0x7FA00000, 0xFFA00000,
               0x7F800001, 0xFF800001, 0x7FFFFFFF, 0xFFFFFFFF, 0x7FC12345, 0x7F912345,
               0x7FE00000, 0x7FF00000, 0x7FD55555, 0x7FBFFFFF, 0x7F8000FF, 0x7F800100]
    out.extend(special)
    a = np.array(out, dtype=np.uint64).astype(np.uint32)
    rnd_bits = rng.integers(0, 1 << 32, size=1 << 15, dtype=np.uint64).astype(np.uint32)
    gauss = (rng.standard_normal(1 << 14) * np.exp2(rng.integers(-12, 12, 1 << 14))).astype(np.float32)
    return np.unique(np.concatenate([a, rnd_bits, gauss.view(np.uint32)]))


def mxfp_inputs(dtype: str, block: int, rng: np.random.Generator) -> tuple[np.ndarray, dict]:
    """Blocks (rows) of `block` values as raw bits of `dtype`, grouped into named sections."""
    tdt = TORCH_DT[dtype]
    g = torch.Generator().manual_seed(int(rng.integers(1 << 31)))
    sections = {}

    def add(name, t):
        t = t.reshape(-1, block)
        sections[name] = t

    add("randn100", (torch.randn(96, block, generator=g) * 100.0).to(tdt))
    add("randn1", torch.randn(96, block, generator=g).to(tdt))
    chi = (torch.randn(96, block, 3, generator=g) ** 2).sum(-1) / 3.0
    add("student_t", (torch.randn(96, block, generator=g) / chi.sqrt() * 0.02).to(tdt))
    o = (torch.randn(32, block, generator=g) * 100.0)
    if dtype != "float16":
        o[:, 0] *= 2.0 ** 32
    else:
        o[:, 0] *= 2.0 ** 8
    add("outlier", o.to(tdt))

    # zeros / subnormal-range inputs of the input dtype
    z = torch.zeros(8, block)
    z[1] = -0.0
    z[2, ::2] = -0.0
    add("zeros", z.to(tdt))
    nb = NP_BITS[dtype]
    man_bits = {"float32": 23, "bfloat16": 7, "float16": 10}[dtype]
    sign_bit = 1 << (31 if dtype == "float32" else 15)
    sub = rng.integers(0, 1 << man_bits, size=(16, block), dtype=np.uint64)
    sub |= (rng.integers(0, 2, size=(16, block), dtype=np.uint64) * sign_bit)
    sub[0] = 0
    add("subnormal_in", from_bits(sub.astype(nb), dtype))
    # one normal value among subnormal inputs
    mix = sub[:8].copy()
    small_normal = {"float32": 0x00800000, "bfloat16": 0x0080, "float16": 0x0400}[dtype]
    for i in range(8):
        mix[i, i] = small_normal + i * 3 + (sign_bit if i % 2 else 0)
    add("subnormal_mix", from_bits(mix.astype(nb), dtype))

    # planted specials
    base = (torch.randn(48, block, generator=g) * 3.0).to(tdt)
    sp = bits_of(base).astype(np.uint64)
    inf_b = {"float32": 0x7F800000, "bfloat16": 0x7F80, "float16": 0x7C00}[dtype]
    qnan_b = {"float32": 0x7FC00000, "bfloat16": 0x7FC0, "float16": 0x7E00}[dtype]
    snan_b = {"float32": 0x7F800001, "bfloat16": 0x7F81, "float16": 0x7C01}[dtype]
    pay_b = {"float32": 0x7FD2A5A5, "bfloat16": 0x7FD3, "float16": 0x7F55}[dtype]
    allone = {"float32": 0x7FFFFFFF, "bfloat16": 0x7FFF, "float16": 0x7FFF}[dtype]
    kinds = [inf_b, inf_b | sign_bit, qnan_b, qnan_b | sign_bit, snan_b, pay_b,
             pay_b | sign_bit, allone]
    for i in range(48):
        pos = int(rng.integers(block))
        sp[i, pos] = kinds[i % len(kinds)]
        if i >= 32:  # two specials in the block
            sp[i, (pos + 5) % block] = kinds[(i * 3 + 1) % len(kinds)]
    sp[47, :] = inf_b  # a block of only +inf
    add("specials", from_bits(sp.astype(nb), dtype))

    # block max exactly a power of two / just around it
    emin, emax = {"float32": (-126, 127), "bfloat16": (-126, 127), "float16": (-14, 15)}[dtype]
    ks = list(range(emin, emax + 1))
    rows = []
    for k in ks:
        r = torch.rand(block, generator=g, dtype=torch.float64) * 2.0 - 1.0
        r = r * (2.0 ** k) * 0.999
        r[int(rng.integers(block))] = (2.0 ** k) * (1 if k % 2 else -1)
        rows.append(r)
    add("pow2_max", torch.stack(rows).to(torch.float32).to(tdt))
    rows = []
    for k in ks:  # max is the largest value below 2^(k+1) in this dtype
        r = torch.rand(block, generator=g, dtype=torch.float64) * (2.0 ** k)
        t = r.to(torch.float32).to(tdt)
        tb = bits_of(t).astype(np.uint64)
        top = (((k + {"float32": 127, "bfloat16": 127, "float16": 15}[dtype]) << man_bits)
               | ((1 << man_bits) - 1))
        tb[int(rng.integers(block))] = top
        rows.append(tb)
    add("below_pow2_max", from_bits(np.stack(rows).astype(nb), dtype))

    if dtype == "float32":
        # log2 rounding band: amax = 2^k * (1 - j*2^-24), j small
        rows = []
        for k in range(-125, 129):
            for j in (1, 2, 3, 5, 6, 11, 12, 22, 23, 44, 45, 46, 64):
                r = (torch.rand(block, generator=g) * 0.5).numpy().astype(np.float32)
                r = (r * np.float32(2.0) ** np.float32(min(k - 1, 127))).astype(np.float32)
                rb = r.view(np.uint32).astype(np.uint64)
                bits = (((k - 1 + 127) << 23) | ((1 << 23) - j))
                rb[int(rng.integers(block))] = bits | (0x80000000 if (k + j) % 3 == 0 else 0)
                rows.append(rb)
        add("log2_band", from_bits(np.stack(rows).astype(np.uint32), dtype))

    if dtype != "float16":
        # huge in-block dynamic range: quotients that land in the fp32 subnormal range or at 0
        rows = []
        for top_e in (127, 126, 120, 100, 60, 30, 24, 23, 22, 10, 0, -10, -60, -100):
            for rep in range(2):
                eb = np.clip(top_e + 127 - rng.integers(100, 200, size=block), 1, 254).astype(np.uint64)
                mb = rng.integers(0, 1 << man_bits, size=block, dtype=np.uint64)
                if rep == 0:
                    mb[::3] = 0
                sb = rng.integers(0, 2, size=block, dtype=np.uint64) * sign_bit
                rb = sb | (eb << man_bits) | mb
                # a ladder of exact powers of two straddling the underflow thresholds
                for i, d in enumerate(range(118, 118 + min(16, block - 1))):
                    e_i = top_e + 127 - (d + i * 2)
                    if 1 <= e_i <= 254:
                        rb[i] = (e_i << man_bits) | (sign_bit if i % 2 else 0) | (mb[i] if i % 4 == 3 else 0)
                rb[block - 1] = ((top_e + 127) << man_bits) | (3 << (man_bits - 2)) | (sign_bit if rep else 0)
                rows.append(rb)
        add("wide_range", from_bits(np.stack(rows).astype(nb), dtype))

    order = list(sections)
    mat = torch.cat([sections[k] for k in order], dim=0)
    index = {}
    row = 0
    for k in order:
        n = sections[k].shape[0]
        index[k] = (row, row + n)
        row += n
    return bits_of(mat), index


# --------------------------------------------------------------------------- main
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference/src")
    ap.add_argument("--skip-full", action="store_true", help="skip the full-size config hashes")
    args = ap.parse_args()
    sys.path.insert(0, args.ref)
    from mase_triton.minifloat import fake as mf_fake  # reference
    from mase_triton.minifloat.meta import MinifloatMeta  # reference
    from mase_triton.mxfp import fake as mx_fake  # reference
    from mase_triton.mxfp.meta import MXFPMeta  # reference

    torch.manual_seed(0)
    rng = np.random.default_rng(20240611)

    # ---------------- minifloat extract: fp32 corner inputs, all configs
    x32 = minifloat_fp32_inputs(rng)
    store = {"x_f32_bits": x32}
    xt = from_bits(x32, "float32")
    for (e, m, fin, rnd) in MINIFLOAT_CONFIGS:
        meta = MinifloatMeta(exp_bits=e, frac_bits=m, is_finite=fin, round_mode=rnd)
        store["codes_" + cfg_key(e, m, fin, rnd)] = u16(mf_fake.extract_minifloat_component(xt, meta))
    np.savez_compressed(os.path.join(HERE, "minifloat_extract_f32.npz"), **store)
    print("minifloat_extract_f32:", x32.size, "inputs x", len(MINIFLOAT_CONFIGS), "configs")

    # ---------------- minifloat extract: every bf16 and every fp16 bit pattern, rn presets
    all16 = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    store = {}
    for dt in ("bfloat16", "float16"):
        xt = from_bits(all16, dt)
        for (e, m) in PRESETS:
            for fin in (True, False):
                if not fin and (e, m) in ((2, 1), (2, 3)):
                    continue
                meta = MinifloatMeta(exp_bits=e, frac_bits=m, is_finite=fin, round_mode="rn")
                store[f"{dt}_{cfg_key(e, m, fin, 'rn')}"] = u16(
                    mf_fake.extract_minifloat_component(xt, meta))
    np.savez_compressed(os.path.join(HERE, "minifloat_extract_all16.npz"), **store)
    print("minifloat_extract_all16 written")

    # ---------------- minifloat compose: the whole code space of each config
    store = {}
    seen = set()
    for (e, m, fin, _r) in MINIFLOAT_CONFIGS:
        if (e, m, fin) in seen:
            continue
        seen.add((e, m, fin))
        meta = MinifloatMeta(exp_bits=e, frac_bits=m, is_finite=fin, round_mode="rn")
        n_codes = 1 << (e + m + 1)
        codes = np.arange(n_codes, dtype=np.uint32).astype(np.uint16)
        # plus junk above the sign bit, which compose must ignore or mask as the fake does
        extra = (rng.integers(0, 1 << 16, size=256, dtype=np.uint64)).astype(np.uint16)
        codes = np.concatenate([codes, extra])
        ct = torch.from_numpy(codes.view(np.int16).copy()).view(torch.uint16)
        k = f"e{e}m{m}_{'fin' if fin else 'inf'}"
        store["codes_" + k] = codes
        for dt in ("float32", "bfloat16", "float16"):
            y = mf_fake.compose_minifloat_component(ct, meta, output_dtype=TORCH_DT[dt])
            store[f"out_{dt}_{k}"] = bits_of(y)
    np.savez_compressed(os.path.join(HERE, "minifloat_compose.npz"), **store)
    print("minifloat_compose written")

    # ---------------- MXFP extract + compose on structured blocks
    for dt in ("bfloat16", "float16", "float32"):
        xb, index = mxfp_inputs(dt, 32, rng)
        store = {"x_bits": xb}
        for name, (lo, hi) in index.items():
            store["section_" + name] = np.array([lo, hi], dtype=np.int64)
        x = from_bits(xb, dt)
        for tag, (e, m) in MXFP_FORMATS.items():
            meta = MXFPMeta(block_size=32, scale_exp_bits=8, element_exp_bits=e,
                            element_frac_bits=m, element_is_finite=True, round_mode="rn")
            sc, el = mx_fake.extract_mxfp_components(x.flatten(), meta)
            assert sc.dtype == torch.uint8 and el.dtype == torch.uint8
            store[f"scales_{tag}"] = sc.numpy().copy()
            store[f"elements_{tag}"] = el.numpy().copy()
            for odt in sorted({dt, "float32"}):
                y = mx_fake.compose_mxfp_tensor(sc, el, meta, output_dtype=TORCH_DT[odt])
                store[f"dq_{odt}_{tag}"] = bits_of(y)
        np.savez_compressed(os.path.join(HERE, f"mxfp_blocks_{dt}.npz"), **store)
        print(f"mxfp_blocks_{dt}:", xb.shape[0], "blocks")

    # other block sizes and rounding modes (bf16 + fp32 inputs)
    store = {}
    for dt in ("bfloat16", "float32"):
        for bs in (8, 16, 64, 128):
            xb, _ = mxfp_inputs(dt, bs, rng)
            xb = xb[:: 7 if dt == "float32" else 3]
            x = from_bits(xb, dt)
            store[f"x_{dt}_b{bs}"] = xb
            for (e, m, rnd) in ((4, 3, "rn"), (2, 1, "rn"), (3, 2, "rz"), (5, 2, "ru"), (2, 3, "rd")):
                meta = MXFPMeta(block_size=bs, scale_exp_bits=8, element_exp_bits=e,
                                element_frac_bits=m, element_is_finite=True, round_mode=rnd)
                sc, el = mx_fake.extract_mxfp_components(x.flatten(), meta)
                store[f"scales_{dt}_b{bs}_e{e}m{m}_{rnd}"] = sc.numpy().copy()
                store[f"elements_{dt}_b{bs}_e{e}m{m}_{rnd}"] = el.numpy().copy()
                y = mx_fake.compose_mxfp_tensor(sc, el, meta, output_dtype=TORCH_DT[dt])
                store[f"dq_{dt}_b{bs}_e{e}m{m}_{rnd}"] = bits_of(y)
    np.savez_compressed(os.path.join(HERE, "mxfp_blocks_misc.npz"), **store)
    print("mxfp_blocks_misc written")

    # ---------------- MXFP compose: every (scale, code) pair
    sc_all = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(256, 1)
    el_all = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(1, 256).repeat(256, 1)
    store = {}
    for tag, (e, m) in MXFP_FORMATS.items():
        meta = MXFPMeta(block_size=256, scale_exp_bits=8, element_exp_bits=e,
                        element_frac_bits=m, element_is_finite=True, round_mode="rn")
        for odt in ("float32", "bfloat16", "float16"):
            y = mx_fake.compose_mxfp_tensor(sc_all, el_all, meta, output_dtype=TORCH_DT[odt])
            store[f"{odt}_{tag}"] = bits_of(y).reshape(256, 256)
    np.savez_compressed(os.path.join(HERE, "mxfp_compose_table.npz"), **store)
    print("mxfp_compose_table written")

    # ---------------- the reference's own tiny known-answer cases, as run through the fake
    # (test/test_mxfp_fake.py:157-216: block 8, E2M1, values {6,1,.5,0} * 2^-120)
    meta8 = MXFPMeta(block_size=8, scale_exp_bits=8, element_exp_bits=2, element_frac_bits=1,
                     element_is_finite=True, round_mode="rn")
    store = {}
    for dt in ("float32", "bfloat16", "float16"):
        x = torch.tensor([[6.0] * 4 + [-6.0] * 4, [1.0] * 4 + [-1.0] * 4, [0.5] * 4 + [-0.5] * 4,
                          [0.0] * 8], dtype=TORCH_DT[dt]).flatten() * (2 ** -120)
        sc, el = mx_fake.extract_mxfp_components(x, meta8)
        y = mx_fake.compose_mxfp_tensor(sc, el, meta8, output_dtype=TORCH_DT[dt])
        store[f"x_{dt}"] = bits_of(x)
        store[f"scales_{dt}"] = sc.numpy().copy()
        store[f"elements_{dt}"] = el.numpy().copy()
        store[f"dq_{dt}"] = bits_of(y)
    np.savez_compressed(os.path.join(HERE, "mxfp4_known_answer.npz"), **store)

    # ---------------- full-size configs: SHA-256 of inputs and outputs
    if not args.skip_full:
        sys.path.insert(0, os.path.dirname(HERE))
        from workloads import make_c1, make_c2, make_c3  # this repo's seeded generators

        lines = []

        def h(a: np.ndarray) -> str:
            return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()

        x = make_c1()
        meta = MXFPMeta(32, 8, 4, 3, True, "rn")
        sc, el = mx_fake.extract_mxfp_components(x.flatten(), meta)
        y = mx_fake.compose_mxfp_tensor(sc, el, meta, output_dtype=torch.bfloat16)
        lines += [f"c1 input {h(bits_of(x))}", f"c1 scales {h(sc.numpy())}",
                  f"c1 elements {h(el.numpy())}", f"c1 dq_bf16 {h(bits_of(y))}"]
        del sc, el, y
        x = make_c2()
        for (e, m) in ((4, 3), (5, 2)):
            mm = MinifloatMeta(e, m, True, "rn")
            c = mf_fake.extract_minifloat_component(x, mm)
            y = mf_fake.compose_minifloat_component(c, mm, output_dtype=torch.float32)
            lines += [f"c2 input {h(bits_of(x))}", f"c2 codes_e{e}m{m} {h(u16(c))}",
                      f"c2 dq_f32_e{e}m{m} {h(bits_of(y))}"]
        x = make_c3()
        meta = MXFPMeta(32, 8, 2, 1, True, "rn")
        sc, el = mx_fake.extract_mxfp_components(x.flatten(), meta)
        y = mx_fake.compose_mxfp_tensor(sc, el, meta, output_dtype=torch.bfloat16)
        yb = bits_of(y)
        nan = (yb & 0x7FFF) > 0x7F80
        yb[nan] = 0x7FC0  # NaN payload/sign is not stable across torch code paths
        lines += [f"c3 input {h(bits_of(x))}", f"c3 scales {h(sc.numpy())}",
                  f"c3 elements {h(el.numpy())}", f"c3 dq_bf16_nan_canonical {h(yb)}"]
        with open(os.path.join(HERE, "config_hashes.txt"), "w") as f:
            f.write("\n".join(dict.fromkeys(lines)) + "\n")
        print("config_hashes written")


if __name__ == "__main__":
    main()
