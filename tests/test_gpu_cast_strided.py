"""GPU parity tests for MXFP casts with blocks along a non-last axis, read in place.

The reference rotates the block axis last and copies before its flat kernel
(src/mase_triton/mxfp/helpers.py:4-24); scales and elements come out in the order of that
rotated tensor.  Bit-exact against (1) the vectors written by the reference's own "fake" path,
laid out so that their blocks run down the rows of a matrix, (2) the CPU checker applied to the
rotated copy, and (3) this package's flat kernels on the rotated copy.
"""
import pytest
import torch

import oracle
from helpers import PRESETS, assert_bits_equal, assert_int_equal, from_bits, golden

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def mh():
    import mase_hip.mxfp.functional as F
    import mase_hip.mxfp.kernels as mxk
    from mase_hip import _lib
    from mase_hip.mxfp.helpers import flatten_for_quantize
    from mase_hip.mxfp.meta import MXFPMeta

    _lib.load()

    class NS:
        pass

    ns = NS()
    ns.F, ns.mxk, ns.MXFPMeta, ns.flatten = F, mxk, MXFPMeta, flatten_for_quantize
    return ns


def mx_meta(mh, e, m, block=32, rnd="rn", finite=True):
    return mh.MXFPMeta(block_size=block, scale_exp_bits=8, element_exp_bits=e, element_frac_bits=m,
                       element_is_finite=finite, round_mode=rnd)


def rotated(x: torch.Tensor, block_dim: int) -> torch.Tensor:
    """x with ``block_dim`` moved last, flattened (on the CPU, for the checker)."""
    axes = list(range(x.ndim))
    axes.append(axes.pop(block_dim % x.ndim))
    return x.permute(axes).contiguous().flatten()


def unrotated(flat: torch.Tensor, shape, block_dim: int) -> torch.Tensor:
    nd = len(shape)
    block_dim %= nd
    rot = list(shape)
    rot.append(rot.pop(block_dim))
    back = list(range(nd))
    back.insert(block_dim, back.pop())
    return flat.reshape(rot).permute(back).contiguous()


@pytest.mark.parametrize("dt", ["bfloat16", "float16", "float32"])
@pytest.mark.parametrize("blocks_per_column", [1, 4])
def test_reference_vectors_laid_out_down_the_rows(mh, dt, blocks_per_column):
    """The reference's own block vectors (inf/NaN, zero, subnormal, extreme-scale blocks among
    them): column c of the matrix holds blocks c*bpc .. c*bpc+bpc-1, so the expected scales and
    elements are the fixture's, in the fixture's order."""
    d = golden(f"mxfp_blocks_{dt}.npz")
    xb = from_bits(d["x_bits"], dt).reshape(-1, 32)
    n_cols = xb.shape[0] // blocks_per_column
    keep = n_cols * blocks_per_column
    x = xb[:keep].reshape(n_cols, blocks_per_column * 32).t().contiguous().to(DEV)  # [K, inner]
    for tag, (e, m) in PRESETS.items():
        meta = mx_meta(mh, e, m)
        sc, el = mh.mxk.extract_mxfp_components_strided(x, 0, meta)
        assert sc.shape == (keep, 1) and el.shape == (keep, 32)
        assert_int_equal(sc, d["scales_" + tag][:keep], f"scales {dt} {tag}")
        assert_int_equal(el, d["elements_" + tag][:keep], f"elements {dt} {tag}")
        for odt in sorted({dt, "float32"}):
            want = from_bits(d[f"dq_{odt}_{tag}"].reshape(-1)[:keep * 32], odt)
            want = want.reshape(n_cols, blocks_per_column * 32).t().contiguous()
            got = mh.mxk.quantize_dequantize_strided(x, 0, meta, getattr(torch, odt))
            assert got.shape == x.shape and got.is_contiguous()
            assert_bits_equal(got, want, odt, f"qdq {dt}->{odt} {tag}")


@pytest.mark.parametrize("dt", ["bfloat16", "float16", "float32"])
@pytest.mark.parametrize("shape,block_dim", [
    ((64, 8), 0), ((32, 1), 0), ((96, 1028), 0), ((160, 1030), -2), ((3, 64, 20), 1), ((2, 3, 128, 36), -2),
    ((2, 32, 3, 5), 1), ((256, 4096), 0), ((5, 32, 4), -2), ((3, 128, 256), 1), ((2, 256, 2, 64), 1), ((384, 128), 0),
])
def test_strided_vs_checker_on_the_rotated_copy(mh, dt, shape, block_dim):
    g = torch.Generator().manual_seed(sum(shape) + block_dim)
    x = torch.randn(*shape, generator=g) * torch.exp2(torch.randint(-30, 30, shape, generator=g).float().mul(0.25).round())
    x[torch.rand(*shape, generator=g) < 0.01] = 0.0
    x = x.to(getattr(torch, dt))
    xd = x.to(DEV)
    flat = rotated(x, block_dim)
    for tag, (e, m) in PRESETS.items():
        meta = mx_meta(mh, e, m)
        sc_w, el_w = oracle.extract_mxfp(flat, 32, e, m)
        sc, el = mh.mxk.extract_mxfp_components_strided(xd, block_dim, meta)
        assert_int_equal(sc, sc_w, f"scales {dt} {tag}")
        assert_int_equal(el, el_w, f"elements {dt} {tag}")
        want = unrotated(oracle.compose_mxfp(sc_w, el_w, 32, e, m, True, x.dtype), shape, block_dim)
        assert_bits_equal(mh.mxk.quantize_dequantize_strided(xd, block_dim, meta, x.dtype), want, dt, f"qdq {dt} {tag}")


@pytest.mark.parametrize("inner", [64, 128])
def test_strided_special_blocks_and_scales(mh, inner):
    """(inner = 128 with K = 128 takes the whole-line-store extract kernel.)  bf16 matrix whose columns hold inf / NaN, all-zero blocks, blocks of subnormals, very large
    and very small magnitudes (scales near 0 and 254): the packed fast path must hand these to
    the exact routine."""
    K = 128
    g = torch.Generator().manual_seed(21)
    x = torch.randn(K, inner, generator=g)
    x[:, 1] *= 2.0 ** 120
    x[:, 2] *= 2.0 ** -120
    x[:, 3] = 0.0
    x[5, 4] = float("inf")
    x[40, 5] = float("nan")
    x[70, 6] = float("-inf")
    x[:, 7] *= 2.0 ** -133
    x[32:64, 8] = 0.0
    x[:, 9] *= 2.0 ** 127
    x[:, 10] = torch.where(torch.rand(K, generator=g) < 0.5, -0.0, 0.0)
    x[:, 11] *= 2.0 ** -100
    x = x.to(torch.bfloat16)
    xd = x.to(DEV)
    flat = rotated(x, 0)
    for tag, (e, m) in PRESETS.items():
        meta = mx_meta(mh, e, m)
        sc_w, el_w = oracle.extract_mxfp(flat, 32, e, m)
        sc, el = mh.mxk.extract_mxfp_components_strided(xd, 0, meta)
        assert_int_equal(sc, sc_w, f"scales {tag}")
        assert_int_equal(el, el_w, f"elements {tag}")
        want = unrotated(oracle.compose_mxfp(sc_w, el_w, 32, e, m, True, torch.bfloat16), (K, inner), 0)
        assert_bits_equal(mh.mxk.quantize_dequantize_strided(xd, 0, meta, torch.bfloat16), want, "bfloat16", f"qdq {tag}")


def test_strided_round_modes_and_output_dtypes(mh):
    K, inner = 64, 40
    g = torch.Generator().manual_seed(23)
    x = (torch.randn(K, inner, generator=g) * 5).to(torch.bfloat16)
    xd = x.to(DEV)
    flat = rotated(x, 0)
    for rnd in ("ru", "rd", "rz"):
        meta = mx_meta(mh, 4, 3, rnd=rnd)
        sc_w, el_w = oracle.extract_mxfp(flat, 32, 4, 3, True, rnd)
        sc, el = mh.mxk.extract_mxfp_components_strided(xd, 0, meta)
        assert_int_equal(sc, sc_w, f"scales {rnd}")
        assert_int_equal(el, el_w, f"elements {rnd}")
        for odt in (torch.float32, torch.float16, torch.bfloat16):
            want = unrotated(oracle.compose_mxfp(sc_w, el_w, 32, 4, 3, True, odt), (K, inner), 0)
            name = str(odt).removeprefix("torch.")
            assert_bits_equal(mh.mxk.quantize_dequantize_strided(xd, 0, meta, odt), want, name, f"qdq {rnd} {name}")


def test_strided_unaligned_view_and_in_place(mh):
    g = torch.Generator().manual_seed(25)
    base = torch.randn(64 * 36 + 1, generator=g).to(torch.bfloat16)
    x = base[1:].view(64, 36)
    xd = base.to(DEV)[1:].view(64, 36)
    meta = mx_meta(mh, 3, 2)
    sc_w, el_w = oracle.extract_mxfp(rotated(x, 0), 32, 3, 2)
    sc, el = mh.mxk.extract_mxfp_components_strided(xd, 0, meta)
    assert_int_equal(sc, sc_w, "scales")
    assert_int_equal(el, el_w, "elements")
    # in place through the C ABI: out == x
    from mase_hip import _lib
    y = x.clone().to(DEV)
    _lib.check(_lib.load().mase_hip_qdq_mxfp_strided(y.data_ptr(), 2, y.data_ptr(), 2, 1, 64, 36, 32, 3, 2, 1, 0,
                                                     _lib.stream_ptr(y.device)))
    want = unrotated(oracle.compose_mxfp(sc_w, el_w, 32, 3, 2, True, torch.bfloat16), (64, 36), 0)
    assert_bits_equal(y, want, "bfloat16", "in place")


def test_functional_api_takes_the_in_place_route(mh):
    """extract_mxfp_components / quantize_dequantize / compose with block_dim=-2: same tensors
    as the rotated-copy route through the flat kernels; a block axis that is not a multiple of
    32 still goes that way."""
    g = torch.Generator().manual_seed(27)
    meta = mx_meta(mh, 4, 3)
    for shape, bd in (((4, 96, 72), -2), ((96, 72), 0), ((2, 3, 64, 8), 2), ((4, 80, 72), -2)):
        x = torch.randn(*shape, generator=g).to(torch.bfloat16).to(DEV)
        sc, el, tm = mh.F.extract_mxfp_components(x, block_dim=bd, mxfp_meta=meta)
        sc_f, el_f = mh.mxk.extract_mxfp_components(mh.flatten(x, bd), meta)
        assert torch.equal(sc, sc_f) and torch.equal(el, el_f)
        y = mh.F.compose_mxfp_tensor(sc, el, tm)
        q = mh.F.quantize_dequantize(x, block_dim=bd, mxfp_meta=meta)
        assert y.shape == x.shape and q.shape == x.shape
        assert torch.equal(y.contiguous().view(torch.int16), q.contiguous().view(torch.int16))


def test_strided_full_size_weight(mh):
    """14336 x 4096 bf16 matrix quantised down its columns (what mxfp_matmul does to `other`),
    against the flat kernels on the transposed copy."""
    from workloads import make_c3

    x = make_c3().to(DEV)  # [14336, 4096]: blocks along axis 0
    meta = mx_meta(mh, 4, 3)
    sc, el = mh.mxk.extract_mxfp_components_strided(x, 0, meta)
    xt = x.t().contiguous().flatten()
    sc_f, el_f = mh.mxk.extract_mxfp_components(xt, meta)
    assert torch.equal(sc, sc_f) and torch.equal(el, el_f)
    q = mh.mxk.quantize_dequantize_strided(x, 0, meta, torch.bfloat16)
    q_f = mh.mxk.quantize_dequantize(xt, meta, torch.bfloat16).view(4096, 14336).t()
    assert torch.equal(q.view(torch.int16), q_f.contiguous().view(torch.int16))


def test_strided_argument_errors(mh):
    from mase_hip import _lib

    lib = _lib.load()
    x = torch.zeros(64, 8, dtype=torch.bfloat16, device=DEV)
    sc = torch.zeros(16, dtype=torch.uint8, device=DEV)
    el = torch.zeros(512, dtype=torch.uint8, device=DEV)
    s = _lib.stream_ptr(x.device)
    assert lib.mase_hip_extract_mxfp_strided(x.data_ptr(), 2, sc.data_ptr(), el.data_ptr(), 1, 64, 8, 16, 4, 3, 1, 0, s) == -2
    assert lib.mase_hip_extract_mxfp_strided(x.data_ptr(), 2, sc.data_ptr(), el.data_ptr(), 1, 48, 8, 32, 4, 3, 1, 0, s) == -2
    assert lib.mase_hip_extract_mxfp_strided(x.data_ptr(), 2, sc.data_ptr(), el.data_ptr(), 1, 64, 8, 32, 7, 3, 1, 0, s) == -1
    assert lib.mase_hip_extract_mxfp_strided(None, 2, sc.data_ptr(), el.data_ptr(), 1, 64, 8, 32, 4, 3, 1, 0, s) == -1
    assert lib.mase_hip_qdq_mxfp_strided(x.data_ptr(), 2, x.data_ptr(), 0, 1, 64, 8, 32, 4, 3, 1, 0, s) == -1
    assert lib.mase_hip_extract_mxfp_strided(x.data_ptr(), 2, sc.data_ptr(), el.data_ptr(), 0, 64, 8, 32, 4, 3, 1, 0, s) == 0
