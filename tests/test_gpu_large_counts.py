"""Element counts past 2^31: every kernel indexes with 64 bits.  A 2^31 + 2^21 element bf16 tensor (4.3 GB) is cast in
one call and compared with casts of 2^26-element pieces of it (first, the one ending at 2^31, last), bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def test_casts_past_two_to_the_31():
    from mase_hip.minifloat import kernels as mfk
    from mase_hip.minifloat.meta import FP8_E4M3_fn
    from mase_hip.mxfp import kernels as mxk
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn

    n, piece = (1 << 31) + (1 << 21), 1 << 26
    x = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(1)
    for i in range(0, n, piece):
        m = min(piece, n - i)
        x[i:i + m] = torch.randn(m, generator=g, device=DEV).to(torch.bfloat16)
    starts = (0, (1 << 31) - piece, n - piece)

    sc, el = mxk.extract_mxfp_components(x, MXFP8_E4M3_fn)
    y = mxk.compose_mxfp_tensor(sc, el, MXFP8_E4M3_fn, torch.bfloat16)
    q = mxk.quantize_dequantize(x, MXFP8_E4M3_fn, torch.bfloat16)
    for lo in starts:
        s2, e2 = mxk.extract_mxfp_components(x[lo:lo + piece].clone(), MXFP8_E4M3_fn)
        blocks = slice(lo // 32, (lo + piece) // 32)
        assert torch.equal(sc[blocks], s2) and torch.equal(el[blocks], e2), lo
        y2 = mxk.compose_mxfp_tensor(s2, e2, MXFP8_E4M3_fn, torch.bfloat16).view(torch.int16)
        assert torch.equal(y[lo:lo + piece].view(torch.int16), y2), lo
        assert torch.equal(q[lo:lo + piece].view(torch.int16), y2), lo
    del sc, el, y, q

    codes = mfk.extract_minifloat_component(x, FP8_E4M3_fn)
    z = mfk.compose_minifloat_component(codes, FP8_E4M3_fn, torch.bfloat16)
    for lo in starts:
        c2 = mfk.extract_minifloat_component(x[lo:lo + piece].clone(), FP8_E4M3_fn)
        assert torch.equal(codes[lo:lo + piece], c2), lo
        assert torch.equal(z[lo:lo + piece].view(torch.int16), mfk.compose_minifloat_component(c2, FP8_E4M3_fn, torch.bfloat16).view(torch.int16)), lo
