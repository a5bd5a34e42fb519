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


def _gemm_operands(M, N, K, seed):
    """Quantised bf16 activations, MXFP8 weight components and the dequantised weight, generated on the GPU in pieces."""
    import mase_hip.mxfp.functional as F
    from mase_hip.mxfp import kernels as mxk
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn

    g = torch.Generator(device=DEV).manual_seed(seed)
    step = max(1, (1 << 27) // K)
    a = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
    for i in range(0, M, step):
        m = min(step, M - i)
        a[i:i + m] = mxk.quantize_dequantize(torch.randn(m * K, generator=g, device=DEV).to(torch.bfloat16), MXFP8_E4M3_fn,
                                             torch.bfloat16).view(m, K)
    w = torch.empty(N, K, dtype=torch.bfloat16, device=DEV)
    for i in range(0, N, step):
        m = min(step, N - i)
        w[i:i + m] = (0.02 * torch.randn(m, K, generator=g, device=DEV)).to(torch.bfloat16)
    sc, el, tm = F.extract_mxfp_components(w, block_dim=1, mxfp_meta=MXFP8_E4M3_fn)
    return a, sc, el, F.compose_mxfp_tensor(sc, el, tm)


def test_gemm_activations_past_4_gib_many_rows():
    """270336 x 8192 bf16 activations (4.4 GB): the tile kernels address with a 64-bit base per tile."""
    from mase_hip.mxfp import kernels as mxk
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn

    M, N, K = 270336, 256, 8192
    a, sc, el, wd = _gemm_operands(M, N, K, 0)
    y = mxk.mxfp_gemm(a, None, None, None, sc, el, MXFP8_E4M3_fn, None, M, N, K, torch.bfloat16)
    for lo in (0, 131072 - 512, 262144 - 512, M - 1024):   # around the rows where 32-bit byte offsets would wrap
        ref = (a[lo:lo + 1024].float() @ wd.float().T).to(torch.bfloat16).double()
        assert ((y[lo:lo + 1024].double() - ref).norm() / ref.norm()).item() <= 1e-3, lo


@pytest.mark.parametrize("K,split_k", [(1 << 23, True), (1 << 23, False), ((1 << 23) - 64, True)])
def test_gemm_activations_past_4_gib_long_k(K, split_k):
    """300 rows of 2^23 k (5 GB): the 128 x 128 kernel with K split over workgroups and unsplit, and (K not a multiple of
    128) the 256 x 128 kernel; fp32 output against float64."""
    from mase_hip.mxfp import kernels as mxk
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn

    M, N = 300, 128
    a, sc, el, wd = _gemm_operands(M, N, K, 1)
    y = mxk.mxfp_gemm(a, None, None, None, sc, el, MXFP8_E4M3_fn, None, M, N, K, torch.float32, split_k=split_k)
    ref = a.double() @ wd.double().T
    assert ((y.double() - ref).norm() / ref.norm()).item() <= 1e-4
