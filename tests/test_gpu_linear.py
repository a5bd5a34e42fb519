"""GPU parity tests for the dequant-fused MXFP GEMM, mxfp_linear / mxfp_matmul and the PTQ
layers.  Tolerance: relative Frobenius error <= 1e-3 against dequantize-then-matmul with fp32
(or wider) accumulation, as stated for this path; fp32 outputs are held to 1e-5."""
import pytest
import torch

import oracle
from helpers import PRESETS

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
REL_FRO_TOL = 1e-3


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


def preset(mh, tag):
    return getattr(mh.meta, tag)


def make_operands(M, N, K, x_tag, w_tag, seed=0):
    """bf16 x, w on the CPU plus their checker-side quantisation."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    xe, xm = PRESETS[x_tag]
    we, wm = PRESETS[w_tag]
    x_dq = oracle.qdq_mxfp(x, 32, xe, xm)
    w_sc, w_el = oracle.extract_mxfp(w, 32, we, wm)
    w_dq = oracle.compose_mxfp(w_sc, w_el, 32, we, wm, True, torch.bfloat16).view(N, K)
    return x, w, x_dq, w_sc, w_el, w_dq


@pytest.mark.parametrize("MNK", [(64, 64, 64), (128, 128, 32), (200, 136, 96), (1, 1, 32), (257, 129, 160), (384, 512, 1024)])
@pytest.mark.parametrize("x_tag,w_tag", [("MXFP8_E4M3_fn", "MXFP8_E4M3_fn"), ("MXFP8_E4M3_fn", "OCP_MXFP6_E3M2"),
                                         ("MXFP8_E5M2_fn", "OCP_MXFP4_E2M1"), ("OCP_MXFP6_E2M3", "MXFP8_E5M2_fn")])
def test_gemm_vs_checker(mh, MNK, x_tag, w_tag):
    M, N, K = MNK
    x, w, x_dq, w_sc, w_el, w_dq = make_operands(M, N, K, x_tag, w_tag, seed=M + N + K)
    y_ref = oracle.matmul_nt(x_dq, w_dq)  # float64 accumulation of the exact dequantised operands
    w_meta = preset(mh, w_tag)
    # dense (already quantised) A
    y32 = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), w_meta, None, M, N, K, torch.float32)
    assert y32.shape == (M, N)
    assert rel_fro(y32, y_ref) <= 1e-5
    y16 = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), w_meta, None, M, N, K, torch.bfloat16)
    assert rel_fro(y16, y_ref.to(torch.bfloat16)) <= REL_FRO_TOL
    # MXFP A: same bf16 operands, same summation order -> identical bits
    xe, xm = PRESETS[x_tag]
    x_sc, x_el = oracle.extract_mxfp(x, 32, xe, xm)
    y32b = mh.mxk.mxfp_gemm(None, x_sc.to(DEV), x_el.to(DEV), preset(mh, x_tag), w_sc.to(DEV), w_el.to(DEV), w_meta, None,
                            M, N, K, torch.float32)
    assert rel_fro(y32b, y32) <= 1e-6  # (another kernel, another summation order, for some shapes)


def test_gemm_bias_and_dtypes(mh):
    M, N, K = 96, 160, 128
    x, w, x_dq, w_sc, w_el, w_dq = make_operands(M, N, K, "MXFP8_E4M3_fn", "MXFP8_E4M3_fn", seed=3)
    w_meta = preset(mh, "MXFP8_E4M3_fn")
    for bdt in (torch.float32, torch.bfloat16, torch.float16):
        b = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(bdt)
        y_ref = oracle.matmul_nt(x_dq, w_dq) + b.float()
        for odt, tol in ((torch.float32, 1e-5), (torch.bfloat16, REL_FRO_TOL), (torch.float16, REL_FRO_TOL)):
            y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), w_meta, b.to(DEV), M, N, K, odt)
            assert y.dtype == odt
            assert rel_fro(y, y_ref.to(odt)) <= tol


def test_gemm_special_values_propagate(mh):
    """A weight block that held an inf composes to NaN/inf (scale 255) and must poison exactly
    the outputs of that row, as dequantize-then-matmul does."""
    M, N, K = 64, 64, 64
    g = torch.Generator().manual_seed(2)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    w[5, 40] = float("inf")
    w_sc, w_el = oracle.extract_mxfp(w, 32, 4, 3)
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), None,
                         M, N, K, torch.float32).cpu()
    assert y[:, 5].isnan().all()
    keep = torch.ones(N, dtype=torch.bool)
    keep[5] = False
    assert y[:, keep].isfinite().all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layer_type", ["XqWqB", "XWqB", "XqWB", "XWB", "XqWqBq"])
@pytest.mark.parametrize("bias", [True, False])
def test_mxfp_linear_fused_matches_separate(mh, dtype, layer_type, bias):
    """backend="fused" against backend="separate" (compose, then the vendor GEMM), both on the GPU."""
    M, N, K = 192, 256, 512
    g = torch.Generator().manual_seed(7)
    x = (torch.randn(3, M // 3, K, generator=g) * 3).to(dtype).to(DEV)
    lin = torch.nn.Linear(K, N, bias=bias, dtype=dtype, device=DEV)
    x_meta = preset(mh, "MXFP8_E4M3_fn") if layer_type.startswith("Xq") else None
    w_meta = preset(mh, "OCP_MXFP6_E3M2") if "Wq" in layer_type else None
    b_meta = preset(mh, "MXFP8_E4M3_fn") if layer_type.endswith("Bq") and bias else None
    fused = mh.MXFPLinearPTQ.from_linear(lin, x_meta, w_meta, b_meta, layer_type, "fused")
    separate = mh.MXFPLinearPTQ.from_linear(lin, x_meta, w_meta, b_meta, layer_type, "separate")
    y_f, y_s = fused(x), separate(x)
    assert y_f.shape == (3, M // 3, N) and y_f.dtype == dtype
    assert rel_fro(y_f, y_s) <= (REL_FRO_TOL if dtype == torch.bfloat16 else 1e-5)


def test_mxfp_linear_vs_cpu_reference_path(mh):
    """mxfp_linear(XqWqB, fused) against the tensor-op restatement of the reference's CPU path."""
    from oracle import torch_fake

    M, N, K = 256, 384, 512
    x, w, *_ = make_operands(M, N, K, "MXFP8_E4M3_fn", "MXFP8_E4M3_fn", seed=11)
    w_sc, w_el, w_tm = mh.F.extract_mxfp_components(w.to(DEV), block_dim=1, mxfp_meta=preset(mh, "MXFP8_E4M3_fn"))
    y = mh.F.mxfp_linear(x=x.to(DEV), x_meta=preset(mh, "MXFP8_E4M3_fn"), w=None, w_scales=w_sc, w_elements=w_el,
                         w_tensor_meta=w_tm, b=None, b_scales=None, b_elements=None, b_tensor_meta=None,
                         layer_type="XqWqB", backend="fused")
    y_ref = torch_fake.mxfp_linear_xq_wq(x, w_sc.cpu(), w_el.cpu(), (N, K), torch.bfloat16, (4, 3), (4, 3))
    assert y.dtype == torch.bfloat16
    assert rel_fro(y, y_ref) <= REL_FRO_TOL


@pytest.mark.parametrize("MNK,w_tag,odt", [
    ((4096, 4096, 128), "MXFP8_E4M3_fn", torch.bfloat16),    # 256 tiles, a single 128-k macro step per tile
    ((2048, 8320, 384), "OCP_MXFP6_E3M2", torch.bfloat16),   # 260 tiles: some workgroups take two, one XCD is short
    ((8192, 2048, 1024), "OCP_MXFP4_E2M1", torch.float16),   # one tile per workgroup, fp16 output
    ((1536, 16384, 256), "MXFP8_E5M2_fn", torch.bfloat16),   # 3 tile rows: the last group of tile rows is a single row
    ((16384, 1024, 512), "OCP_MXFP6_E2M3", torch.bfloat16),  # tall problem: 32 x 8 tiles
    ((1000, 14336, 256), "MXFP8_E4M3_fn", torch.bfloat16),   # M not a multiple of 512: the last tile row is shifted up
    ((3001, 5376, 384), "OCP_MXFP6_E3M2", torch.float16),    # 6 tile rows, the last one overlapping by 71 rows
    ((2048, 8320, 384), "MXFP8_E4M3_fn", torch.float32),     # fp32 output: 16 staging passes per tile, several tiles per workgroup
    ((1000, 12288, 128), "OCP_MXFP4_E2M1", torch.float32),   # fp32 output, shifted last tile row
    ((2048, 8320, 1536), "MXFP8_E4M3_fn", torch.bfloat16),   # K % 512 == 0: scales fetched 16 bytes at a time, three fetches per tile, several tiles per workgroup
    ((4096, 4096, 2560), "OCP_MXFP4_E2M1", torch.float32),   # the same with five fetches per tile, one tile per workgroup
    ((1024, 8192, 2176), "OCP_MXFP6_E2M3", torch.bfloat16),  # 17 macro steps: not a multiple of four, scales fetched every step
])
def test_gemm_large_tile_shapes(mh, MNK, w_tag, odt):
    """Shapes for which the launcher picks the 512 x 128 tile kernel (its tiles fill the CUs in whole rounds; dense A, no
    bias): the whole output
    against an fp32 dequantize-then-matmul on the GPU, and a sample of it against float64 accumulation."""
    M, N, K = MNK
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    we, wm = PRESETS[w_tag]
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    w_sc, w_el = oracle.extract_mxfp(w, 32, we, wm)
    w_dq = oracle.compose_mxfp(w_sc, w_el, 32, we, wm, True, torch.bfloat16).view(N, K)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, w_tag), None, M, N, K, odt)
    assert y.shape == (M, N) and y.dtype == odt
    tol = 1e-5 if odt == torch.float32 else REL_FRO_TOL
    y_gpu = (x_dq.to(DEV).float() @ w_dq.to(DEV).float().T).to(odt)
    assert rel_fro(y, y_gpu) <= tol
    rows = torch.arange(0, M, 61)
    cols = torch.arange(0, N, 37)
    y_ref = oracle.matmul_nt(x_dq[rows], w_dq[cols]).to(odt)
    assert rel_fro(y[rows.to(DEV)][:, cols.to(DEV)], y_ref) <= tol


@pytest.mark.parametrize("bdt", [torch.float32, torch.bfloat16, torch.float16])
def test_gemm_large_tile_bias(mh, bdt):
    """Bias on the 512 x 128 tile kernel (added to the fp32 accumulators before the output rounding)."""
    M, N, K = 4096, 4096, 256
    g = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(bdt)
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    w_sc, w_el = oracle.extract_mxfp(w, 32, 4, 3)
    w_dq = oracle.compose_mxfp(w_sc, w_el, 32, 4, 3, True, torch.bfloat16).view(N, K)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), b.to(DEV),
                         M, N, K, torch.bfloat16)
    y_gpu = (x_dq.to(DEV).float() @ w_dq.to(DEV).float().T + b.to(DEV).float()).to(torch.bfloat16)
    assert rel_fro(y, y_gpu) <= REL_FRO_TOL
    rows = torch.arange(0, M, 97)
    y_ref = (oracle.matmul_nt(x_dq[rows], w_dq) + b.float()).to(torch.bfloat16)
    assert rel_fro(y[rows.to(DEV)], y_ref) <= REL_FRO_TOL
    # the bias must land on the right columns: compare against the same call without it
    y0 = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), None,
                          M, N, K, torch.bfloat16)
    col_shift = (y.float() - y0.float()).mean(dim=0).cpu()
    assert torch.allclose(col_shift, b.float(), atol=0.02, rtol=0.02)
    # fp32 output: the bias lands exactly
    y32 = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), b.to(DEV),
                           M, N, K, torch.float32)
    y32_0 = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), None,
                             M, N, K, torch.float32)
    assert rel_fro(y32, x_dq.to(DEV).float() @ w_dq.to(DEV).float().T + b.to(DEV).float()) <= 1e-5
    assert torch.allclose((y32 - y32_0).cpu(), b.float().expand(M, N), atol=1e-5, rtol=1e-5)


def test_gemm_large_tile_special_values(mh):
    """Scale 255 (a block that held an inf) on the 512 x 128 tile kernel: that output column is NaN, the rest finite."""
    M, N, K = 4096, 4096, 256
    g = torch.Generator().manual_seed(11)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    w[777, 200] = float("inf")
    w[5, 3] = float("nan")
    w_sc, w_el = oracle.extract_mxfp(w, 32, 4, 3)
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), None,
                         M, N, K, torch.bfloat16).cpu()
    bad = torch.zeros(N, dtype=torch.bool)
    bad[777] = bad[5] = True
    assert y[:, bad].isnan().all()
    assert y[:, ~bad].isfinite().all()


@pytest.mark.parametrize("MNK,w_tag,odt,with_bias", [
    # one workgroup per 16 rows of W (M <= 64 and N up to 8192, 12288 for M <= 16)
    ((1, 1024, 128), "MXFP8_E4M3_fn", torch.bfloat16, False),     # one row, a single macro step
    ((16, 2048, 640), "OCP_MXFP4_E2M1", torch.float32, True),     # 5 macro steps, look-ahead 8: all loads in the prologue
    ((8, 8192, 1408), "MXFP8_E4M3_fn", torch.bfloat16, False),    # 11 macro steps: the 9-slot ring wraps
    ((12, 12288, 256), "OCP_MXFP6_E2M3", torch.float16, True),    # the largest N this kernel takes
    ((24, 6144, 896), "OCP_MXFP6_E3M2", torch.bfloat16, True),    # two 16-row tiles of A, look-ahead 4; 7 macro steps
    ((33, 512, 1024), "OCP_MXFP6_E3M2", torch.bfloat16, True),    # four tiles of A, the third holds one row
    ((64, 8192, 512), "OCP_MXFP4_E2M1", torch.float16, False),    # four full tiles, look-ahead 2
    ((64, 80, 256), "MXFP8_E5M2_fn", torch.float32, False),       # five workgroups; N not a multiple of 32
    # one workgroup per 32 rows of W
    ((8, 14336, 256), "MXFP8_E4M3_fn", torch.bfloat16, True),     # M <= 16: 16-row A stages, look-ahead 8
    ((16, 12320, 1280), "OCP_MXFP4_E2M1", torch.float32, False),  # 10 macro steps: that ring wraps
    ((24, 9216, 896), "OCP_MXFP6_E3M2", torch.bfloat16, True),    # 16 < M <= 32; 7 macro steps
    ((64, 8224, 512), "OCP_MXFP4_E2M1", torch.float16, False),    # two m-tiles
    ((100, 1024, 896), "OCP_MXFP6_E2M3", torch.bfloat16, False),  # four m-tiles, ragged; fewer workgroups than CUs: look-ahead 3
    ((128, 16512, 256), "MXFP8_E4M3_fn", torch.float32, True),    # four m-tiles, 516 workgroups: look-ahead 1
    ((128, 4096, 1536), "MXFP8_E4M3_fn", torch.float32, True),    # (K long enough to be split over workgroups instead)
    ((65, 96, 256), "MXFP8_E5M2_fn", torch.float16, False),       # three workgroups
])
def test_gemm_few_rows(mh, MNK, w_tag, odt, with_bias):
    """M <= 128 with K % 128 == 0 takes a kernel that streams W once: one workgroup per 16 rows of W (16x16x32 MFMA) for
    M <= 64 and moderate N, else one per 32 rows (32x32x16 MFMA, N % 32 == 0); in both K is split over the wavefronts
    and the partial sums are added through LDS."""
    M, N, K = MNK
    g = torch.Generator().manual_seed(M * 7 + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16) if with_bias else None
    we, wm = PRESETS[w_tag]
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    w_sc, w_el = oracle.extract_mxfp(w, 32, we, wm)
    w_dq = oracle.compose_mxfp(w_sc, w_el, 32, we, wm, True, torch.bfloat16).view(N, K)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, w_tag),
                         None if b is None else b.to(DEV), M, N, K, odt)
    assert y.shape == (M, N) and y.dtype == odt
    y_ref = oracle.matmul_nt(x_dq, w_dq)
    if b is not None:
        y_ref = y_ref + b.float()
    assert rel_fro(y, y_ref.to(odt)) <= (1e-5 if odt == torch.float32 else REL_FRO_TOL)


@pytest.mark.parametrize("M", [8, 40, 100])  # 16-row kernel with one / four tiles of A, 32-row kernel
def test_gemm_few_rows_special_values(mh, M):
    N, K = 256, 384
    g = torch.Generator().manual_seed(13)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    w[77, 300] = float("inf")
    w_sc, w_el = oracle.extract_mxfp(w, 32, 4, 3)
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), None,
                         M, N, K, torch.float32).cpu()
    assert y[:, 77].isnan().all()
    keep = torch.ones(N, dtype=torch.bool)
    keep[77] = False
    assert y[:, keep].isfinite().all()


@pytest.mark.parametrize("MNK,w_tag,odt,with_bias", [
    ((129, 128, 128), "MXFP8_E4M3_fn", torch.bfloat16, False),     # two m-tiles (the second holds one row), one macro step
    ((256, 256, 256), "OCP_MXFP4_E2M1", torch.float32, True),      # two macro steps: prologue only, fp32 output
    ((200, 384, 896), "OCP_MXFP6_E3M2", torch.bfloat16, True),     # 7 macro steps: the 6-step unrolled loop wraps, ragged M
    ((511, 1024, 1664), "MXFP8_E5M2_fn", torch.float16, False),    # four m-tiles, 13 macro steps, generic decode of E5M2
    ((384, 2048, 2048), "OCP_MXFP6_E2M3", torch.bfloat16, False),  # 48 tiles, K rotation wraps (16 n-tiles = 16 macro steps)
    ((300, 4352, 512), "MXFP8_E4M3_fn", torch.bfloat16, True),     # 34 n-tiles, more than the 4 macro steps: rotation modulo
    ((257, 128, 64), "MXFP8_E4M3_fn", torch.bfloat16, False),      # 256 x 128 tiles: two m-tiles (one row in the second), one step
    ((512, 256, 320), "OCP_MXFP6_E3M2", torch.float32, True),      # 5 steps of 64 k (K not a multiple of 128), fp32 output
    ((400, 640, 832), "OCP_MXFP4_E2M1", torch.float16, True),      # 13 steps: the 6-step unrolled loop wraps twice
    ((250, 1024, 1152), "MXFP8_E5M2_fn", torch.bfloat16, True),    # 128 x 128 tiles, 9 macro steps
    ((384, 14336, 256), "MXFP8_E4M3_fn", torch.bfloat16, False),   # 256 x 128 tiles by tile count: 224 of them against 336 of 128 x 128
    ((1100, 4096, 384), "OCP_MXFP6_E2M3", torch.float16, True),    # 256 x 128 tiles for many rows: 160 tiles in one round, ragged M
    ((1024, 4096, 256), "MXFP8_E4M3_fn", torch.bfloat16, True),    # 128 x 128 tiles for many rows: 256 tiles, exactly one per CU
])
def test_gemm_mid_rows(mh, MNK, w_tag, odt, with_bias):
    """M > 128 with N % 128 == 0: the 128 x 128 tile kernel (K % 128 == 0; eight wavefronts, K halves added through LDS,
    loads and compose placed between the MFMAs) or the 256 x 128 tile kernel (K % 64 == 0; eight wavefronts of 64 x 64,
    64-k steps), whichever the launcher estimates faster from the tile counts."""
    M, N, K = MNK
    g = torch.Generator().manual_seed(M * 3 + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.float32) if with_bias else None
    we, wm = PRESETS[w_tag]
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    w_sc, w_el = oracle.extract_mxfp(w, 32, we, wm)
    w_dq = oracle.compose_mxfp(w_sc, w_el, 32, we, wm, True, torch.bfloat16).view(N, K)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, w_tag),
                         None if b is None else b.to(DEV), M, N, K, odt)
    assert y.shape == (M, N) and y.dtype == odt
    y_gpu = x_dq.to(DEV).float() @ w_dq.to(DEV).float().T
    if b is not None:
        y_gpu = y_gpu + b.to(DEV)
    assert rel_fro(y, y_gpu.to(odt)) <= (1e-5 if odt == torch.float32 else REL_FRO_TOL)
    rows = torch.arange(0, M, 7)
    cols = torch.arange(0, N, 5)
    y_ref = oracle.matmul_nt(x_dq[rows], w_dq[cols])
    if b is not None:
        y_ref = y_ref + b[cols]
    assert rel_fro(y[rows.to(DEV)][:, cols.to(DEV)], y_ref.to(odt)) <= (1e-5 if odt == torch.float32 else REL_FRO_TOL)


@pytest.mark.parametrize("MNK,splits,w_tag,odt,with_bias", [
    ((256, 512, 2048), 4, "MXFP8_E4M3_fn", torch.bfloat16, True),      # 8 tiles, 16 macro steps of K: 4 splits of 4
    ((511, 1024, 3328), 4, "OCP_MXFP6_E3M2", torch.float32, False),    # 26 macro steps as 7 + 7 + 7 + 5, ragged M
    ((250, 1024, 2176), 4, "OCP_MXFP4_E2M1", torch.bfloat16, True),    # 17 macro steps as 5 + 5 + 5 + 2
    ((100, 1024, 2048), 4, "OCP_MXFP6_E2M3", torch.float16, True),     # one row of tiles, most of its rows past M
    ((65, 128, 8192), 16, "MXFP8_E5M2_fn", torch.bfloat16, False),     # a single tile, 16 splits (the most)
    ((384, 4096, 4096), 2, "MXFP8_E4M3_fn", torch.bfloat16, False),    # 96 tiles: a second workgroup per tile still fits
    ((512, 4096, 1024), 1, "MXFP8_E4M3_fn", torch.bfloat16, False),    # short K, large output: the partial sums would cost more
])
def test_gemm_split_k(mh, MNK, splits, w_tag, odt, with_bias):
    """Few 128 x 128 output tiles and a long K: given a workspace the library splits K over several workgroups per tile
    (fp32 partial sums, then a kernel that adds them and the bias).  Checked against the CPU checker and against the
    same call without a workspace."""
    from mase_hip import _lib

    M, N, K = MNK
    assert _lib.load().mase_hip_mxfp_gemm_workspace_bytes(1, M, N, K) == (splits * M * N * 4 if splits > 1 else 0)
    assert _lib.load().mase_hip_mxfp_gemm_workspace_bytes(0, M, N, K) == 0   # MXFP A is not split
    g = torch.Generator().manual_seed(M + 5 * N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.float32) if with_bias else None
    we, wm = PRESETS[w_tag]
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    w_sc, w_el = oracle.extract_mxfp(w, 32, we, wm)
    w_dq = oracle.compose_mxfp(w_sc, w_el, 32, we, wm, True, torch.bfloat16).view(N, K)
    args = (x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, w_tag), None if b is None else b.to(DEV),
            M, N, K, odt)
    y = mh.mxk.mxfp_gemm(*args)
    assert y.shape == (M, N) and y.dtype == odt
    y_ref = oracle.matmul_nt(x_dq, w_dq)
    if b is not None:
        y_ref = y_ref + b.float()
    tol = 1e-5 if odt == torch.float32 else REL_FRO_TOL
    assert rel_fro(y, y_ref.to(odt)) <= tol
    y_plain = mh.mxk.mxfp_gemm(*args, split_k=False)
    assert rel_fro(y, y_plain) <= tol
    if odt == torch.float32:
        assert not torch.equal(y, y_plain)  # another order of additions: equality would mean K was not split
    if splits == 1:
        assert torch.equal(y, y_plain)


@pytest.mark.parametrize("MNK,splits,odt,with_bias", [
    ((300, 4096, 12288), 4, torch.bfloat16, True),    # 2 x 32 tiles of 256 x 128, the second tile row mostly past M; 4 splits of 24
    ((384, 4096, 12416), 4, torch.float32, False),    # 97 macro steps as 25 + 25 + 25 + 22
    ((1000, 4096, 12288), 4, torch.bfloat16, True),   # 2 x 32 tiles of 512 x 128, the second shifted up to end at row M - 1; 4 splits
    ((1024, 4096, 12288), 4, torch.float32, False),   # the same tiles, fp32 output
    ((1024, 4096, 12800), 4, torch.bfloat16, False),  # 512 x 128 tiles, four splits of 25 macro steps: not a multiple of four, scales fetched every step
    ((1024, 4096, 6400), 2, torch.bfloat16, True),    # 50 macro steps in two splits of 25 (256 x 128 tiles: 64 tiles of 512 x 128 price higher here)
])
def test_gemm_split_k_larger_tiles(mh, MNK, splits, odt, with_bias):
    """Long K and an output too large for more than two splits of its 128 x 128 tiles: the split runs on 256 x 128 or
    512 x 128 tiles (the smaller tiles would allow fewer splits, or none).  The whole output against an fp32
    dequantize-then-matmul on the GPU, a sample of it against float64 accumulation, and the unsplit call."""
    from mase_hip import _lib

    M, N, K = MNK
    assert _lib.load().mase_hip_mxfp_gemm_workspace_bytes(1, M, N, K) == splits * M * N * 4
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16) if with_bias else None
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    w_sc, w_el = oracle.extract_mxfp(w, 32, 4, 3)
    w_dq = oracle.compose_mxfp(w_sc, w_el, 32, 4, 3, True, torch.bfloat16).view(N, K)
    args = (x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), None if b is None else b.to(DEV),
            M, N, K, odt)
    y = mh.mxk.mxfp_gemm(*args)
    tol = 1e-5 if odt == torch.float32 else REL_FRO_TOL
    y_gpu = x_dq.to(DEV).float() @ w_dq.to(DEV).float().T
    if b is not None:
        y_gpu = y_gpu + b.to(DEV).float()
    assert rel_fro(y, y_gpu.to(odt)) <= tol
    rows, cols = torch.arange(0, M, 7), torch.arange(0, N, 53)
    y_ref = oracle.matmul_nt(x_dq[rows], w_dq[cols])
    if b is not None:
        y_ref = y_ref + b[cols].float()
    assert rel_fro(y[rows.to(DEV)][:, cols.to(DEV)], y_ref.to(odt)) <= tol
    y_plain = mh.mxk.mxfp_gemm(*args, split_k=False)
    assert rel_fro(y, y_plain) <= tol
    if odt == torch.float32:
        assert not torch.equal(y, y_plain)


def test_gemm_split_k_special_values(mh):
    M, N, K = 200, 256, 2048
    g = torch.Generator().manual_seed(21)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    w[77, 300] = float("inf")      # first split
    w[130, 1999] = float("nan")    # last split
    w_sc, w_el = oracle.extract_mxfp(w, 32, 4, 3)
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), None,
                         M, N, K, torch.bfloat16).cpu()
    bad = torch.zeros(N, dtype=torch.bool)
    bad[77] = bad[130] = True
    assert y[:, bad].isnan().all()
    assert y[:, ~bad].isfinite().all()


def test_gemm_workspace_too_small_or_absent(mh):
    """The C entry point with a workspace falls back to the unsplit product when the workspace is missing or short."""
    from mase_hip import _lib

    lib = _lib.load()
    M, N, K = 256, 512, 2048
    g = torch.Generator(device=DEV).manual_seed(8)
    a = mh.mxk.quantize_dequantize(torch.randn(M * K, generator=g, device=DEV).to(torch.bfloat16), preset(mh, "MXFP8_E4M3_fn"),
                                   torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g, device=DEV)).to(torch.bfloat16)
    w_sc, w_el = mh.mxk.extract_mxfp_components(w.view(-1), preset(mh, "MXFP8_E4M3_fn"))
    need = lib.mase_hip_mxfp_gemm_workspace_bytes(1, M, N, K)
    assert need == 4 * M * N * 4
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)

    def run(ws_ptr, ws_bytes):
        y = torch.full((M, N), float("nan"), dtype=torch.float32, device=DEV)
        rc = lib.mase_hip_mxfp_gemm_ws(a.data_ptr(), 2, None, None, 0, 0, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, None, 0,
                                       y.data_ptr(), 0, M, N, K, 32, ws_ptr, ws_bytes, _lib.stream_ptr(torch.device(DEV)))
        assert rc == 0, lib.mase_hip_last_error()
        torch.cuda.synchronize()
        return y

    y_plain = mh.mxk.mxfp_gemm(a.view(M, K), None, None, None, w_sc, w_el, preset(mh, "MXFP8_E4M3_fn"), None, M, N, K,
                               torch.float32, split_k=False)
    y_split = run(ws.data_ptr(), need)
    assert rel_fro(y_split, y_plain) <= 1e-5 and not torch.equal(y_split, y_plain)
    assert torch.equal(run(None, need), y_plain)                 # no workspace
    assert torch.equal(run(ws.data_ptr(), need - 1), y_plain)    # one byte short
    assert lib.mase_hip_mxfp_gemm_ws(a.data_ptr(), 2, None, None, 0, 0, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, None, 0,
                                     y_plain.data_ptr(), 0, M, N, K, 32, ws.data_ptr() + 4, need - 4,
                                     _lib.stream_ptr(torch.device(DEV))) == -1   # misaligned workspace


@pytest.mark.parametrize("M", [200, 300])
def test_gemm_mid_rows_special_values(mh, M):
    """Scale 255 (a block that held an inf or NaN) on the 128 x 128 (M = 200, K = 640) and 256 x 128 (M = 300, K = 576,
    not a multiple of 128) tile kernels: those output columns are NaN, the rest finite."""
    N, K = 512, (640 if M == 200 else 576)
    g = torch.Generator().manual_seed(17)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16)
    w[77, 300] = float("inf")
    w[400, K - 1] = float("nan")
    w_sc, w_el = oracle.extract_mxfp(w, 32, 4, 3)
    x_dq = oracle.qdq_mxfp(x, 32, 4, 3)
    y = mh.mxk.mxfp_gemm(x_dq.to(DEV), None, None, None, w_sc.to(DEV), w_el.to(DEV), preset(mh, "MXFP8_E4M3_fn"), None,
                         M, N, K, torch.bfloat16).cpu()
    bad = torch.zeros(N, dtype=torch.bool)
    bad[77] = bad[400] = True
    assert y[:, bad].isnan().all()
    assert y[:, ~bad].isfinite().all()


@pytest.mark.parametrize("backend", ["fused", "fused_bf16", "fused_scaled"])
def test_config_c4_full_size(mh, backend):
    """x [16384,4096] . W [14336,4096]^T, both MXFP8 E4M3, on either kernel family ("fused" picks the block-scaled one
    here).  The whole output is compared with the GPU dequantize-then-matmul (fp32 accumulate, bf16 out); a sample of
    rows and columns with float64 accumulation on the CPU."""
    from workloads import make_c4

    x, w = make_c4()
    fmt = preset(mh, "MXFP8_E4M3_fn")
    xd, wd = x.to(DEV), w.to(DEV)
    w_sc, w_el, w_tm = mh.F.extract_mxfp_components(wd, block_dim=1, mxfp_meta=fmt)
    args = dict(x=xd, x_meta=fmt, w=None, w_scales=w_sc, w_elements=w_el, w_tensor_meta=w_tm, b=None, b_scales=None,
                b_elements=None, b_tensor_meta=None, layer_type="XqWqB")
    y = mh.F.mxfp_linear(**args, backend=backend)
    y_sep = mh.F.mxfp_linear(**args, backend="separate")
    assert y.shape == (16384, 14336) and y.dtype == torch.bfloat16
    num = (y.float() - y_sep.float()).square().sum().double().sqrt().item()
    den = y_sep.float().square().sum().double().sqrt().item()
    assert num / den <= REL_FRO_TOL
    rows = torch.arange(0, 16384, 257)
    cols = torch.arange(0, 14336, 113)
    x_dq = oracle.qdq_mxfp(x[rows], 32, 4, 3)
    w_dq = oracle.qdq_mxfp(w[cols], 32, 4, 3)
    y_ref = oracle.matmul_nt(x_dq, w_dq).to(torch.bfloat16)
    assert rel_fro(y[rows.to(DEV)][:, cols.to(DEV)], y_ref) <= REL_FRO_TOL


def test_fused_backend_picks_the_kernel_family_by_rows(mh):
    """backend="fused": without a prepared weight operand the bf16 kernels below SCALED_FROM_ROWS_UNPREPARED rows
    (bit-identical to "fused_bf16") and the block-scaled kernels from there on (bit-identical to "fused_scaled"); with the
    operand at hand the block-scaled kernels at every row count, for a K its weight-streaming kernels take in one piece and
    for a longer one.  Every result within the tolerance of the float64 checker."""
    from mase_hip.mxfp.functional import linear as lin

    fmt = preset(mh, "MXFP8_E4M3_fn")
    g = torch.Generator().manual_seed(11)
    for K in (512, 4608):
        w = torch.randn(256, K, generator=g).mul(0.02).to(torch.bfloat16)
        w_sc, w_el, w_tm = mh.F.extract_mxfp_components(w.to(DEV), block_dim=1, mxfp_meta=fmt)
        w_op = lin.scaled_weight_operand(w_sc, w_el, w_tm)
        w_dq = oracle.qdq_mxfp(w, 32, 4, 3)
        for rows in (1, 16, 17, 33, 56, 64, lin.SCALED_FROM_ROWS_UNPREPARED - 8, lin.SCALED_FROM_ROWS_UNPREPARED):
            x = torch.randn(rows, K, generator=g).to(torch.bfloat16)
            args = dict(x=x.to(DEV), x_meta=fmt, w=None, w_scales=w_sc, w_elements=w_el, w_tensor_meta=w_tm, b=None, b_scales=None,
                        b_elements=None, b_tensor_meta=None, layer_type="XqWqB")
            y_bf16 = mh.F.mxfp_linear(**args, backend="fused_bf16")
            y_scaled = mh.F.mxfp_linear(**args, backend="fused_scaled")
            assert torch.equal(mh.F.mxfp_linear(**args, backend="fused"), y_scaled if rows >= lin.SCALED_FROM_ROWS_UNPREPARED else y_bf16)
            assert torch.equal(mh.F.mxfp_linear(**args, backend="fused", w_operand=w_op), y_scaled), (K, rows)
            assert lin.takes_scaled_route(rows, True) and lin.takes_scaled_route(rows, False) == (rows >= lin.SCALED_FROM_ROWS_UNPREPARED)
            y_ref = oracle.matmul_nt(oracle.qdq_mxfp(x, 32, 4, 3), w_dq).to(torch.bfloat16)
            assert rel_fro(y_bf16, y_ref) <= REL_FRO_TOL
            assert rel_fro(y_scaled, y_ref) <= REL_FRO_TOL
    # what the block-scaled route does not take goes to the bf16 kernels under "fused" and is refused under "fused_scaled"
    x = torch.randn(2048, K, generator=g).to(torch.bfloat16).to(DEV)
    fmt5 = preset(mh, "MXFP8_E5M2_fn")
    args = dict(x=x, x_meta=fmt5, w=None, w_scales=w_sc, w_elements=w_el, w_tensor_meta=w_tm, b=None, b_scales=None,
                b_elements=None, b_tensor_meta=None, layer_type="XqWqB")
    assert torch.equal(mh.F.mxfp_linear(**args, backend="fused"), mh.F.mxfp_linear(**args, backend="fused_bf16"))
    with pytest.raises(NotImplementedError):
        mh.F.mxfp_linear(**args, backend="fused_scaled")


def test_layer_keeps_and_refreshes_its_weight_operand(mh):
    """MXFPLinearPTQ builds the block-scaled form of its weight on the first forward that takes that route, reuses it,
    and rebuilds it when the components are replaced."""
    fmt, wfmt = preset(mh, "MXFP8_E4M3_fn"), preset(mh, "OCP_MXFP6_E3M2")
    g = torch.Generator().manual_seed(4)
    lin = torch.nn.Linear(512, 264, bias=True, dtype=torch.bfloat16, device=DEV)
    layer = mh.MXFPLinearPTQ.from_linear(lin, fmt, wfmt, None, "XqWqB", "fused")
    sep = mh.MXFPLinearPTQ.from_linear(lin, fmt, wfmt, None, "XqWqB", "separate")
    small = torch.randn(40, 512, generator=g).to(torch.bfloat16).to(DEV)
    big = torch.randn(3, 200, 512, generator=g).to(torch.bfloat16).to(DEV)
    bf16_only = mh.MXFPLinearPTQ.from_linear(lin, fmt, wfmt, None, "XqWqB", "fused_bf16")
    bf16_only(small)
    assert bf16_only._scaled_w is None          # 40 rows on the bf16 kernels: no kernel there reads it, nothing cached
    assert layer._scaled_w is None
    layer(small)
    assert layer._scaled_w is not None
    layer.invalidate_weight_operand()
    y = layer(big)
    first = layer._scaled_w
    assert first is not None and y.shape == (3, 200, 264)
    assert rel_fro(y, sep(big)) <= REL_FRO_TOL
    layer(big)
    assert layer._scaled_w is first
    assert "_scaled_w" not in layer.state_dict() and len(layer.state_dict()) == len(sep.state_dict())
    # new weights in place: the cached form must follow
    lin2 = torch.nn.Linear(512, 264, bias=True, dtype=torch.bfloat16, device=DEV)
    other = mh.MXFPLinearPTQ.from_linear(lin2, fmt, wfmt, None, "XqWqB", "separate")
    layer.load_state_dict(other.state_dict())
    y2 = layer(big)
    assert layer._scaled_w is not first
    assert rel_fro(y2, other(big)) <= REL_FRO_TOL
    # a write that bypasses the version counter needs the explicit call
    second = layer._scaled_w
    layer.w_elements.data.copy_(sep.w_elements.data)
    layer.w_scales.data.copy_(sep.w_scales.data)
    layer.bias.data.copy_(sep.bias.data)
    layer.invalidate_weight_operand()
    assert rel_fro(layer(big), sep(big)) <= REL_FRO_TOL and layer._scaled_w is not second


def test_layer_repeat_calls_skip_the_checks_and_notice_changes(mh, monkeypatch):
    """A call like the previous one on the block-scaled route goes straight to the two kernels (same bits as the checked
    path); another shape, backend, activation format or weight goes through the checks again."""
    import mase_hip.mxfp.functional as MXFP_F
    import mase_hip.mxfp.layers as layers_mod

    calls = [0]
    real = MXFP_F.mxfp_linear

    def counted(*a, **k):
        calls[0] += 1
        return real(*a, **k)

    monkeypatch.setattr(layers_mod.MXFP_F, "mxfp_linear", counted)
    fmt, fmt4 = preset(mh, "MXFP8_E4M3_fn"), preset(mh, "OCP_MXFP4_E2M1")
    g = torch.Generator().manual_seed(8)
    lin = torch.nn.Linear(512, 264, bias=True, dtype=torch.bfloat16, device=DEV)
    layer = mh.MXFPLinearPTQ.from_linear(lin, fmt, fmt, None, "XqWqB", "fused")
    x = torch.randn(2, 8, 512, generator=g).to(torch.bfloat16).to(DEV)
    y0 = layer(x)
    y1 = layer(x)
    y2 = layer(x + 0)                                   # another tensor of the same kind
    assert calls[0] == 1 and torch.equal(y0, y1) and torch.equal(y0, y2) and y1.shape == (2, 8, 264)
    layer(x[:1])                                        # other shape
    assert calls[0] == 2
    layer(x)
    layer(x)
    assert calls[0] == 3
    layer.x_mxfp_meta = fmt4                            # other activation format
    y4 = layer(x)
    assert calls[0] == 4 and not torch.equal(y4, y0)
    assert torch.equal(y4, mh.MXFPLinearPTQ.from_linear(lin, fmt4, fmt, None, "XqWqB", "fused")(x))
    calls[0] = 4                                        # (the line above counted one for the other layer)
    layer.x_mxfp_meta = fmt
    layer(x)
    assert calls[0] == 5
    with torch.no_grad():
        layer.w_elements.copy_(layer.w_elements ^ 0x80)  # every sign flipped
        layer.bias.zero_()
    y5 = layer(x)
    assert calls[0] == 6
    layer.bias = None                                   # the fast path reads the bias of the moment
    y6 = layer(x)
    assert calls[0] == 6 and torch.equal(y5, y6)
    lin0 = torch.nn.Linear(512, 264, bias=False, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        lin0.weight.copy_(lin.weight)
    assert torch.equal(y6, -mh.MXFPLinearPTQ.from_linear(lin0, fmt, fmt, None, "XqWqB", "fused")(x))
    calls[0] = 6
    layer.backend = "separate"
    y7 = layer(x)
    assert calls[0] == 7 and rel_fro(y7, y6) <= REL_FRO_TOL
    layer.backend = "fused"
    layer(x)
    assert layer._fast_sig is not None
    y8 = layer(x[:, :0])                                # no rows: nothing to compute, nothing to remember
    assert y8.shape == (2, 0, 264) and layer._fast_sig is None


@pytest.mark.filterwarnings("ignore:mase_hip. an operand is not 16-byte aligned")
@pytest.mark.parametrize("backend", ["fused", "fused_bf16", "fused_scaled"])
@pytest.mark.parametrize("layer_type", ["XqWqB", "XWqB"])
def test_linear_input_layouts(mh, backend, layer_type):
    """Inputs as torch.nn.functional.linear takes them: one vector, no rows, a strided view, many leading axes; every fused
    backend against float64 on the quantised operands (the casts that produce them are checked bit for bit elsewhere), and
    in shape and dtype against "separate" on the same layer (whose bf16 result is rounded twice, product and bias, when
    torch is handed a strided 3-D input: not a yardstick for 1e-3)."""
    if backend == "fused_scaled" and layer_type != "XqWqB":
        pytest.skip("the block-scaled route needs quantised activations")
    fmt = preset(mh, "MXFP8_E4M3_fn")
    g = torch.Generator().manual_seed(12)
    lin = torch.nn.Linear(512, 136, bias=True, dtype=torch.bfloat16, device=DEV)
    x_meta = fmt if layer_type.startswith("Xq") else None
    layer = mh.MXFPLinearPTQ.from_linear(lin, x_meta, fmt, None, layer_type, backend)
    sep = mh.MXFPLinearPTQ.from_linear(lin, x_meta, fmt, None, layer_type, "separate")
    base = torch.randn(6, 70, 1024, generator=g).to(torch.bfloat16).to(DEV)
    cases = {
        "vector": base[0, 0, :512],
        "no rows": base[:, :0, :512],
        "no batch": base[:0, :, :512],
        "row-strided view": base[..., :512],
        "element-strided view": base[..., ::2],
        "transposed batch axes": base[..., :512].transpose(0, 1),
        "five axes": base[..., :512].reshape(2, 3, 7, 10, 512),
        "offset by one element": base.view(-1)[1:1 + 9 * 512].view(9, 512),
    }
    w_dq = mh.F.compose_mxfp_tensor(sep.w_scales, sep.w_elements, sep.w_tensor_meta).double()
    for name, x in cases.items():
        y, y_sep = layer(x), sep(x)
        assert y.shape == y_sep.shape == (*x.shape[:-1], 136) and y.dtype == y_sep.dtype, name
        if x.numel():
            x_dq = mh.F.quantize_dequantize(x, block_dim=-1, mxfp_meta=x_meta) if x_meta is not None else x
            y_ref = (x_dq.double() @ w_dq.t() + lin.bias.double()).to(y.dtype)
            assert rel_fro(y, y_ref) <= REL_FRO_TOL, name
            assert rel_fro(layer(x), y_ref) <= REL_FRO_TOL, name      # and again (the layer's repeat-call path)
            assert rel_fro(y_sep, y_ref) <= 4 * REL_FRO_TOL, name


@pytest.mark.parametrize("backend", ["fused", "fused_bf16"])
def test_config_c5_swiglu_chain(mh, backend):
    """down(silu(gate(x)) * up(x)) with MXFP6 E3M2 weights and MXFP8 E4M3 activations, on either kernel family ("fused"
    takes the block-scaled kernels at these sizes).

    Each of the three GEMMs (the down projection sums over K = 14336, the longest accumulation of any configuration) is held
    to 1e-3 against a float64 dequantize-then-matmul built from the checker's components, on a sample of rows and columns and
    on the very activations the GPU layer saw: that is the bar of this path, and it is the same for both kernel families.
    The chain's output is a weaker statement, because the quantiser between the layers amplifies: an intermediate that
    differs in its last bf16 bit can land in another MXFP8 code (a step of 2^-3 of its value) when the next layer quantises
    it.  The bf16 kernels differ from backend="separate" only in the order of fp32 additions, so their chain stays within 1e-3
    of it over the whole tensor and within 3e-3 of the checker's own chain on the sampled rows (three per-layer errors adding
    up).  The block-scaled matrix unit adds a block's products with fewer bits than fp32 (1 - 2e-5 per GEMM), which flips
    about one bf16 rounding in 300 of gate / up and from there one MXFP8 code in a few hundred of the down layer's input:
    its chain is held to 5e-3 against both."""
    from workloads import make_c5

    x, wg, wu, wd = make_c5()
    xfmt, wfmt = preset(mh, "MXFP8_E4M3_fn"), preset(mh, "OCP_MXFP6_E3M2")

    def layers(backend):
        out = []
        for w in (wg, wu, wd):
            lin = torch.nn.Linear(w.shape[1], w.shape[0], bias=False, dtype=torch.bfloat16, device=DEV)
            lin.weight.data.copy_(w)
            out.append(mh.MXFPLinearPTQ.from_linear(lin, xfmt, wfmt, None, "XqWqB", backend))
        return out

    def mlp(ls, inp):
        g, u, d = ls
        return d(torch.nn.functional.silu(g(inp)) * u(inp))

    xd = x.to(DEV)
    fused = layers(backend)
    y = mlp(fused, xd)
    y_sep = mlp(layers("separate"), xd)
    assert y.shape == (4, 2048, 4096)
    scaled = backend != "fused_bf16"
    assert fused[0]._scaled_w is not None   # both kernel families read the kept weight operand at these sizes
    assert rel_fro(y, y_sep) <= (5 * REL_FRO_TOL if scaled else REL_FRO_TOL)

    # ---- per layer, against the checker (float64 accumulation, bf16 output like the layer's)
    x2 = x.view(-1, 4096)
    rows = torch.arange(5, 8192, 523)                       # 16 rows of the 8192
    cols_wide = torch.arange(3, 14336, 389)                 # 37 of the 14336 outputs of gate / up
    cols_down = torch.arange(1, 4096, 111)                  # 37 of the 4096 outputs of down
    g_gpu, u_gpu = fused[0](xd).view(-1, 14336), fused[1](xd).view(-1, 14336)
    h_gpu = torch.nn.functional.silu(g_gpu) * u_gpu         # what the down layer is given
    d_gpu = fused[2](h_gpu)
    x_dq = oracle.qdq_mxfp(x2[rows], 32, 4, 3)
    for name, w, got in (("gate", wg, g_gpu), ("up", wu, u_gpu)):
        ref = oracle.matmul_nt(x_dq, oracle.qdq_mxfp(w[cols_wide], 32, 3, 2)).to(torch.bfloat16)
        err = rel_fro(got[rows.to(DEV)][:, cols_wide.to(DEV)], ref)
        assert err <= REL_FRO_TOL, f"{name}: {err}"
    h_dq = oracle.qdq_mxfp(h_gpu[rows.to(DEV)].cpu(), 32, 4, 3)
    ref = oracle.matmul_nt(h_dq, oracle.qdq_mxfp(wd[cols_down], 32, 3, 2)).to(torch.bfloat16)
    err = rel_fro(d_gpu[rows.to(DEV)][:, cols_down.to(DEV)], ref)
    assert err <= REL_FRO_TOL, f"down: {err}"

    # ---- the whole chain on the sampled rows, every step from the checker
    g_ref = oracle.matmul_nt(x_dq, oracle.qdq_mxfp(wg, 32, 3, 2)).to(torch.bfloat16)
    u_ref = oracle.matmul_nt(x_dq, oracle.qdq_mxfp(wu, 32, 3, 2)).to(torch.bfloat16)
    h_ref = torch.nn.functional.silu(g_ref) * u_ref
    y_ref = oracle.matmul_nt(oracle.qdq_mxfp(h_ref, 32, 4, 3), oracle.qdq_mxfp(wd, 32, 3, 2)).to(torch.bfloat16)
    err = rel_fro(y.view(-1, 4096)[rows.to(DEV)], y_ref)
    assert err <= (5 if scaled else 3) * REL_FRO_TOL, f"chain: {err}"


def test_forward_swiglu_is_the_expression(mh):
    """MXFPLinearPTQ.forward_swiglu(gate, up) against layer(silu(gate) * up): on the block-scaled route one kernel forms the
    product and quantises it (reading the two halves of a stacked projection's output as views), elsewhere the
    expression itself runs.  The fused kernel rounds where the two tensor operations round, so the outputs agree far
    inside the path's 1e-3 (the last bit of the exponential may move an element to a neighbouring code now and then);
    the down projection is also held to 1e-3 against a float64 product of the checker's dequantised operands, computed
    from the very gate and up values the layer saw."""
    from workloads import make_c5

    x, wg, wu, wd = make_c5()
    xfmt, wfmt = preset(mh, "MXFP8_E4M3_fn"), preset(mh, "OCP_MXFP6_E3M2")

    def layer(w, backend):
        lin = torch.nn.Linear(w.shape[1], w.shape[0], bias=False, dtype=torch.bfloat16, device=DEV)
        lin.weight.data.copy_(w)
        return mh.MXFPLinearPTQ.from_linear(lin, xfmt, wfmt, None, "XqWqB", backend)

    inter = wg.shape[0]
    gu, down = layer(torch.cat([wg, wu]), "fused"), layer(wd, "fused")
    t = gu(x.to(DEV))                                        # [4, 2048, 2 * 14336]
    gate, up = t[..., :inter], t[..., inter:]
    y = down.forward_swiglu(gate, up)
    y_expr = down(torch.nn.functional.silu(gate) * up)
    assert y.shape == y_expr.shape == (4, 2048, 4096)
    assert rel_fro(y, y_expr) <= 1e-4
    # against the checker on a sample of rows and columns
    rows = torch.arange(7, 8192, 523)
    cols = torch.arange(2, 4096, 111)
    g_cpu, u_cpu = gate.reshape(-1, inter)[rows.to(DEV)].cpu(), up.reshape(-1, inter)[rows.to(DEV)].cpu()
    h_cpu = torch.nn.functional.silu(g_cpu) * u_cpu
    ref = oracle.matmul_nt(oracle.qdq_mxfp(h_cpu, 32, 4, 3), oracle.qdq_mxfp(wd[cols], 32, 3, 2)).to(torch.bfloat16)
    err = rel_fro(y.view(-1, 4096)[rows.to(DEV)][:, cols.to(DEV)], ref)
    assert err <= REL_FRO_TOL, err
    # few rows, another backend, mismatched shapes: the expression
    small = t[0, :16]
    assert torch.equal(down.forward_swiglu(small[:, :inter], small[:, inter:]), down(torch.nn.functional.silu(small[:, :inter]) * small[:, inter:]))
    sep = layer(wd, "separate")
    part = t[0, :256]
    assert torch.equal(sep.forward_swiglu(part[:, :inter], part[:, inter:]), sep(torch.nn.functional.silu(part[:, :inter]) * part[:, inter:]))


def test_mxfp_matmul_one_matrix_takes_the_block_scaled_route(mh):
    """mxfp_matmul(XqWq, fused) of bfloat16 operands against ONE matrix with enough rows: the block-scaled GEMM, as in
    mxfp_linear.  Bit-identical to the same three kernels called by hand, within 1e-3 of backend="separate" and of a float64
    product of the checker's dequantised operands; with fewer rows, or batched `other`, the bf16 route as before."""
    from mase_hip.mxfp.functional import linear as lin

    fmt = preset(mh, "MXFP8_E4M3_fn")
    g = torch.Generator().manual_seed(8)
    K, N = 1024, 520
    a = torch.randn(2, 300, K, generator=g).to(torch.bfloat16)
    b = (0.05 * torch.randn(K, N, generator=g)).to(torch.bfloat16)
    assert 2 * 300 >= lin.SCALED_FROM_ROWS_UNPREPARED
    ad, bd = a.to(DEV), b.to(DEV)
    y = mh.F.mxfp_matmul(ad, bd, fmt, fmt, "XqWq", "fused")
    assert y.shape == (2, 300, N)
    w_sc, w_el = mh.mxk.extract_mxfp_components_strided(bd, -2, fmt)
    by_hand = mh.mxk.mxfp_gemm_scaled(mh.mxk.scaled_operand_from_dense(ad.reshape(-1, K), fmt),
                                      mh.mxk.scaled_operand_from_mxfp(w_sc, w_el, fmt, N, K), None, torch.bfloat16)
    assert torch.equal(y.view(-1, N), by_hand)
    assert rel_fro(y, mh.F.mxfp_matmul(ad, bd, fmt, fmt, "XqWq", "separate")) <= REL_FRO_TOL
    a_dq = oracle.qdq_mxfp(a.view(-1, K), 32, 4, 3)
    b_dq = oracle.qdq_mxfp(b.t().contiguous(), 32, 4, 3)            # blocks along K: rows of b^T
    y_ref = (a_dq.double() @ b_dq.double().t()).to(torch.bfloat16)
    assert rel_fro(y.view(-1, N), y_ref) <= REL_FRO_TOL
    # `other` with batch axes of one is the same matrix
    assert torch.equal(mh.F.mxfp_matmul(ad, bd.view(1, K, N), fmt, fmt, "XqWq", "fused"), y)
    # few rows: the bf16 kernels (another summation order: equal within the tolerance, not bit for bit required)
    few = ad[0, :64]
    assert rel_fro(mh.F.mxfp_matmul(few, bd, fmt, fmt, "XqWq", "fused"), mh.F.mxfp_matmul(few, bd, fmt, fmt, "XqWq", "separate")) <= REL_FRO_TOL


@pytest.mark.parametrize("func_type", ["XW", "XqW", "XWq", "XqWq"])
@pytest.mark.parametrize("backend", ["separate", "fused"])
def test_mxfp_matmul(mh, func_type, backend):
    g = torch.Generator().manual_seed(0)
    a = (torch.randn(2, 4, 128, 1024, generator=g) * 5).to(torch.bfloat16).to(DEV)
    b = (torch.randn(2, 4, 1024, 512, generator=g) * 3).to(torch.bfloat16).to(DEV)
    fmt = preset(mh, "MXFP8_E4M3_fn")
    y = mh.F.mxfp_matmul(a, b, fmt if "Xq" in func_type else None, fmt if "Wq" in func_type else None, func_type, backend)
    y_ref = torch.matmul(a, b)
    assert y.shape == y_ref.shape
    ratio = ((y - y_ref).abs().mean() / y_ref.abs().mean()).item()
    assert ratio == 0 if func_type == "XW" else ratio < 0.2  # reference test/test_mxfp_functional.py:248-252
    # and against the checker's quantisation of the same operands
    a_q = oracle.qdq_mxfp(a.cpu(), 32, 4, 3) if "Xq" in func_type else a.cpu()
    if "Wq" in func_type:
        bt = b.cpu().transpose(-1, -2).contiguous()
        b_q = oracle.qdq_mxfp(bt, 32, 4, 3).transpose(-1, -2)
    else:
        b_q = b.cpu()
    y_chk = torch.matmul(a_q.float(), b_q.float()).to(torch.bfloat16)
    assert rel_fro(y, y_chk) <= REL_FRO_TOL


@pytest.mark.parametrize("a_shape,b_shape,dtype", [
    ((3, 40, 256), (256, 192), torch.bfloat16),          # matrix `other`: one GEMM over all rows
    ((2, 600, 128), (2, 128, 320), torch.bfloat16),      # batched launch, 256 x 256 tiles (N not a multiple of 128)
    ((40, 16, 64), (40, 64, 96), torch.bfloat16),        # many batches, few rows each (16-row weight-streaming kernel)
    ((2, 4, 24, 96), (4, 96, 64), torch.bfloat16),       # `other` broadcast along the first batch axis (its components are expanded)
    ((3, 1, 24, 96), (1, 5, 96, 64), torch.bfloat16),    # both operands broadcast along one axis each
    ((24, 96), (5, 96, 64), torch.bfloat16),             # matrix `input` against batched `other`: A shared (stride 0)
    ((1, 1, 24, 96), (2, 3, 96, 64), torch.bfloat16),    # the same with explicit unit batch axes
    ((6, 200, 256), (6, 256, 256), torch.bfloat16),      # 128 x 128 tile kernel, batched
    ((2, 50, 128), (2, 128, 72), torch.float32),         # fp32 in and out
    ((2, 3, 32), (2, 32, 4), torch.bfloat16),            # outputs of a product not 16-byte aligned: dense route
    ((4, 48), (48, 40), torch.bfloat16),                 # contraction axis not a multiple of 32
])
def test_mxfp_matmul_fused_routes(mh, a_shape, b_shape, dtype):
    """Every route of the fused backend against the checker's quantisation of the same operands
    (`other` quantised down its second-to-last axis)."""
    g = torch.Generator().manual_seed(sum(a_shape))
    a = (torch.randn(*a_shape, generator=g) * 5).to(dtype)
    b = (torch.randn(*b_shape, generator=g) * 3).to(dtype)
    fmt = preset(mh, "MXFP8_E4M3_fn")
    a_q = oracle.qdq_mxfp(a, 32, 4, 3)
    bt = b.transpose(-1, -2).contiguous()
    b_q = oracle.qdq_mxfp(bt.flatten(), 32, 4, 3).view(bt.shape).transpose(-1, -2)
    for func_type in ("XqWq", "XWq"):
        y = mh.F.mxfp_matmul(a.to(DEV), b.to(DEV), fmt if func_type == "XqWq" else None, fmt, func_type, "fused")
        y_chk = torch.matmul((a_q if func_type == "XqWq" else a).double(), b_q.double()).to(dtype)
        assert y.shape == y_chk.shape and y.dtype == dtype
        tol = REL_FRO_TOL if dtype == torch.bfloat16 else 1e-5
        assert rel_fro(y, y_chk) <= tol, func_type
        y_sep = mh.F.mxfp_matmul(a.to(DEV), b.to(DEV), fmt if func_type == "XqWq" else None, fmt, func_type, "separate")
        assert rel_fro(y, y_sep) <= tol, func_type


def test_linear_with_inf_nan_element_format_takes_the_dense_route(mh):
    """element_is_finite=False: codes with the top exponent field mean inf / NaN.  The GEMM decodes that field as an ordinary
    binade, so such weights must not reach it: fused equals separate bit for bit (both compose, then F.linear)."""
    g = torch.Generator().manual_seed(12)
    M, N, K = 64, 128, 256
    meta = mh.meta.MXFPMeta(block_size=32, scale_exp_bits=8, element_exp_bits=4, element_frac_bits=3, element_is_finite=False,
                            round_mode="rn")
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w_el = torch.randint(0, 0x78, (N * K // 32, 32), generator=g, dtype=torch.uint8)
    w_el[5, 7] = 0x78                                   # +inf in this format, 256 in the finite one
    w_el[9, 1] = 0xFB                                   # NaN
    w_sc = torch.randint(120, 130, (N * K // 32, 1), generator=g, dtype=torch.uint8)
    tm = mh.meta.MXFPTensorMeta(device="cuda:0", dtype="bfloat16", shape=(N, K), block_dim=1, meta=meta)
    args = dict(x=x, x_meta=preset(mh, "MXFP8_E4M3_fn"), w=None, w_scales=w_sc.to(DEV), w_elements=w_el.to(DEV), w_tensor_meta=tm,
                b=None, b_scales=None, b_elements=None, b_tensor_meta=None, layer_type="XqWqB")
    y_f = mh.F.mxfp_linear(**args, backend="fused")
    y_s = mh.F.mxfp_linear(**args, backend="separate")
    row_inf, row_nan = (5 * 32 + 7) // K, (9 * 32 + 1) // K
    assert y_f[:, row_nan].isnan().all() and not torch.isfinite(y_f[:, row_inf]).any()
    same = (y_f.view(torch.int16) == y_s.view(torch.int16)) | (y_f.isnan() & y_s.isnan())
    assert same.all()
    with pytest.raises(AssertionError):
        mh.mxk.mxfp_gemm(x, None, None, None, w_sc.to(DEV), w_el.to(DEV), meta, None, M, N, K, torch.bfloat16)


def test_gemm_batched_entry_point(mh):
    """mase_hip_mxfp_gemm_batched through the C ABI: every product bit-identical to the single-product entry point on the same
    operands (the same kernel runs on every grid plane), with per-product, shared (stride 0) and padded strides, on shapes that
    take different kernels; and its argument checks."""
    from mase_hip import _lib

    lib = _lib.load()
    fmt = preset(mh, "MXFP8_E4M3_fn")
    stream = _lib.stream_ptr(torch.device(DEV))
    g = torch.Generator(device=DEV).manual_seed(21)
    for (B, M, N, K), a_shared, w_shared, pad in (((8, 128, 512, 1024), False, False, 0), ((5, 16, 256, 256), True, False, 0),
                                                  ((3, 300, 256, 128), False, True, 0), ((4, 640, 1536, 256), False, False, 64),
                                                  ((20, 1, 32, 32), False, False, 0), ((3, 70, 96, 160), False, False, 32)):
        a_stride = 0 if a_shared else M * K + pad
        w_stride = 0 if w_shared else N * K + pad
        y_stride = M * N + pad
        n_a = -(-((B - 1) * a_stride + M * K) // 32) * 32
        a = mh.mxk.quantize_dequantize(torch.randn(n_a, generator=g, device=DEV).to(torch.bfloat16), fmt, torch.bfloat16)
        w_el = torch.randint(0, 256, ((B - 1) * w_stride + N * K,), generator=g, device=DEV, dtype=torch.uint8)
        w_el[w_el % 128 == 127] = 0x3F                                  # keep the products finite
        w_sc = torch.randint(118, 130, (((B - 1) * w_stride + N * K) // 32,), generator=g, device=DEV, dtype=torch.uint8)
        y = torch.full(((B - 1) * y_stride + M * N,), float("nan"), dtype=torch.bfloat16, device=DEV)
        rc = lib.mase_hip_mxfp_gemm_batched(a.data_ptr(), 2, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, y.data_ptr(), 2, M, N, K, 32, B,
                                            a_stride, w_stride, y_stride, stream)
        assert rc == 0, lib.mase_hip_last_error()
        for b in range(B):
            y1 = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            rc = lib.mase_hip_mxfp_gemm(a.data_ptr() + 2 * b * a_stride, 2, None, None, 0, 0, w_sc.data_ptr() + b * w_stride // 32,
                                        w_el.data_ptr() + b * w_stride, 4, 3, None, 0, y1.data_ptr(), 2, M, N, K, 32, stream)
            assert rc == 0, lib.mase_hip_last_error()
            got = y[b * y_stride: b * y_stride + M * N].view(M, N)
            assert torch.isfinite(got.float()).all(), (B, M, N, K, b)
            assert torch.equal(got.view(torch.int16), y1.view(torch.int16)), (B, M, N, K, b)
        if pad:                                                          # the gaps between the products are left alone
            assert y[M * N: y_stride].isnan().all()
    p = a.data_ptr()
    bad = lambda **kw: lib.mase_hip_mxfp_gemm_batched(p, 2, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, y.data_ptr(), 2, 16, 32, 32, 32,
                                                      kw.get("B", 2), kw.get("a", 512), kw.get("w", 1024), kw.get("y", 512), stream)
    assert bad(B=0) == -1 and bad(B=70000) == -1
    assert bad(a=100) == -1 and bad(w=1000) == -1 and bad(y=100) == -1   # products would overlap
    assert bad(a=516) == -1 and bad(w=1040) == -1 and bad(y=516) == -1   # misaligned products
    assert lib.mase_hip_mxfp_gemm_batched(None, 2, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, y.data_ptr(), 2, 16, 32, 32, 32, 2, 512, 1024, 512,
                                          stream) == -1
    torch.cuda.synchronize()


def test_gemm_dispatch_boundaries(mh):
    """Shapes on both sides of every kernel-selection threshold (rows 16 / 17, 64 / 65, 128 / 129, 511 / 512 / 513; N and K that do
    or do not divide by the tile sizes; few and many tiles), each against fp32 dequantize-then-matmul on the GPU."""
    g = torch.Generator().manual_seed(99)
    fmt = preset(mh, "MXFP8_E4M3_fn")
    shapes = []
    for M in (1, 16, 17, 32, 33, 64, 65, 127, 128, 129, 255, 256, 257, 383, 511, 512, 513, 640, 1023, 1025):
        for N, K in ((128, 128), (96, 128), (160, 160), (256, 384), (384, 96), (48, 256)):
            shapes.append((M, N, K))
    shapes += [(16, 12288, 128), (16, 12304, 128), (17, 8192, 128), (17, 12288, 128), (64, 8208, 128), (64, 8224, 128),
               (129, 12288, 128), (511, 12288, 128), (512, 12288, 128), (513, 12288, 256), (640, 12416, 128), (130, 4160, 256)]
    worst = 0.0
    for M, N, K in shapes:
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
        x_dq = oracle.qdq_mxfp(x.flatten(), 32, 4, 3).view(M, K).to(DEV)
        w_sc, w_el = oracle.extract_mxfp(w, 32, 4, 3)
        w_dq = oracle.compose_mxfp(w_sc, w_el, 32, 4, 3, True, torch.bfloat16).view(N, K).to(DEV)
        b = torch.randn(N, generator=g).to(torch.bfloat16).to(DEV)
        for odt in (torch.bfloat16, torch.float32):
            y = mh.mxk.mxfp_gemm(x_dq, None, None, None, w_sc.to(DEV), w_el.to(DEV), fmt, b, M, N, K, odt)
            y_ref = (x_dq.float() @ w_dq.float().T + b.float()).to(odt)
            err = rel_fro(y, y_ref)
            worst = max(worst, err)
            assert err <= (REL_FRO_TOL if odt == torch.bfloat16 else 1e-5), (M, N, K, odt, err)
    assert worst > 0.0  # summation orders differ: exact equality everywhere would mean the kernels did not run
