"""mase_hip_mxfp_gemm_static_ws: the K-split GEMM with its partial sums in a device array that belongs to the library,
for callers that cannot allocate.  Called through the C ABI and held bit for bit to mase_hip_mxfp_gemm_ws with a
workspace from torch (the same kernels and the same split plan run, so the additions happen in the same order), on two
calls in a row, the second on a smaller product that finds the first one's partial sums in the array."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _operands(mxk, meta, M, N, K, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    a = mxk.quantize_dequantize(torch.randn(M * K, generator=g, device=DEV).to(torch.bfloat16), meta, torch.bfloat16)
    w = (0.02 * torch.randn(N, K, generator=g, device=DEV)).to(torch.bfloat16)
    w_sc, w_el = mxk.extract_mxfp_components(w.view(-1), meta)
    bias = torch.randn(N, generator=g, device=DEV).to(torch.bfloat16)
    return a, w_sc, w_el, bias


def both(M, N, K, seed, out_code, out_dtype):
    """The product through mase_hip_mxfp_gemm_static_ws and through mase_hip_mxfp_gemm_ws with a workspace from torch; also the
    free device memory before and after the former.  The split plan depends on the device's compute-unit count: a shape
    that is not split there, or asks for more than the static array holds, skips the test."""
    import mase_hip.mxfp.kernels as mxk
    from mase_hip import _lib
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn as meta

    lib = _lib.load()
    stream = _lib.stream_ptr(torch.device(DEV))
    limit = 32 * 1024 * 1024
    a, w_sc, w_el, bias = _operands(mxk, meta, M, N, K, seed)
    need = lib.mase_hip_mxfp_gemm_workspace_bytes(1, M, N, K)
    if not 0 < need <= limit:
        pytest.skip(f"({M}, {N}, {K}) asks for {need} bytes of partial sums on this device: not a split shape that fits the static workspace")
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    y_ref = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
    rc = lib.mase_hip_mxfp_gemm_ws(a.data_ptr(), 2, None, None, 0, 0, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, bias.data_ptr(), 2,
                                   y_ref.data_ptr(), out_code, M, N, K, 32, ws.data_ptr(), need, stream)
    assert rc == 0, lib.mase_hip_last_error()
    y = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    rc = lib.mase_hip_mxfp_gemm_static_ws(a.data_ptr(), 2, None, None, 0, 0, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, bias.data_ptr(), 2,
                                          y.data_ptr(), out_code, M, N, K, 32, stream)
    assert rc == 0, lib.mase_hip_last_error()
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    # the split really ran: the unsplit kernels add in another order
    y_unsplit = torch.empty_like(y)
    assert lib.mase_hip_mxfp_gemm(a.data_ptr(), 2, None, None, 0, 0, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, bias.data_ptr(), 2,
                                  y_unsplit.data_ptr(), out_code, M, N, K, 32, stream) == 0
    torch.cuda.synchronize()
    assert not torch.equal(y.view(torch.uint8), y_unsplit.view(torch.uint8)), "the split path left no trace in the result"
    return y, y_ref, free_before, free_after


def test_static_workspace_matches_caller_workspace():
    # the first call on the device looks up the array (and may load the code object): not part of the memory comparison
    y, y_ref, _, _ = both(256, 2048, 14336, 1, 2, torch.bfloat16)
    assert torch.isfinite(y.float()).all() and torch.equal(y.view(torch.int16), y_ref.view(torch.int16))
    # second call, smaller product, fp32 output: the array still holds the first call's sums
    y, y_ref, free0, free1 = both(256, 512, 2048, 2, 0, torch.float32)
    assert torch.isfinite(y).all() and torch.equal(y.view(torch.int32), y_ref.view(torch.int32))
    assert free1 == free0, "the call changed the amount of free device memory"
    # and the first shape again, after the smaller one
    y, y_ref, free0, free1 = both(256, 2048, 14336, 3, 2, torch.bfloat16)
    assert torch.equal(y.view(torch.int16), y_ref.view(torch.int16)) and free1 == free0


def test_static_workspace_refuses_what_does_not_fit():
    from mase_hip import _lib

    lib = _lib.load()
    limit = 32 * 1024 * 1024
    shape = None
    for M in (512, 1024, 1536, 2048, 3072, 4096):
        for N, K in ((4096, 14336), (2048, 28672), (8192, 14336), (14336, 28672)):
            if lib.mase_hip_mxfp_gemm_workspace_bytes(1, M, N, K) > limit:
                shape = (M, N, K)
                break
        if shape:
            break
    if shape is None:
        pytest.skip("no candidate shape splits into more than the static workspace on this device")
    M, N, K = shape
    a = torch.zeros(M * K, dtype=torch.bfloat16, device=DEV)
    w_sc = torch.zeros(N * K // 32, dtype=torch.uint8, device=DEV)
    w_el = torch.zeros(N * K, dtype=torch.uint8, device=DEV)
    y = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
    rc = lib.mase_hip_mxfp_gemm_static_ws(a.data_ptr(), 2, None, None, 0, 0, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, None, 0, y.data_ptr(), 2,
                                          M, N, K, 32, _lib.stream_ptr(torch.device(DEV)))
    assert rc == -2
    assert b"static workspace" in lib.mase_hip_last_error()
    torch.cuda.synchronize()


def test_static_workspace_unsplit_shape_runs_without_the_array():
    """A shape that is not split takes the ordinary kernels; same result as mase_hip_mxfp_gemm."""
    import mase_hip.mxfp.kernels as mxk
    from mase_hip import _lib
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn as meta

    lib = _lib.load()
    M, N, K = 48, 1024, 512
    assert lib.mase_hip_mxfp_gemm_workspace_bytes(1, M, N, K) == 0
    a, w_sc, w_el, _ = _operands(mxk, meta, M, N, K, 4)
    stream = _lib.stream_ptr(torch.device(DEV))
    y0 = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    y1 = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    assert lib.mase_hip_mxfp_gemm(a.data_ptr(), 2, None, None, 0, 0, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, None, 0, y0.data_ptr(), 2,
                                  M, N, K, 32, stream) == 0
    assert lib.mase_hip_mxfp_gemm_static_ws(a.data_ptr(), 2, None, None, 0, 0, w_sc.data_ptr(), w_el.data_ptr(), 4, 3, None, 0, y1.data_ptr(), 2,
                                            M, N, K, 32, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
    # an unsplit call first and a split call after it (the order of a caller who warms up on a small shape)
    y, y_ref, _, _ = both(256, 2048, 14336, 5, 2, torch.bfloat16)
    assert torch.equal(y.view(torch.int16), y_ref.view(torch.int16))
