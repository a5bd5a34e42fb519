"""CPU tests of the host side: the C-ABI library loads and exports what include/mase_hip.h
declares, argument checking that needs no GPU, format descriptors, layout helpers and the layer
plumbing.  Nothing here launches a kernel."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from mase_hip import _lib

    if not os.path.exists(_lib.library_path()):
        import importlib.util

        spec = importlib.util.spec_from_file_location("mase_hip_build", os.path.join(ROOT, "mase-triton_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build_library(verbose=False)
    return _lib.load()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mase_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mase_hip_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    from mase_hip import _lib

    names = declared_symbols()
    assert len(names) == 28
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/mase_hip.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes signatures out of step with the header"
    assert lib.mase_hip_abi_version() == 1


def test_argument_errors_without_a_gpu(lib):
    """Validation happens before any HIP call, so it can be exercised on a CPU-only host."""
    buf = (ctypes.c_uint8 * 256)()
    p = ctypes.addressof(buf)
    p += (-p) % 16
    assert lib.mase_hip_extract_mxfp(p, 2, p, p, 63, 32, 4, 3, 1, 0, None) == -1
    assert b"multiple of block_size" in lib.mase_hip_last_error()
    assert lib.mase_hip_extract_mxfp(p, 2, p, p, 64, 32, 6, 1, 1, 0, None) == -1
    assert lib.mase_hip_extract_mxfp(p, 5, p, p, 64, 32, 4, 3, 1, 0, None) == -1
    assert lib.mase_hip_extract_mxfp(p, 2, p, p, 64, 32, 4, 3, 1, 9, None) == -1
    assert lib.mase_hip_extract_mxfp(None, 2, p, p, 64, 32, 4, 3, 1, 0, None) == -1
    assert lib.mase_hip_extract_minifloat(p, 0, p, 16, 8, 8, 1, 0, None) == -1
    assert lib.mase_hip_extract_minifloat(p + 2, 2, p, 16, 4, 3, 1, 0, None) == -1
    assert b"aligned" in lib.mase_hip_last_error()
    assert lib.mase_hip_compose_minifloat(p, p, 3, 16, 4, 3, 1, None) == -1
    assert lib.mase_hip_qdq_minifloat(p, 0, p, 2, 16, 4, 3, 1, 0, None) == -1  # in place with different sizes
    # the block-scaled route: shapes and formats it does not take are refused before any launch
    assert lib.mase_hip_scaled_padded_rows(1) == 256 and lib.mase_hip_scaled_padded_rows(257) == 512
    assert lib.mase_hip_scaled_operand_from_dense(p, 2, 4, 3, 8, 96, p, p, None) == -2     # K % 128
    assert lib.mase_hip_scaled_operand_from_dense(p, 2, 5, 2, 8, 128, p, p, None) == -2    # E5M2
    assert lib.mase_hip_scaled_operand_from_dense(p, 0, 4, 3, 8, 128, p, p, None) == -2    # fp32 input
    assert lib.mase_hip_scaled_operand_from_dense_minifloat(p, 2, 5, 2, 8, 128, p, p, None) == -2    # E5M2
    assert lib.mase_hip_scaled_operand_from_dense_minifloat(p, 1, 4, 3, 8, 128, p, p, None) == -2    # fp16 input
    assert lib.mase_hip_scaled_operand_from_dense_minifloat(None, 2, 4, 3, 8, 128, p, p, None) == -1
    assert lib.mase_hip_mxfp_linear_scaled_scratch_bytes(16, 4096, 4096) == 256 * 4096 + 32 * 256 * 4      # the operand of x alone
    assert lib.mase_hip_mxfp_linear_scaled_scratch_bytes(40, 4096, 14336) == 256 * 14336 + 112 * 256 * 4 + 4 * 40 * 4096 * 4
    assert lib.mase_hip_mxfp_linear_scaled_scratch_bytes(16, 4096, 384) == 0
    assert lib.mase_hip_mxfp_linear_scaled(p, 2, 4, 3, 0, p, p, None, 0, p, 2, 8, 8, 512, None, 0, None) == -1          # no scratch
    assert lib.mase_hip_mxfp_linear_scaled(p, 2, 4, 3, 0, p, p, None, 0, p, 2, 8, 8, 512, p, 1024, None) == -1         # scratch too small
    assert lib.mase_hip_mxfp_linear_scaled(p, 2, 4, 3, 0, p, p, None, 0, p, 2, 8, 8, 384, p, 1 << 20, None) == -2      # K % 256
    assert lib.mase_hip_mxfp_linear_scaled(None, 2, 4, 3, 0, None, None, None, 0, None, 2, 0, 8, 512, None, 0, None) == 0  # no rows
    assert lib.mase_hip_scaled_operand_from_swiglu(p, None, 2, 128, 4, 3, 8, 128, p, p, None) == -1   # no up
    assert lib.mase_hip_scaled_operand_from_swiglu(p, p, 2, 64, 4, 3, 8, 128, p, p, None) == -1     # row stride below K
    assert lib.mase_hip_scaled_operand_from_swiglu(p, p, 2, 132, 4, 3, 8, 128, p, p, None) == -1    # row stride not a multiple of 8
    assert lib.mase_hip_scaled_operand_from_mxfp(p, p + 4, 4, 3, 8, 128, p, p, None) == -1  # alignment
    assert lib.mase_hip_mxfp_gemm_scaled(p, p, p, p, None, 0, p, 2, 8, 8, 384, None) == -2  # K % 256
    assert lib.mase_hip_mxfp_gemm_scaled(p, p, p, p, None, 0, p, 2, 8, 12, 512, None) == -2  # N % 8
    assert lib.mase_hip_mxfp_gemm_scaled(p, None, p, p, None, 0, p, 2, 8, 8, 512, None) == -1
    assert lib.mase_hip_mxfp_gemm(p, 2, None, None, 0, 0, p, p, 4, 3, None, 0, p, 2, 16, 16, 48, 32, None) == -1
    assert lib.mase_hip_mxfp_gemm(p, 2, None, None, 0, 0, p, p, 4, 3, None, 0, p, 2, 16, 16, 64, 16, None) == -2
    assert lib.mase_hip_mxfp_gemm(p, 0, None, None, 0, 0, p, p, 4, 3, None, 0, p, 2, 16, 16, 64, 32, None) == -2
    # n == 0 is a valid no-op, and so is a product with no rows of A
    assert lib.mase_hip_mxfp_gemm(None, 2, None, None, 0, 0, None, None, 4, 3, None, 0, None, 2, 0, 16, 64, 32, None) == 0
    assert lib.mase_hip_mxfp_gemm_scaled(None, None, None, None, None, 0, None, 2, 0, 8, 512, None) == 0
    assert lib.mase_hip_mxfp_gemm_prepared_w(None, 2, None, None, None, 0, None, 2, 0, 128, 128, None) == 0
    assert lib.mase_hip_mxfp_gemm(p, 2, None, None, 0, 0, p, p, 4, 3, None, 0, p, 2, -1, 16, 64, 32, None) == -1
    assert lib.mase_hip_mxfp_gemm(p, 2, None, None, 0, 0, p, p, 4, 3, None, 0, p, 2, 0, 0, 64, 32, None) == -1
    assert lib.mase_hip_extract_mxfp(None, 2, None, None, 0, 32, 4, 3, 1, 0, None) == 0
    assert lib.mase_hip_qdq_minifloat(None, 0, None, 0, 0, 4, 3, 1, 0, None) == 0


def test_cpu_tensors_are_refused_loudly():
    import mase_hip.minifloat.functional as MF
    import mase_hip.mxfp.functional as F
    from mase_hip.minifloat.meta import FP8_E4M3_fn
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn

    x = torch.randn(64)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        F.extract_mxfp_components(x, 0, MXFP8_E4M3_fn)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        F.quantize_dequantize(x, 0, MXFP8_E4M3_fn)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        MF.extract_minifloat_component(x, FP8_E4M3_fn)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        MF.quantize_dequantize(x, FP8_E4M3_fn)


def test_product_does_not_import_the_checker():
    """Nothing under the package may reach into oracle/ (it is test infrastructure)."""
    pkg = os.path.join(ROOT, "mase-triton_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src, f"{os.path.join(dirpath, f)} mentions the checker"


# ----------------------------------------------------------------------------- descriptors
def test_minifloat_presets_match_reference_table():
    # (max_normal, min_normal, max_subnormal, min_subnormal): reference test/test_minifloat_fake.py:43-55
    from mase_hip.minifloat import meta as M

    table = {
        M.FP4_E2M1_fn: (6.0, 1.0, 0.5, 0.5),
        M.FP6_E2M3_fn: (7.5, 1.0, 0.875, 0.125),
        M.FP6_E3M2_fn: (28.0, 0.25, 0.1875, 0.0625),
        M.FP8_E4M3_fn: (480.0, 2 ** -6, 2 ** -6 * 0.875, 2 ** -9),
    }
    for meta, want in table.items():
        assert (meta.max_normal, meta.min_normal, meta.max_subnormal, meta.min_subnormal) == want
        assert meta.is_finite and meta.round_mode == "rn"
    assert M.FP8_E5M2_fn.max_normal == 114688.0
    assert M.FP8_E4M3_fn.n_bits == 8 and M.FP6_E3M2_fn.n_bits == 6 and M.FP4_E2M1_fn.n_bits == 4
    assert M.MinifloatMeta(4, 3, False, "rn").max_normal == 240.0
    with pytest.raises(AssertionError):
        M.MinifloatMeta(8, 8, True, "rn")
    with pytest.raises(AssertionError):
        M.MinifloatMeta(0, 3, True, "rn")


def test_mxfp_meta_rules():
    from mase_hip.mxfp import meta as X

    for preset, em in ((X.MXFP8_E4M3_fn, (4, 3)), (X.MXFP8_E5M2_fn, (5, 2)), (X.OCP_MXFP6_E2M3, (2, 3)),
                       (X.OCP_MXFP6_E3M2, (3, 2)), (X.OCP_MXFP4_E2M1, (2, 1))):
        assert (preset.element_exp_bits, preset.element_frac_bits) == em
        assert preset.block_size == 32 and preset.scale_exp_bits == 8 and preset.element_is_finite
        assert preset.round_mode == "rn"
        el = preset.element_meta
        assert (el.exp_bits, el.frac_bits, el.is_finite, el.round_mode) == (*em, True, "rn")
    with pytest.raises(AssertionError):
        X.MXFPMeta(32, 7, 4, 3, True, "rn")
    with pytest.raises(AssertionError):
        X.MXFPMeta(32, 8, 3, 3, True, "rn")
    tm = X.MXFPTensorMeta(device=torch.device("cpu"), dtype=torch.bfloat16, shape=torch.Size([4, 64]), block_dim=1,
                          meta=X.MXFP8_E4M3_fn)
    assert (tm.device, tm.dtype, tm.shape) == ("cpu", "bfloat16", (4, 64))
    moved = tm.create(device="cuda:0")
    assert moved.device == "cuda:0" and moved.shape == tm.shape and moved.meta is tm.meta
    with pytest.raises(Exception):
        tm.device = "x"  # frozen


def test_minifloat_tensor_meta():
    from mase_hip.minifloat.meta import FP8_E4M3_fn, MinifloatTensorMeta

    tm = MinifloatTensorMeta(device=torch.device("cpu"), dtype=torch.float16, shape=torch.Size([3, 5]), meta=FP8_E4M3_fn)
    assert (tm.device, tm.dtype, tm.shape) == ("cpu", "float16", (3, 5))
    assert tm.create(dtype=torch.float32).dtype == "float32"


@pytest.mark.parametrize("block_dim", [0, 1, 2, -1, -2, -3])
def test_flatten_permute_round_trip(block_dim):
    # reference test/test_mxfp_functional.py:27-39
    from mase_hip.mxfp.functional import flatten_for_quantize, permute_for_dequantize

    x = torch.arange(24).reshape(2, 3, 4)
    flat = flatten_for_quantize(x, block_dim)
    assert flat.ndim == 1
    # the block axis is the fastest-varying one of the flat array
    moved = x.movedim(block_dim, -1)
    assert torch.equal(flat, moved.reshape(-1))
    back = permute_for_dequantize(flat, ori_shape=tuple(x.shape), block_dim=block_dim)
    assert back.shape == x.shape and torch.equal(back, x)


def test_parse_linear_type_and_errors():
    import mase_hip.mxfp.functional as F
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn, MXFPTensorMeta

    tm = MXFPTensorMeta("cpu", "float32", (4, 32), 1, MXFP8_E4M3_fn)
    assert F.parse_mxfp_linear_type(None, None, None) == "XWB"
    assert F.parse_mxfp_linear_type(MXFP8_E4M3_fn, tm, None) == "XqWqB"
    assert F.parse_mxfp_linear_type(None, tm, tm) == "XWqBq"
    x, w = torch.randn(2, 32), torch.randn(4, 32)
    kw = dict(x=x, x_meta=None, w=w, w_scales=None, w_elements=None, w_tensor_meta=None, b=None, b_scales=None,
              b_elements=None, b_tensor_meta=None)
    with pytest.raises(NotImplementedError):
        F.mxfp_linear(**kw, layer_type="YWB", backend="separate")
    with pytest.raises(NotImplementedError):
        F.mxfp_linear(**kw, layer_type="XWB", backend="magic")
    # unquantised operands never touch a kernel: plain linear on any device
    assert torch.equal(F.mxfp_linear(**kw, layer_type="XWB", backend="separate"), torch.nn.functional.linear(x, w))
    assert torch.equal(F.mxfp_linear(**kw, layer_type="XWB", backend="fused"), torch.nn.functional.linear(x, w))
    assert torch.equal(F.mxfp_matmul(x, w.t(), None, None, "XW", "fused"), x @ w.t())


def test_alias_as_mase_triton():
    import mase_hip

    mase_hip.alias_as_mase_triton()
    import mase_triton.mxfp.functional as MXFP_F
    from mase_triton.minifloat.functional import quantize_dequantize
    from mase_triton.mxfp.layers import MXFPLinearPTQ

    assert MXFP_F.extract_mxfp_tensor is MXFP_F.extract_mxfp_components
    assert MXFPLinearPTQ.__module__ == "mase_hip.mxfp.layers"
    assert callable(quantize_dequantize)


# ----------------------------------------------------------------------------- layers (no kernels involved)
def _cpu_components(n_out=8, n_in=64):
    from mase_hip.mxfp.meta import MXFP8_E4M3_fn, MXFPTensorMeta

    sc = torch.full((n_out * n_in // 32, 1), 127, dtype=torch.uint8)
    el = torch.zeros((n_out * n_in // 32, 32), dtype=torch.uint8)
    tm = MXFPTensorMeta("cpu", "float32", (n_out, n_in), 1, MXFP8_E4M3_fn)
    return sc, el, tm


def test_layer_from_quantized_plumbing_and_dtype_guard():
    from mase_hip.mxfp.layers import MXFPLinearPTQ
    from mase_hip.utils.qlayer import ChangeDtypeError, devices_equal

    sc, el, tm = _cpu_components()
    layer = MXFPLinearPTQ.from_quantized(sc, el, tm, bias=torch.zeros(8), b_scales=None, b_elements=None, b_tensor_meta=None,
                                         x_mxfp_meta=None, layer_type="XWqB", backend="separate")
    assert (layer.in_features, layer.out_features) == (64, 8)
    assert layer.weight is None and layer.bias.dtype == torch.float32
    assert layer.w_scales.dtype == torch.uint8 and not layer.w_scales.requires_grad
    assert set(layer.state_dict()) == {"bias", "w_scales", "w_elements"}
    assert "layer_type=XWqB" in repr(layer)
    layer.to(dtype=torch.float16)  # nn.Module.to only casts floating-point parameters
    assert layer.bias.dtype == torch.float16 and layer.w_elements.dtype == torch.uint8
    with pytest.raises(ChangeDtypeError):
        layer._apply(lambda t: t.to(torch.int32))  # anything that would re-type the codes
    layer2 = MXFPLinearPTQ.from_quantized(sc, el, tm, None, None, None, None, None, "XWqB", "separate")
    layer2.to(device="cpu")  # no dtype change: allowed
    assert layer2.w_tensor_meta.device == "cpu"
    assert devices_equal("cuda", "cuda:0") and not devices_equal("cpu", "cuda:0")


def test_layer_constructor_contract():
    from mase_hip.minifloat.layers import MinifloatLinearPTQ
    from mase_hip.minifloat.meta import FP8_E4M3_fn, MinifloatTensorMeta
    from mase_hip.mxfp.layers import MXFPLinearPTQ

    sc, el, tm = _cpu_components()
    with pytest.raises(AssertionError):  # both a dense weight and components
        MXFPLinearPTQ(torch.zeros(8, 64), None, None, None, None, "XWqB", w_scales=sc, w_elements=el, w_tensor_meta=tm)
    with pytest.raises(ValueError):  # both a dense bias and bias components
        MXFPLinearPTQ(None, torch.zeros(8), None, None, None, "XWqBq", w_scales=sc, w_elements=el, w_tensor_meta=tm,
                      b_scales=sc, b_elements=el, b_tensor_meta=tm)
    with pytest.raises(AssertionError):
        MXFPLinearPTQ(torch.zeros(8, 64, 2), None, None, None, None, "XWB")
    dense = MXFPLinearPTQ(torch.randn(8, 64), torch.randn(8), None, None, None, "XWB", backend="separate")
    x = torch.randn(3, 64)
    assert torch.equal(dense(x), torch.nn.functional.linear(x, dense.weight, dense.bias))

    codes = torch.zeros(8, 64, dtype=torch.uint16)
    mtm = MinifloatTensorMeta("cpu", "float32", (8, 64), FP8_E4M3_fn)
    ml = MinifloatLinearPTQ.from_quantized(codes, mtm, None, None, None, None, "XWqB", "separate")
    assert (ml.in_features, ml.out_features) == (64, 8) and set(ml.state_dict()) == {"w_element"}
    with pytest.raises(ValueError):
        MinifloatLinearPTQ(None, torch.zeros(8), None, None, None, "XWqBq", w_element=codes, w_tensor_meta=mtm,
                           b_element=codes[0], b_tensor_meta=mtm)


def test_kernel_manager_flag():
    from mase_hip.manager import KernelManager

    KernelManager.enable_autotune()
    assert KernelManager.autotune_is_enabled()
    KernelManager.disable_autotune()
    assert not KernelManager.autotune_is_enabled()
