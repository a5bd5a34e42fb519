"""GPU tests for the bit-packed storage form of element codes and the exported form of a
quantised layer: pack / unpack against the numpy bit-stream checker (bit-exact), and a layer
exported, saved, loaded with ``weights_only=True`` and rebuilt gives the same outputs."""
import io

import numpy as np
import pytest
import torch

from oracle import packing as chk

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def mx():
    import mase_hip.mxfp.functional as F
    from mase_hip import _lib
    from mase_hip.mxfp import meta, packing
    from mase_hip.mxfp.layers import MXFPLinearPTQ

    _lib.load()

    class NS:
        pass

    ns = NS()
    ns.F, ns.meta, ns.packing, ns.Layer = F, meta, packing, MXFPLinearPTQ
    return ns


@pytest.mark.parametrize("tag,bits", [("OCP_MXFP4_E2M1", 4), ("OCP_MXFP6_E2M3", 6), ("OCP_MXFP6_E3M2", 6)])
@pytest.mark.parametrize("n", [32, 64 * 5, 32 * 1025, 1 << 20])
def test_pack_unpack_vs_checker(mx, tag, bits, n):
    fmt = getattr(mx.meta, tag)
    assert mx.packing.code_bits(fmt) == bits
    rng = np.random.default_rng(n + bits)
    codes = rng.integers(0, 1 << bits, size=n, dtype=np.uint8)
    el = torch.from_numpy(codes).to(DEV).view(-1, 32)
    packed = mx.packing.pack_elements(el, fmt)
    assert packed.dtype == torch.uint8 and packed.numel() == n * bits // 8 == mx.packing.packed_nbytes(n, fmt)
    assert np.array_equal(packed.cpu().numpy(), chk.pack_codes(codes, bits))
    back = mx.packing.unpack_elements(packed, fmt, n)
    assert back.shape == (n // 32, 32) and np.array_equal(back.cpu().numpy().reshape(-1), codes)
    # the checker's unpack of the kernel's bytes, and the kernel's unpack of the checker's bytes
    assert np.array_equal(chk.unpack_codes(packed.cpu().numpy(), bits, n), codes)
    from_chk = mx.packing.unpack_elements(torch.from_numpy(chk.pack_codes(codes, bits)).to(DEV), fmt, n)
    assert np.array_equal(from_chk.cpu().numpy().reshape(-1), codes)


def test_pack_every_code_value_at_every_position(mx):
    for tag, bits in (("OCP_MXFP4_E2M1", 4), ("OCP_MXFP6_E3M2", 6)):
        fmt = getattr(mx.meta, tag)
        base = np.tile(np.arange(1 << bits, dtype=np.uint8), 16)
        for shift in range(16):
            codes = np.roll(base, shift)
            packed = mx.packing.pack_elements(torch.from_numpy(codes).to(DEV), fmt)
            assert np.array_equal(packed.cpu().numpy(), chk.pack_codes(codes, bits))
            assert np.array_equal(mx.packing.unpack_elements(packed, fmt, codes.size).cpu().numpy().reshape(-1), codes)


def test_pack_drops_bits_above_the_code_width_and_keeps_8_bit_formats(mx):
    fmt4 = mx.meta.OCP_MXFP4_E2M1
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).to(DEV)
    back = mx.packing.unpack_elements(mx.packing.pack_elements(codes, fmt4), fmt4, 256)
    assert torch.equal(back.reshape(-1), codes & 15)
    fmt8 = mx.meta.MXFP8_E4M3_fn
    p8 = mx.packing.pack_elements(codes.view(8, 32), fmt8)
    assert torch.equal(p8, codes) and torch.equal(mx.packing.unpack_elements(p8, fmt8, 256), codes.view(8, 32))


def test_pack_argument_errors(mx):
    from mase_hip import _lib

    lib = _lib.load()
    a = torch.zeros(64, dtype=torch.uint8, device=DEV)
    b = torch.zeros(64, dtype=torch.uint8, device=DEV)
    s = _lib.stream_ptr(a.device)
    assert lib.mase_hip_pack_codes(a.data_ptr(), b.data_ptr(), 64, 5, s) == -1
    assert lib.mase_hip_pack_codes(a.data_ptr(), b.data_ptr(), 40, 4, s) == -1
    assert lib.mase_hip_pack_codes(None, b.data_ptr(), 64, 4, s) == -1
    assert lib.mase_hip_pack_codes(a.data_ptr() + 4, b.data_ptr(), 32, 4, s) == -1
    assert lib.mase_hip_unpack_codes(a.data_ptr(), b.data_ptr(), 0, 6, s) == 0


@pytest.mark.parametrize("w_tag", ["OCP_MXFP4_E2M1", "OCP_MXFP6_E3M2", "MXFP8_E4M3_fn"])
@pytest.mark.parametrize("layer_type,bias", [("XqWqB", True), ("XWqB", False), ("XqWqBq", True)])
def test_layer_export_save_load_rebuild(mx, w_tag, layer_type, bias):
    K, N = 256, 192
    lin = torch.nn.Linear(K, N, bias=bias, dtype=torch.bfloat16, device=DEV)
    x_meta = mx.meta.MXFP8_E4M3_fn if layer_type.startswith("Xq") else None
    w_meta = getattr(mx.meta, w_tag)
    b_meta = mx.meta.MXFP8_E4M3_fn if layer_type.endswith("Bq") else None
    layer = mx.Layer.from_linear(lin, x_meta, w_meta, b_meta, layer_type, "fused")
    blob = io.BytesIO()
    torch.save(layer.export_quantized(), blob)
    per_code = mx.packing.code_bits(w_meta) / 8
    assert layer.export_quantized()["w"]["elements_packed"].numel() == int(N * K * per_code)
    blob.seek(0)
    d = torch.load(blob, weights_only=True, map_location="cpu")  # tensors, strings, numbers only
    rebuilt = mx.Layer.from_exported(d, backend="fused", device=DEV)
    assert rebuilt.layer_type == layer_type and rebuilt.w_tensor_meta == layer.w_tensor_meta
    assert torch.equal(rebuilt.w_scales, layer.w_scales) and torch.equal(rebuilt.w_elements, layer.w_elements)
    x = torch.randn(40, K, dtype=torch.bfloat16, device=DEV)
    assert torch.equal(rebuilt(x), layer(x))
