"""GPU parity tests for minifloat_linear / minifloat_matmul / MinifloatLinearPTQ.  The fused
backend sends weights in the formats the MXFP GEMM decodes through that GEMM (codes narrowed to
one byte, unit block scales); the rest goes compose -> dense GEMM.  Tolerance: relative
Frobenius error <= 1e-3 against dequantize-then-matmul in fp64 on the checker's values, rounded
once to the output dtype; fp32 outputs of the MFMA route are held to 1e-5."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
REL_FRO_TOL = 1e-3


def rel_fro(y, y_ref):
    y, y_ref = y.double().cpu(), y_ref.double().cpu()
    return ((y - y_ref).norm() / y_ref.norm()).item()


@pytest.fixture(scope="module")
def mf():
    import mase_hip.minifloat.functional as F
    from mase_hip import _lib
    from mase_hip.minifloat import meta
    from mase_hip.minifloat.layers import MinifloatLinearPTQ

    _lib.load()

    class NS:
        pass

    ns = NS()
    ns.F, ns.meta, ns.Layer = F, meta, MinifloatLinearPTQ
    return ns


def checker_linear(x, x_meta, w_codes, w_meta, bias):
    """fp64 x_dq @ w_dq^T + b from the CPU checker's quantisation."""
    x = x.cpu()
    x_dq = x if x_meta is None else oracle.qdq_minifloat(x, x_meta.exp_bits, x_meta.frac_bits, x_meta.is_finite,
                                                          x_meta.round_mode)
    w_dq = oracle.compose_minifloat(w_codes.cpu(), w_meta.exp_bits, w_meta.frac_bits, w_meta.is_finite, torch.float32)
    y = x_dq.double().reshape(-1, x.shape[-1]) @ w_dq.double().t()
    if bias is not None:
        y = y + bias.double().cpu()
    return y.view(*x.shape[:-1], -1)


W_TAGS = ["FP8_E4M3_fn", "FP8_E5M2_fn", "FP6_E2M3_fn", "FP6_E3M2_fn", "FP4_E2M1_fn"]


@pytest.mark.parametrize("w_tag", W_TAGS)
@pytest.mark.parametrize("MNK", [(96, 256, 512), (8, 128, 256), (200, 136, 96)])
def test_minifloat_linear_fused_vs_checker(mf, w_tag, MNK):
    """XqWqB through the MFMA route: every weight format the GEMM decodes, shapes that take the
    few-row, the 256x256-tile and the bounds-checked kernels."""
    M, N, K = MNK
    g = torch.Generator().manual_seed(3)
    x = (2 * torch.randn(M, K, generator=g)).to(torch.bfloat16)
    w = (0.5 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    x_meta, w_meta = mf.meta.FP8_E4M3_fn, getattr(mf.meta, w_tag)
    w_codes, w_tm = mf.F.extract_minifloat_component(w.to(DEV), w_meta)
    assert torch.equal(w_codes.cpu(), oracle.extract_minifloat(w, w_meta.exp_bits, w_meta.frac_bits))
    y = mf.F.minifloat_linear(x=x.to(DEV), x_meta=x_meta, w=None, w_element=w_codes, w_tensor_meta=w_tm,
                              b=b.to(DEV), b_element=None, b_tensor_meta=None, layer_type="XqWqB", backend="fused")
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    assert rel_fro(y, checker_linear(x, x_meta, w_codes, w_meta, b).to(y.dtype)) <= REL_FRO_TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layer_type", ["XqWqB", "XWqB", "XqWB", "XWB", "XqWqBq"])
@pytest.mark.parametrize("bias", [True, False])
def test_minifloat_layer_fused_matches_separate(mf, dtype, layer_type, bias):
    M, N, K = 192, 256, 512
    g = torch.Generator().manual_seed(7)
    x = (torch.randn(3, M // 3, K, generator=g) * 3).to(dtype).to(DEV)
    lin = torch.nn.Linear(K, N, bias=bias, dtype=dtype, device=DEV)
    with torch.no_grad():
        lin.weight.mul_(16)  # minifloat has no block scale: bring the weights into FP6's range
    x_meta = mf.meta.FP8_E4M3_fn if layer_type.startswith("Xq") else None
    w_meta = mf.meta.FP6_E3M2_fn if "Wq" in layer_type else None
    b_meta = mf.meta.FP8_E4M3_fn if layer_type.endswith("Bq") and bias else None
    fused = mf.Layer.from_linear(lin, x_meta, w_meta, b_meta, layer_type, "fused")
    separate = mf.Layer.from_linear(lin, x_meta, w_meta, b_meta, layer_type, "separate")
    y_f, y_s = fused(x), separate(x)
    assert y_f.shape == (3, M // 3, N) and y_f.dtype == dtype
    # a dense fp32 x is not rounded to bf16: that case stays on the dense route and is bit-equal
    mfma_route = "Wq" in layer_type and (dtype == torch.bfloat16 or layer_type.startswith("Xq"))
    if not mfma_route:
        assert torch.equal(y_f, y_s)
    assert rel_fro(y_f, y_s) <= (REL_FRO_TOL if dtype == torch.bfloat16 else 1e-5)


def test_minifloat_linear_wide_formats_use_dense_route(mf):
    """Weight formats wider than a byte, or with inf/NaN codes, are composed and multiplied by
    the dense GEMM: bit-equal to the separate backend."""
    M, N, K = 64, 128, 256
    g = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16).to(DEV)
    for w_meta in (mf.meta.MinifloatMeta(5, 6, True, "rn"), mf.meta.MinifloatMeta(4, 3, False, "rn")):
        w_codes, w_tm = mf.F.extract_minifloat_component(w, w_meta)
        assert not mf.F.gemm_weight_eligible(w_tm)
        kw = dict(x=x, x_meta=mf.meta.FP8_E4M3_fn, w=None, w_element=w_codes, w_tensor_meta=w_tm, b=None,
                  b_element=None, b_tensor_meta=None, layer_type="XqWqB")
        y_f = mf.F.minifloat_linear(**kw, backend="fused")
        y_s = mf.F.minifloat_linear(**kw, backend="separate")
        assert torch.equal(y_f, y_s)
        assert rel_fro(y_f, checker_linear(x, mf.meta.FP8_E4M3_fn, w_codes, w_meta, None).to(y_f.dtype)) <= REL_FRO_TOL


def test_minifloat_linear_ignores_code_bits_above_the_format(mf):
    """The decode reads only the low 1+E+M bits of a code (fake.py:97-123); so does the
    narrowing to one byte."""
    M, N, K = 32, 64, 128
    g = torch.Generator().manual_seed(9)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randn(N, K, generator=g).to(torch.bfloat16).to(DEV)
    w_meta = mf.meta.FP6_E2M3_fn
    w_codes, w_tm = mf.F.extract_minifloat_component(w, w_meta)
    noisy = (w_codes.to(torch.int32) | (torch.randint(0, 4, (N, K), generator=g).to(DEV) << 6)).to(torch.uint16)
    kw = dict(x=x, x_meta=None, w=None, w_tensor_meta=w_tm, b=None, b_element=None, b_tensor_meta=None,
              layer_type="XWqB", backend="fused")
    assert torch.equal(mf.F.minifloat_linear(w_element=w_codes, **kw), mf.F.minifloat_linear(w_element=noisy, **kw))


def test_minifloat_layer_large_and_few_rows(mf):
    """One layer applied to a large batch (persistent large-tile kernel) and to a few rows
    (weight-streaming kernel), checked against fp64 on the checker's values."""
    N, K = 3072, 256
    g = torch.Generator().manual_seed(13)
    w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    lin = torch.nn.Linear(K, N, bias=True, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    x_meta, w_meta = mf.meta.FP8_E4M3_fn, mf.meta.FP8_E4M3_fn
    layer = mf.Layer.from_linear(lin, x_meta, w_meta, None, "XqWqB", "fused")
    for M in (2048, 16):
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        y = layer(x.to(DEV))
        assert rel_fro(y, checker_linear(x, x_meta, layer.w_element, w_meta, b).to(y.dtype)) <= REL_FRO_TOL


def test_minifloat_layer_follows_weight_updates(mf):
    """The one-byte copy of the codes kept by the layer is rebuilt when the codes change."""
    N, K = 64, 128
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16, device=DEV)
    layer = mf.Layer.from_linear(lin, None, mf.meta.FP8_E4M3_fn, None, "XWqB", "fused")
    x = torch.randn(16, K, dtype=torch.bfloat16, device=DEV)
    y0 = layer(x)
    assert "_narrowed" not in layer.state_dict() and set(layer.state_dict()) == {"w_element"}
    with torch.no_grad():
        layer.w_element.copy_((layer.w_element.to(torch.int32) ^ 0x80).to(torch.uint16))  # flip every sign
    y1 = layer(x)
    assert torch.equal(y1, -y0)
    cpu_layer = layer.to("cpu")
    assert cpu_layer._narrowed is None


@pytest.mark.parametrize("func_type", ["XW", "XqW", "XWq", "XqWq"])
@pytest.mark.parametrize("backend", ["separate", "fused"])
def test_minifloat_matmul(mf, func_type, backend):
    g = torch.Generator().manual_seed(17)
    a = torch.randn(4, 48, 96, generator=g).to(torch.bfloat16)
    b = torch.randn(96, 80, generator=g).to(torch.bfloat16)
    am, bm = mf.meta.FP8_E4M3_fn, mf.meta.FP6_E3M2_fn
    y = mf.F.minifloat_matmul(a.to(DEV), b.to(DEV), am if "Xq" in func_type else None,
                              bm if "Wq" in func_type else None, func_type, backend)
    a_dq = oracle.qdq_minifloat(a, am.exp_bits, am.frac_bits) if "Xq" in func_type else a
    b_dq = oracle.qdq_minifloat(b, bm.exp_bits, bm.frac_bits) if "Wq" in func_type else b
    assert y.shape == (4, 48, 80) and y.dtype == torch.bfloat16
    assert rel_fro(y, (a_dq.double() @ b_dq.double()).to(y.dtype)) <= REL_FRO_TOL


@pytest.mark.parametrize("w_tag", W_TAGS)
@pytest.mark.parametrize("a_shape,b_shape,dtype", [
    ((4, 48, 96), (96, 80), torch.bfloat16),             # matrix `other`: one GEMM over all rows
    ((3, 40, 128), (3, 128, 64), torch.bfloat16),        # one batched launch
    ((2, 1, 24, 64), (1, 5, 64, 32), torch.bfloat16),    # broadcast batch axes
    ((24, 64), (5, 64, 32), torch.bfloat16),             # matrix `input` shared by every product
    ((2, 50, 128), (2, 128, 72), torch.float32),         # fp32 in and out
    ((4, 48), (48, 40), torch.bfloat16),                 # contraction axis not a multiple of 32: dense route
])
def test_minifloat_matmul_fused_routes(mf, w_tag, a_shape, b_shape, dtype):
    """backend="fused" with `other` in every one-byte format the GEMM decodes: the codes go through the MFMA GEMM with unit
    block scales, whatever the batch axes; against fp64 on the checker's quantised values and against backend="separate"."""
    g = torch.Generator().manual_seed(sum(a_shape) + len(w_tag))
    a = torch.randn(*a_shape, generator=g).to(dtype)
    b = (2.0 * torch.randn(*b_shape, generator=g)).to(dtype)
    am, bm = mf.meta.FP8_E4M3_fn, getattr(mf.meta, w_tag)
    b_dq = oracle.qdq_minifloat(b, bm.exp_bits, bm.frac_bits)
    for func_type in ("XqWq", "XWq"):
        if func_type == "XWq" and dtype == torch.float32:
            continue                                     # a dense fp32 input is not rounded to bf16: dense route, covered above
        y = mf.F.minifloat_matmul(a.to(DEV), b.to(DEV), am if func_type == "XqWq" else None, bm, func_type, "fused")
        a_dq = oracle.qdq_minifloat(a, am.exp_bits, am.frac_bits) if func_type == "XqWq" else a
        y_chk = torch.matmul(a_dq.double(), b_dq.double()).to(dtype)
        assert y.shape == y_chk.shape and y.dtype == dtype
        tol = REL_FRO_TOL if dtype == torch.bfloat16 else 1e-5
        assert rel_fro(y, y_chk) <= tol, func_type
        y_sep = mf.F.minifloat_matmul(a.to(DEV), b.to(DEV), am if func_type == "XqWq" else None, bm, func_type, "separate")
        assert rel_fro(y, y_sep) <= tol, func_type


def test_minifloat_matmul_fused_takes_the_gemm(mf, monkeypatch):
    """The fused backend really leaves `other` in code form: torch.matmul is not called on the GEMM route."""
    g = torch.Generator().manual_seed(5)
    a = torch.randn(3, 40, 128, generator=g).to(torch.bfloat16).to(DEV)
    b = torch.randn(3, 128, 64, generator=g).to(torch.bfloat16).to(DEV)

    def boom(*args, **kwargs):
        raise AssertionError("dense matmul called")

    monkeypatch.setattr(torch, "matmul", boom)
    y = mf.F.minifloat_matmul(a, b, mf.meta.FP8_E4M3_fn, mf.meta.FP8_E4M3_fn, "XqWq", "fused")
    assert y.shape == (3, 40, 64)


# ------------------------------------------------------------------ the block-scaled route
SCALED_TAGS = ["FP8_E4M3_fn", "FP6_E2M3_fn", "FP6_E3M2_fn", "FP4_E2M1_fn"]


def _awkward_activations(rows, K, g):
    """bf16 values over the whole range of the formats: saturating ones (the top E4M3 code, which the operand re-encodes),
    subnormals of the target formats, zeros of both signs, bf16 subnormals, inf and NaN."""
    x = torch.randn(rows, K, generator=g) * torch.exp2(torch.randint(-12, 10, (rows, K), generator=g).float())
    x = x.to(torch.bfloat16)
    flat = x.view(-1)
    specials = torch.tensor([float("inf"), float("-inf"), float("nan"), 0.0, -0.0, 480.0, -480.0, 448.0, 1e-40, -1e-40, 7.5, 28.0, 6.0],
                            dtype=torch.float32).to(torch.bfloat16)
    idx = torch.randperm(flat.numel(), generator=g)[: 16 * specials.numel()]
    flat[idx] = specials.repeat(16)
    return x


@pytest.mark.parametrize("tag", SCALED_TAGS)
@pytest.mark.parametrize("rows,K", [(70, 512), (256, 128), (1, 1280)])
def test_minifloat_scaled_operand_is_the_extracted_codes(mf, tag, rows, K):
    """The one-pass operand of x holds, bit for bit, what the separate steps give: extract_minifloat (checked against the CPU
    checker), one byte per code, unit scales, the MXFP operand kernel."""
    from mase_hip.mxfp import kernels as K_

    meta = getattr(mf.meta, tag)
    g = torch.Generator().manual_seed(rows + K)
    x = _awkward_activations(rows, K, g)
    codes16, tm = mf.F.extract_minifloat_component(x.to(DEV), meta)
    assert torch.equal(codes16.cpu(), oracle.extract_minifloat(x, meta.exp_bits, meta.frac_bits))
    by_steps = mf.F.linear.scaled_weight_operand(codes16, tm)
    one_pass = K_.scaled_operand_from_dense_minifloat(x.to(DEV), meta.exp_bits, meta.frac_bits)
    assert torch.equal(one_pass.codes[:rows], by_steps.codes[:rows])
    assert torch.equal(one_pass.scales[:, :rows], by_steps.scales[:, :rows])
    unit = one_pass.scales[:, :rows].view(torch.uint8)
    assert bool(((unit == 127) | (unit == 128)).all())          # 128: a block re-encoded for the top E4M3 code
    assert bool((unit == 128).any()) == (tag == "FP8_E4M3_fn")


@pytest.mark.parametrize("tag", SCALED_TAGS)
def test_minifloat_scaled_operand_every_bf16_pattern(mf, tag):
    """All 65536 bfloat16 bit patterns, in order (so that most wavefronts take the table look-up and the ones that hold inf
    and NaN the per-element routine): the same codes as the separate steps."""
    from mase_hip.mxfp import kernels as K_

    meta = getattr(mf.meta, tag)
    x = torch.arange(65536, dtype=torch.int32).to(torch.uint16).view(torch.bfloat16).view(512, 128)
    codes16, tm = mf.F.extract_minifloat_component(x.to(DEV), meta)
    assert torch.equal(codes16.cpu(), oracle.extract_minifloat(x, meta.exp_bits, meta.frac_bits))
    by_steps = mf.F.linear.scaled_weight_operand(codes16, tm)
    one_pass = K_.scaled_operand_from_dense_minifloat(x.to(DEV), meta.exp_bits, meta.frac_bits)
    assert torch.equal(one_pass.codes[:512], by_steps.codes[:512])
    assert torch.equal(one_pass.scales[:, :512], by_steps.scales[:, :512])


@pytest.mark.parametrize("x_tag,w_tag", [("FP8_E4M3_fn", "FP8_E4M3_fn"), ("FP8_E4M3_fn", "FP4_E2M1_fn"), ("FP6_E3M2_fn", "FP6_E2M3_fn"),
                                         ("FP4_E2M1_fn", "FP8_E4M3_fn")])
@pytest.mark.parametrize("MNK", [(300, 264, 768), (16, 512, 512), (1030, 256, 1024)])
def test_minifloat_linear_scaled_vs_checker(mf, x_tag, w_tag, MNK):
    """XqWqB on the block-scaled matrix instruction (forced) against fp64 on the checker's values and against the bf16 route;
    the activations saturate here and there, so E4M3 blocks of x get re-encoded."""
    M, N, K = MNK
    g = torch.Generator().manual_seed(M + N)
    x = (3 * torch.randn(M, K, generator=g)).to(torch.bfloat16)
    x.view(-1)[torch.randperm(M * K, generator=g)[: M * K // 64]] = 1000.0
    w = (0.5 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    b = torch.randn(N, generator=g).to(torch.bfloat16)
    x_meta, w_meta = getattr(mf.meta, x_tag), getattr(mf.meta, w_tag)
    w_codes, w_tm = mf.F.extract_minifloat_component(w.to(DEV), w_meta)
    kw = dict(x=x.to(DEV), x_meta=x_meta, w=None, w_element=w_codes, w_tensor_meta=w_tm, b=b.to(DEV), b_element=None,
              b_tensor_meta=None, layer_type="XqWqB")
    y = mf.F.minifloat_linear(**kw, backend="fused_scaled")
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    assert rel_fro(y, checker_linear(x, x_meta, w_codes, w_meta, b).to(y.dtype)) <= REL_FRO_TOL
    assert rel_fro(y, mf.F.minifloat_linear(**kw, backend="fused_bf16")) <= REL_FRO_TOL
    assert rel_fro(y, mf.F.minifloat_linear(**kw, backend="separate")) <= REL_FRO_TOL


def test_minifloat_layer_routes(mf, monkeypatch):
    """Which GEMM a layer's call takes: the block-scaled one for quantised bf16 activations in its formats (every row
    count: the layer keeps the weight operand), the bf16 one otherwise; the weight operand is built once and follows the codes."""
    from mase_hip.mxfp import kernels as K_

    calls = {"scaled": 0, "bf16": 0, "prepare": 0}
    real_scaled, real_bf16, real_prepare = K_.mxfp_gemm_scaled, K_.mxfp_gemm, K_.scaled_operand_from_mxfp

    def count(name, fn):
        def wrapped(*a, **k):
            calls[name] += 1
            return fn(*a, **k)
        return wrapped

    monkeypatch.setattr(K_, "mxfp_gemm_scaled", count("scaled", real_scaled))
    monkeypatch.setattr(K_, "linear_scaled", count("scaled", K_.linear_scaled))     # (operand of x and the same GEMM behind one call)
    monkeypatch.setattr(K_, "mxfp_gemm", count("bf16", real_bf16))
    monkeypatch.setattr(K_, "scaled_operand_from_mxfp", count("prepare", real_prepare))
    N, K = 256, 512
    lin = torch.nn.Linear(K, N, bias=True, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        lin.weight.mul_(16)  # minifloat has no block scale: bring the weights into FP6's range
    g = torch.Generator().manual_seed(21)
    layer = mf.Layer.from_linear(lin, mf.meta.FP8_E4M3_fn, mf.meta.FP6_E3M2_fn, None, "XqWqB", "fused")
    separate = mf.Layer.from_linear(lin, mf.meta.FP8_E4M3_fn, mf.meta.FP6_E3M2_fn, None, "XqWqB", "separate")
    for rows in (64, 16, 24, 256):
        before = dict(calls)
        x = torch.randn(rows, K, generator=g).to(torch.bfloat16).to(DEV)
        y = layer(x)
        assert (calls["scaled"] - before["scaled"], calls["bf16"] - before["bf16"]) == (1, 0), rows
        assert rel_fro(y, separate(x)) <= REL_FRO_TOL
    assert calls["prepare"] == 1
    # ... also with a K beyond what the weight-streaming kernels take in one piece
    lin_long = torch.nn.Linear(4608, N, bias=False, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        lin_long.weight.mul_(16)
    long_k = mf.Layer.from_linear(lin_long, mf.meta.FP8_E4M3_fn, mf.meta.FP6_E3M2_fn, None, "XqWqB", "fused")
    long_sep = mf.Layer.from_linear(lin_long, mf.meta.FP8_E4M3_fn, mf.meta.FP6_E3M2_fn, None, "XqWqB", "separate")
    for rows in (16, 24, 64):
        before = dict(calls)
        x = torch.randn(rows, 4608, generator=g).to(torch.bfloat16).to(DEV)
        y = long_k(x)
        assert (calls["scaled"] - before["scaled"], calls["bf16"] - before["bf16"]) == (1, 0), rows
        assert rel_fro(y, long_sep(x)) <= REL_FRO_TOL
    calls["prepare"] = 1
    x = torch.randn(128, K, generator=g).to(torch.bfloat16).to(DEV)
    y_before = layer(x)
    with torch.no_grad():
        for l in (layer, separate):
            l.w_element.copy_((l.w_element.to(torch.int32) ^ 0x20).to(torch.uint16))   # flip every sign (E3M2 is 6 bits wide)
    y_after = layer(x)
    assert calls["prepare"] == 2
    assert rel_fro(y_after, separate(x)) <= REL_FRO_TOL and rel_fro(y_after, y_before) > 0.5
    # formats and dtypes the instruction does not take stay on the bf16 route; forcing it says why not
    e5m2 = mf.Layer.from_linear(lin, mf.meta.FP8_E4M3_fn, mf.meta.FP8_E5M2_fn, None, "XqWqB", "fused")
    before = dict(calls)
    e5m2(x)
    assert (calls["scaled"], calls["bf16"]) == (before["scaled"], before["bf16"] + 1)
    forced = mf.Layer.from_linear(lin, mf.meta.FP8_E4M3_fn, mf.meta.FP8_E5M2_fn, None, "XqWqB", "fused_scaled")
    with pytest.raises(NotImplementedError):
        forced(x)
    rd = mf.meta.MinifloatMeta(4, 3, True, "rd")
    before = dict(calls)
    mf.Layer.from_linear(lin, rd, mf.meta.FP6_E3M2_fn, None, "XqWqB", "fused")(x)
    assert calls["scaled"] == before["scaled"]


def test_minifloat_layer_repeat_calls_skip_the_checks_and_notice_changes(mf, monkeypatch):
    """As for the MXFP layer: a call like the previous one on the block-scaled route goes straight to the two kernels,
    with the same bits; other shapes, formats and codes go through the checks again."""
    import mase_hip.minifloat.layers as layers_mod

    calls = [0]
    real = layers_mod.MinifloatF.minifloat_linear

    def counted(*a, **k):
        calls[0] += 1
        return real(*a, **k)

    monkeypatch.setattr(layers_mod.MinifloatF, "minifloat_linear", counted)
    lin = torch.nn.Linear(512, 264, bias=True, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        lin.weight.mul_(16)
    g = torch.Generator().manual_seed(31)
    layer = mf.Layer.from_linear(lin, mf.meta.FP8_E4M3_fn, mf.meta.FP6_E3M2_fn, None, "XqWqB", "fused")
    x = (3 * torch.randn(2, 8, 512, generator=g)).to(torch.bfloat16).to(DEV)
    y0, y1 = layer(x), layer(x)
    assert calls[0] == 1 and torch.equal(y0, y1) and y1.shape == (2, 8, 264)
    layer(x[:1])
    layer(x)
    assert calls[0] == 3
    layer.x_minifloat_meta = mf.meta.FP4_E2M1_fn
    y2 = layer(x)
    assert calls[0] == 4 and not torch.equal(y2, y0)
    assert torch.equal(layer(x), y2) and calls[0] == 4
    assert torch.equal(y2, mf.Layer.from_linear(lin, mf.meta.FP4_E2M1_fn, mf.meta.FP6_E3M2_fn, None, "XqWqB", "fused")(x))
    calls[0] = 4                                         # (the line above counted one for the other layer)
    with torch.no_grad():
        layer.w_element.copy_((layer.w_element.to(torch.int32) ^ 0x20).to(torch.uint16))
    y3 = layer(x)
    assert calls[0] == 5 and not torch.equal(y3, y2)
    y4 = layer(x[:, :0])
    assert y4.shape == (2, 0, 264) and layer._fast_sig is None


@pytest.mark.filterwarnings("ignore:mase_hip. an operand is not 16-byte aligned")
@pytest.mark.parametrize("backend", ["fused", "fused_bf16", "fused_scaled"])
def test_minifloat_linear_input_layouts(mf, backend):
    """One vector, no rows, strided and misaligned views, many leading axes through the layer, against float64 on the
    checker's values."""
    lin = torch.nn.Linear(512, 136, bias=True, dtype=torch.bfloat16, device=DEV)
    with torch.no_grad():
        lin.weight.mul_(16)
    x_meta, w_meta = mf.meta.FP8_E4M3_fn, mf.meta.FP6_E2M3_fn
    layer = mf.Layer.from_linear(lin, x_meta, w_meta, None, "XqWqB", backend)
    g = torch.Generator().manual_seed(14)
    base = (2 * torch.randn(6, 70, 1024, generator=g)).to(torch.bfloat16).to(DEV)
    cases = {
        "vector": base[0, 0, :512],
        "no rows": base[:, :0, :512],
        "row-strided view": base[..., :512],
        "element-strided view": base[..., ::2],
        "five axes": base[..., :512].reshape(2, 3, 7, 10, 512),
        "offset by one element": base.view(-1)[1:1 + 9 * 512].view(9, 512),
    }
    for name, x in cases.items():
        y = layer(x)
        assert y.shape == (*x.shape[:-1], 136) and y.dtype == torch.bfloat16, name
        if x.numel():
            y_ref = checker_linear(x, x_meta, layer.w_element, w_meta, lin.bias.detach()).to(y.dtype)
            assert rel_fro(y, y_ref) <= REL_FRO_TOL, name
            assert rel_fro(layer(x), y_ref) <= REL_FRO_TOL, name
