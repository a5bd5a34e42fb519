"""GPU MXFP casts and the MXFP GEMM: tensor-level wrappers over the C ABI.

``extract_mxfp_components`` / ``compose_mxfp_tensor`` have the names and signatures of the
reference's Triton wrappers (src/mase_triton/mxfp/kernels/cast.py:126-160, 237-272); results are
bit-identical to the reference's PyTorch "fake" implementation (src/mase_triton/mxfp/fake.py).
``quantize_dequantize``, the ``*_strided`` casts and ``mxfp_gemm`` have no counterpart there
(fused paths; blocks along a non-last axis without the permuted copy).
"""
from __future__ import annotations

import torch
from torch import Tensor

from .. import _lib
from .meta import MXFPMeta


def _fmt(meta: MXFPMeta):
    assert meta.scale_exp_bits == 8
    return meta.element_exp_bits, meta.element_frac_bits, int(meta.element_is_finite)


def extract_mxfp_components(x: Tensor, mxfp_meta: MXFPMeta) -> tuple[Tensor, Tensor]:
    """1-D float tensor -> (scales uint8 [n/B, 1], elements uint8 [n/B, B])."""
    assert x.ndim == 1
    _lib.require_gpu(x, "input tensor")
    x = _lib.dense(_lib.as_float_input(x))
    n, B = x.numel(), mxfp_meta.block_size
    assert n % B == 0
    scales = torch.empty((n // B, 1), dtype=torch.uint8, device=x.device)
    elements = torch.empty((n // B, B), dtype=torch.uint8, device=x.device)
    with _lib.on_device(x.device):
        _lib.check(_lib.load().mase_hip_extract_mxfp(
            x.data_ptr(), _lib.dtype_code(x.dtype), scales.data_ptr(), elements.data_ptr(), n, B,
            *_fmt(mxfp_meta), _lib.round_code(mxfp_meta.round_mode), _lib.stream_ptr(x.device)))
    return scales, elements


def compose_mxfp_tensor(scales: Tensor, elements: Tensor, mxfp_meta: MXFPMeta, output_dtype: torch.dtype) -> Tensor:
    """(scales, elements) -> flat tensor [n] of ``output_dtype``."""
    assert scales.dtype == torch.uint8
    assert elements.dtype == torch.uint8
    _lib.require_gpu(elements, "elements")
    _lib.require_gpu(scales, "scales")
    scales, elements = _lib.dense(scales), _lib.dense(elements)
    n, B = elements.numel(), mxfp_meta.block_size
    assert n % B == 0 and scales.numel() == n // B
    out = torch.empty((n,), dtype=output_dtype, device=elements.device)
    with _lib.on_device(elements.device):
        _lib.check(_lib.load().mase_hip_compose_mxfp(
            scales.data_ptr(), elements.data_ptr(), out.data_ptr(), _lib.dtype_code(output_dtype), n, B,
            *_fmt(mxfp_meta), _lib.stream_ptr(elements.device)))
    return out


def quantize_dequantize(x: Tensor, mxfp_meta: MXFPMeta, output_dtype: torch.dtype) -> Tensor:
    """compose(extract(x)) for a flat tensor in a single pass; nothing is materialised."""
    assert x.ndim == 1
    _lib.require_gpu(x, "input tensor")
    x = _lib.dense(_lib.as_float_input(x))
    n, B = x.numel(), mxfp_meta.block_size
    assert n % B == 0
    out = torch.empty((n,), dtype=output_dtype, device=x.device)
    with _lib.on_device(x.device):
        _lib.check(_lib.load().mase_hip_qdq_mxfp(
            x.data_ptr(), _lib.dtype_code(x.dtype), out.data_ptr(), _lib.dtype_code(output_dtype), n, B,
            *_fmt(mxfp_meta), _lib.round_code(mxfp_meta.round_mode), _lib.stream_ptr(x.device)))
    return out


def strided_blocks_supported(shape: tuple[int, ...], block_dim: int, mxfp_meta: MXFPMeta) -> bool:
    """Can blocks along ``block_dim`` be taken in place (no permuted copy)?  The axis must not be
    the last one (those blocks are contiguous already) and must hold whole blocks of 32."""
    ndim = len(shape)
    block_dim %= ndim
    return block_dim != ndim - 1 and mxfp_meta.block_size == 32 and shape[block_dim] % 32 == 0


def _strided_extents(shape, block_dim: int) -> tuple[int, int, int]:
    block_dim %= len(shape)
    outer = inner = 1
    for d in shape[:block_dim]:
        outer *= d
    for d in shape[block_dim + 1:]:
        inner *= d
    return outer, shape[block_dim], inner


def extract_mxfp_components_strided(x: Tensor, block_dim: int, mxfp_meta: MXFPMeta) -> tuple[Tensor, Tensor]:
    """N-D float tensor, blocks along ``block_dim`` -> (scales uint8 [n/32, 1], elements uint8
    [n/32, 32]) in the order of the tensor with ``block_dim`` rotated last; no permuted copy."""
    assert strided_blocks_supported(tuple(x.shape), block_dim, mxfp_meta)
    _lib.require_gpu(x, "input tensor")
    x = _lib.dense(_lib.as_float_input(x))
    outer, k_len, inner = _strided_extents(x.shape, block_dim)
    n = x.numel()
    scales = torch.empty((n // 32, 1), dtype=torch.uint8, device=x.device)
    elements = torch.empty((n // 32, 32), dtype=torch.uint8, device=x.device)
    with _lib.on_device(x.device):
        _lib.check(_lib.load().mase_hip_extract_mxfp_strided(
            x.data_ptr(), _lib.dtype_code(x.dtype), scales.data_ptr(), elements.data_ptr(), outer, k_len, inner, 32,
            *_fmt(mxfp_meta), _lib.round_code(mxfp_meta.round_mode), _lib.stream_ptr(x.device)))
    return scales, elements


def quantize_dequantize_strided(x: Tensor, block_dim: int, mxfp_meta: MXFPMeta, output_dtype: torch.dtype) -> Tensor:
    """compose(extract(x)) with blocks along ``block_dim`` in one pass; the result is contiguous
    in x's own shape."""
    assert strided_blocks_supported(tuple(x.shape), block_dim, mxfp_meta)
    _lib.require_gpu(x, "input tensor")
    x = _lib.dense(_lib.as_float_input(x))
    outer, k_len, inner = _strided_extents(x.shape, block_dim)
    out = torch.empty(x.shape, dtype=output_dtype, device=x.device)
    with _lib.on_device(x.device):
        _lib.check(_lib.load().mase_hip_qdq_mxfp_strided(
            x.data_ptr(), _lib.dtype_code(x.dtype), out.data_ptr(), _lib.dtype_code(output_dtype), outer, k_len, inner, 32,
            *_fmt(mxfp_meta), _lib.round_code(mxfp_meta.round_mode), _lib.stream_ptr(x.device)))
    return out


_WS_BYTES: dict[tuple, int] = {}


def _workspace_bytes(lib, dev_index, a_is_dense: bool, M: int, N: int, K: int) -> int:
    """The library's answer depends on the shape and the device only: ask once."""
    key = (dev_index, a_is_dense, M, N, K)
    n = _WS_BYTES.get(key)
    if n is None:
        n = _WS_BYTES[key] = lib.mase_hip_mxfp_gemm_workspace_bytes(int(a_is_dense), M, N, K)
    return n


def mxfp_gemm(
    a: Tensor | None,
    a_scales: Tensor | None,
    a_elements: Tensor | None,
    a_meta: MXFPMeta | None,
    w_scales: Tensor,
    w_elements: Tensor,
    w_meta: MXFPMeta,
    bias: Tensor | None,
    M: int,
    N: int,
    K: int,
    output_dtype: torch.dtype,
    out: Tensor | None = None,
    split_k: bool = True,
) -> Tensor:
    """y[M,N] = A[M,K] @ W[N,K]^T (+ bias) on bf16 MFMA with fp32 accumulation.

    A is either a dense [M,K] tensor (``a``; used as is) or MXFP components blocked along K.
    W is MXFP components of the row-major [N,K] weight, blocked along K.
    ``out``: optional contiguous [M,N] tensor of ``output_dtype`` to write into.
    ``split_k``: allow a temporary for partial sums (a few M*N*4 bytes) where the library asks for one;
    False keeps the call free of allocations other than the output.
    """
    dev = w_elements.device
    _lib.require_gpu(w_elements, "w_elements")
    assert w_scales.dtype == torch.uint8 and w_elements.dtype == torch.uint8
    assert w_meta.block_size == 32 and K % 32 == 0
    assert w_meta.element_is_finite, "the GEMM decodes finite-only element formats (the top exponent field is an ordinary binade)"
    assert w_elements.numel() == N * K and w_scales.numel() == N * K // 32
    w_scales, w_elements = _lib.dense(w_scales), _lib.dense(w_elements)
    a_ptr = a_sc_ptr = a_el_ptr = None
    a_dt, a_e, a_m = 0, 0, 0
    if a is not None:
        _lib.require_gpu(a, "activations")
        a = _lib.dense(a)
        assert a.numel() == M * K
        a_ptr, a_dt = a.data_ptr(), _lib.dtype_code(a.dtype)
    else:
        assert a_meta is not None and a_meta.block_size == 32
        a_scales, a_elements = _lib.dense(a_scales), _lib.dense(a_elements)
        assert a_elements.numel() == M * K and a_scales.numel() == M * K // 32
        a_sc_ptr, a_el_ptr = a_scales.data_ptr(), a_elements.data_ptr()
        a_e, a_m = a_meta.element_exp_bits, a_meta.element_frac_bits
    b_ptr, b_dt = None, 0
    if bias is not None:
        bias = _lib.dense(bias)
        assert bias.numel() == N
        b_ptr, b_dt = bias.data_ptr(), _lib.dtype_code(bias.dtype)
    if out is None:
        y = torch.empty((M, N), dtype=output_dtype, device=dev)
    else:
        assert out.is_contiguous() and out.dtype == output_dtype and out.numel() == M * N and out.device == dev
        y = out
    lib = _lib.load()
    with _lib.on_device(dev):
        # few output tiles and a long K: the library splits K over more workgroups if it is given room for the partial sums
        ws_bytes = _workspace_bytes(lib, dev.index, a is not None, M, N, K) if split_k else 0
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes > 0 else None
        _lib.check(lib.mase_hip_mxfp_gemm_ws(
            a_ptr, a_dt, a_sc_ptr, a_el_ptr, a_e, a_m, w_scales.data_ptr(), w_elements.data_ptr(),
            w_meta.element_exp_bits, w_meta.element_frac_bits, b_ptr, b_dt, y.data_ptr(),
            _lib.dtype_code(output_dtype), M, N, K, 32, None if ws is None else ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev)))
    return y


def mxfp_gemm_batched(a: Tensor, w_scales: Tensor, w_elements: Tensor, w_meta: MXFPMeta, batches: int, M: int, N: int, K: int,
                      output_dtype: torch.dtype, a_batch_stride: int, w_batch_stride: int) -> Tensor:
    """``batches`` products y[b] = A[b] @ W[b]^T in one launch.  ``a`` holds the dense bfloat16 A operands
    ``a_batch_stride`` elements apart, the components hold the weights ``w_batch_stride`` elements apart (blocks along
    K); a stride of 0 shares the operand between all products.  Returns y [batches, M, N]."""
    dev = w_elements.device
    _lib.require_gpu(w_elements, "w_elements")
    _lib.require_gpu(a, "activations")
    assert a.dtype == torch.bfloat16 and w_scales.dtype == torch.uint8 and w_elements.dtype == torch.uint8
    assert w_meta.block_size == 32 and K % 32 == 0
    assert w_meta.element_is_finite, "the GEMM decodes finite-only element formats (the top exponent field is an ordinary binade)"
    a, w_scales, w_elements = _lib.dense(a), _lib.dense(w_scales), _lib.dense(w_elements)
    assert a.numel() >= (batches - 1) * a_batch_stride + M * K
    assert w_elements.numel() >= (batches - 1) * w_batch_stride + N * K
    y = torch.empty((batches, M, N), dtype=output_dtype, device=dev)
    lib = _lib.load()
    with _lib.on_device(dev):
        for first in range(0, batches, 65535):      # one launch takes at most 65535 products
            count = min(65535, batches - first)
            esz = 2
            _lib.check(lib.mase_hip_mxfp_gemm_batched(
                a.data_ptr() + first * a_batch_stride * esz, _lib.dtype_code(a.dtype),
                w_scales.data_ptr() + first * (w_batch_stride // 32), w_elements.data_ptr() + first * w_batch_stride,
                w_meta.element_exp_bits, w_meta.element_frac_bits, y[first].data_ptr(), _lib.dtype_code(output_dtype),
                M, N, K, 32, count, a_batch_stride, w_batch_stride, M * N, _lib.stream_ptr(dev)))
    return y


# ---- the block-scaled matrix instruction route (FP8 bytes and E8M0 scales straight into the matrix unit)
_SCALED_FORMATS = {(4, 3), (2, 3), (3, 2), (2, 1)}


class ScaledOperand:
    """An [rows, K] MXFP matrix in the form the block-scaled GEMM reads: ``codes`` uint8 [rows_pad, K] (E4M3 bytes) and
    ``scales`` int32 [K // 128, rows_pad]; rows past ``rows`` are padding with undefined contents."""

    __slots__ = ("codes", "scales", "rows", "K")

    def __init__(self, codes: Tensor, scales: Tensor, rows: int, K: int):
        self.codes, self.scales, self.rows, self.K = codes, scales, rows, K


def scaled_element_format_supported(exp_bits: int, frac_bits: int) -> bool:
    """Is (exp_bits, frac_bits), finite, an element format the block-scaled GEMM's operands hold?"""
    return (exp_bits, frac_bits) in _SCALED_FORMATS


def scaled_format_supported(meta: MXFPMeta) -> bool:
    return (meta.block_size == 32 and meta.element_is_finite and meta.scale_exp_bits == 8
            and scaled_element_format_supported(meta.element_exp_bits, meta.element_frac_bits))


def scaled_shape_supported(N: int, K: int, output_dtype: torch.dtype) -> bool:
    return K % 256 == 0 and K >= 512 and N % (4 if output_dtype == torch.float32 else 8) == 0


def _scaled_buffers(rows: int, K: int, dev) -> tuple[Tensor, Tensor]:
    rows_pad = (rows + 255) // 256 * 256
    return (torch.empty((rows_pad, K), dtype=torch.uint8, device=dev),
            torch.empty((K // 128, rows_pad), dtype=torch.int32, device=dev))


def scaled_operand_from_dense(x: Tensor, meta: MXFPMeta) -> ScaledOperand:
    """Quantise the bfloat16 matrix x [rows, K] (blocks along K) straight into a block-scaled GEMM operand."""
    assert x.ndim == 2 and x.dtype == torch.bfloat16 and scaled_format_supported(meta) and meta.round_mode == "rn"
    _lib.require_gpu(x, "activations")
    x = _lib.dense(x)
    rows, K = x.shape
    codes, scales = _scaled_buffers(rows, K, x.device)
    if rows == 0:
        return ScaledOperand(codes, scales, rows, K)   # nothing to quantise
    with _lib.on_device(x.device):
        _lib.check(_lib.load().mase_hip_scaled_operand_from_dense(
            x.data_ptr(), _lib.dtype_code(x.dtype), meta.element_exp_bits, meta.element_frac_bits, rows, K,
            codes.data_ptr(), scales.data_ptr(), _lib.stream_ptr(x.device)))
    return ScaledOperand(codes, scales, rows, K)


def scaled_operand_from_dense_minifloat(x: Tensor, exp_bits: int, frac_bits: int) -> ScaledOperand:
    """Round every element of the bfloat16 matrix x [rows, K] to the finite minifloat format (exp_bits, frac_bits), to
    nearest, straight into a block-scaled GEMM operand whose blocks all carry the scale 2^0."""
    assert x.ndim == 2 and x.dtype == torch.bfloat16 and scaled_element_format_supported(exp_bits, frac_bits)
    _lib.require_gpu(x, "activations")
    x = _lib.dense(x)
    rows, K = x.shape
    codes, scales = _scaled_buffers(rows, K, x.device)
    if rows == 0:
        return ScaledOperand(codes, scales, rows, K)   # nothing to quantise
    with _lib.on_device(x.device):
        _lib.check(_lib.load().mase_hip_scaled_operand_from_dense_minifloat(
            x.data_ptr(), _lib.dtype_code(x.dtype), exp_bits, frac_bits, rows, K,
            codes.data_ptr(), scales.data_ptr(), _lib.stream_ptr(x.device)))
    return ScaledOperand(codes, scales, rows, K)


def scaled_operand_from_swiglu(gate: Tensor, up: Tensor, meta: MXFPMeta) -> ScaledOperand:
    """silu(gate) * up (bfloat16 [rows, K] each, unit inner stride, the same row stride: e.g. the two halves of a stacked
    projection's output) quantised straight into a block-scaled GEMM operand; the product is never stored."""
    assert gate.ndim == 2 and gate.shape == up.shape and gate.dtype == up.dtype == torch.bfloat16
    assert scaled_format_supported(meta) and meta.round_mode == "rn"
    _lib.require_gpu(gate, "activations")
    assert gate.device == up.device
    if gate.stride(1) != 1 or up.stride(1) != 1 or gate.stride(0) != up.stride(0) or gate.stride(0) % 8 or gate.data_ptr() % 16 or up.data_ptr() % 16:
        gate, up = gate.contiguous(), up.contiguous()
    rows, K = gate.shape
    codes, scales = _scaled_buffers(rows, K, gate.device)
    if rows == 0:
        return ScaledOperand(codes, scales, rows, K)   # nothing to quantise
    with _lib.on_device(gate.device):
        _lib.check(_lib.load().mase_hip_scaled_operand_from_swiglu(
            gate.data_ptr(), up.data_ptr(), _lib.dtype_code(gate.dtype), gate.stride(0) if rows > 1 else K,
            meta.element_exp_bits, meta.element_frac_bits, rows, K, codes.data_ptr(), scales.data_ptr(), _lib.stream_ptr(gate.device)))
    return ScaledOperand(codes, scales, rows, K)


def scaled_operand_from_mxfp(scales: Tensor, elements: Tensor, meta: MXFPMeta, rows: int, K: int) -> ScaledOperand:
    """MXFP components of a row-major [rows, K] matrix, blocked along K -> block-scaled GEMM operand."""
    assert scaled_format_supported(meta)
    assert scales.dtype == torch.uint8 and elements.dtype == torch.uint8
    _lib.require_gpu(elements, "elements")
    scales, elements = _lib.dense(scales), _lib.dense(elements)
    assert elements.numel() == rows * K and scales.numel() == rows * K // 32
    codes, out_scales = _scaled_buffers(rows, K, elements.device)
    with _lib.on_device(elements.device):
        _lib.check(_lib.load().mase_hip_scaled_operand_from_mxfp(
            scales.data_ptr(), elements.data_ptr(), meta.element_exp_bits, meta.element_frac_bits, rows, K,
            codes.data_ptr(), out_scales.data_ptr(), _lib.stream_ptr(elements.device)))
    return ScaledOperand(codes, out_scales, rows, K)


_SCALED_WS_BYTES: dict[tuple, int] = {}


def mxfp_gemm_scaled(a: ScaledOperand, w: ScaledOperand, bias: Tensor | None, output_dtype: torch.dtype,
                     out: Tensor | None = None, split_k: bool = True) -> Tensor:
    """y[M,N] = A @ W^T (+ bias) on the block-scaled matrix instruction, fp32 accumulation.
    ``split_k``: allow a temporary for partial sums where the library asks for one (few tiles, long K)."""
    assert a.K == w.K
    M, N, K = a.rows, w.rows, a.K
    dev = w.codes.device
    b_ptr, b_dt = None, 0
    if bias is not None:
        bias = _lib.dense(bias)
        assert bias.numel() == N
        b_ptr, b_dt = bias.data_ptr(), _lib.dtype_code(bias.dtype)
    if out is None:
        y = torch.empty((M, N), dtype=output_dtype, device=dev)
    else:
        assert out.is_contiguous() and out.dtype == output_dtype and out.numel() == M * N and out.device == dev
        y = out
    lib = _lib.load()
    with _lib.on_device(dev):
        ws_bytes = 0
        if split_k:
            key = (dev.index, M, N, K)
            ws_bytes = _SCALED_WS_BYTES.get(key)
            if ws_bytes is None:
                ws_bytes = _SCALED_WS_BYTES[key] = lib.mase_hip_mxfp_gemm_scaled_workspace_bytes(M, N, K)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes > 0 else None
        _lib.check(lib.mase_hip_mxfp_gemm_scaled_ws(
            a.codes.data_ptr(), a.scales.data_ptr(), w.codes.data_ptr(), w.scales.data_ptr(), b_ptr, b_dt, y.data_ptr(),
            _lib.dtype_code(output_dtype), M, N, K, None if ws is None else ws.data_ptr(), ws_bytes, _lib.stream_ptr(dev)))
    return y


_LINEAR_SCRATCH_BYTES: dict[tuple, int] = {}


def linear_scaled(x: Tensor, exp_bits: int, frac_bits: int, minifloat: bool, w: ScaledOperand, bias: Tensor | None) -> Tensor:
    """x [M, K] (bfloat16, contiguous, 16-byte aligned) quantised to MXFP elements (exp_bits, frac_bits) with block scales,
    or rounded element by element to that minifloat format, times W^T (+ bias) on the block-scaled matrix instruction:
    ``mxfp_gemm_scaled(scaled_operand_from_dense*(x), w, bias, x.dtype)`` through ONE call into the library (a decode-sized
    product is bound by the host otherwise).  The caller has checked formats and shape."""
    M, K = x.shape
    N = w.rows
    dev = x.device
    lib = _lib.load()
    key = (dev.index, M, N, K)
    nbytes = _LINEAR_SCRATCH_BYTES.get(key)
    if nbytes is None:
        with _lib.on_device(dev):
            nbytes = _LINEAR_SCRATCH_BYTES[key] = lib.mase_hip_mxfp_linear_scaled_scratch_bytes(M, N, K)
    scratch = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    y = torch.empty((M, N), dtype=x.dtype, device=dev)
    assert w.K == K and (bias is None or (bias.numel() == N and bias.device == dev))
    b_ptr, b_dt = (None, 0) if bias is None else (bias.data_ptr(), _lib.dtype_code(bias.dtype))
    with _lib.on_device(dev):
        _lib.check(lib.mase_hip_mxfp_linear_scaled(
            x.data_ptr(), _lib.dtype_code(x.dtype), exp_bits, frac_bits, int(minifloat), w.codes.data_ptr(), w.scales.data_ptr(), b_ptr, b_dt,
            y.data_ptr(), _lib.dtype_code(x.dtype), M, N, K, scratch.data_ptr(), nbytes, _lib.stream_ptr(dev)))
    return y


def prepared_w_shape_supported(M: int, N: int, K: int) -> bool:
    return M >= 512 and N % 128 == 0 and K % 128 == 0 and K <= (1 << 23)


def mxfp_gemm_prepared_w(a: Tensor, w: ScaledOperand, bias: Tensor | None, output_dtype: torch.dtype, out: Tensor | None = None) -> Tensor:
    """y[M,N] = a @ W^T (+ bias): dense bfloat16 ``a`` [M, K] (used as is) against a weight in the block-scaled GEMM's form, on
    the bf16 matrix instruction (W composed to bf16 in registers)."""
    assert a.ndim == 2 and a.dtype == torch.bfloat16 and a.shape[1] == w.K
    _lib.require_gpu(a, "activations")
    a = _lib.dense(a)
    M, N, K = a.shape[0], w.rows, w.K
    dev = w.codes.device
    b_ptr, b_dt = None, 0
    if bias is not None:
        bias = _lib.dense(bias)
        assert bias.numel() == N
        b_ptr, b_dt = bias.data_ptr(), _lib.dtype_code(bias.dtype)
    if out is None:
        y = torch.empty((M, N), dtype=output_dtype, device=dev)
    else:
        assert out.is_contiguous() and out.dtype == output_dtype and out.numel() == M * N and out.device == dev
        y = out
    with _lib.on_device(dev):
        _lib.check(_lib.load().mase_hip_mxfp_gemm_prepared_w(
            a.data_ptr(), _lib.dtype_code(a.dtype), w.codes.data_ptr(), w.scales.data_ptr(), b_ptr, b_dt, y.data_ptr(),
            _lib.dtype_code(output_dtype), M, N, K, _lib.stream_ptr(dev)))
    return y
