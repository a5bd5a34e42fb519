"""Post-training-quantised linear layer with MXFP operands
(API of src/mase_triton/mxfp/layers.py:11-211)."""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor, nn

from ..utils.qlayer import ChangeDtypeError
from . import functional as MXFP_F
from .meta import MXFPMeta, MXFPTensorMeta

LayerType = Literal["XWB", "XWBq", "XWqB", "XWqBq", "XqWB", "XqWBq", "XqWqB", "XqWqBq"]


class MXFPLinearPTQ(nn.Module):
    """``y = x W^T + b`` with any of x / W / b held or rounded in an MXFP format.

    A quantised weight is stored as two frozen uint8 parameters, ``w_scales`` [N*K/B, 1] and
    ``w_elements`` [N*K/B, B], blocked along in_features; likewise ``b_scales``/``b_elements``.
    Their dtype may never change (``.to(dtype=...)`` raises ``ChangeDtypeError``); moving the
    module between devices refreshes the device recorded in the tensor metas.  Unlike the
    reference, ``backend="fused"`` (the default) works: it runs the fused MFMA GEMMs.  Where the block-scaled route
    applies, the layer keeps the weight a second time in that kernel's form (``N * K * 33 / 32`` bytes, built on the
    first such forward and rebuilt when the components change or move; not part of ``state_dict``).
    """

    in_features: int
    out_features: int
    _CODE_PARAMS = ("w_scales", "w_elements", "b_scales", "b_elements")

    def __init__(
        self,
        weight: Tensor | None,
        bias: Tensor | None,
        x_mxfp_meta: MXFPMeta | None,
        w_mxfp_meta: MXFPMeta | None,
        b_mxfp_meta: MXFPMeta | None,
        layer_type: LayerType,
        backend: Literal["separate", "fused", "fused_bf16", "fused_scaled"] = "fused",
        dtype: torch.dtype | None = None,
        device: torch.device | None = None,
        w_scales: Tensor | None = None,
        w_elements: Tensor | None = None,
        w_tensor_meta: MXFPTensorMeta | None = None,
        b_scales: Tensor | None = None,
        b_elements: Tensor | None = None,
        b_tensor_meta: MXFPTensorMeta | None = None,
    ):
        super().__init__()
        assert weight is None or weight.ndim == 2
        assert bias is None or bias.ndim == 1
        have_w_parts = w_scales is not None and w_elements is not None and w_tensor_meta is not None
        have_b_parts = b_scales is not None and b_elements is not None and b_tensor_meta is not None
        assert (weight is not None) ^ have_w_parts
        if bias is not None and have_b_parts:
            raise ValueError("Either bias or b_scales, b_elements, b_tensor_meta must be None, not both.")
        if weight is None:
            out_features, in_features = w_tensor_meta.shape
        else:
            out_features, in_features = weight.shape
        assert bias is None or bias.shape[0] == out_features

        self.in_features, self.out_features = in_features, out_features
        self.x_mxfp_meta, self.w_mxfp_meta, self.b_mxfp_meta = x_mxfp_meta, w_mxfp_meta, b_mxfp_meta
        self.layer_type = layer_type
        self.backend = backend
        self.dtype, self.device = dtype, device

        self._scaled_w = self._scaled_w_key = None   # the weight in the block-scaled GEMM's form, and what it was built from
        self._fast_sig = None                        # what the last call on the block-scaled route looked like (see forward)
        self.weight = self.bias = None
        self.w_scales = self.w_elements = self.w_tensor_meta = None
        self.b_scales = self.b_elements = self.b_tensor_meta = None

        if "Wq" in layer_type:
            if w_scales is None:
                w_scales, w_elements, w_tensor_meta = MXFP_F.extract_mxfp_components(
                    weight, block_dim=1, mxfp_meta=w_mxfp_meta)
            self.w_scales = nn.Parameter(w_scales, requires_grad=False)
            self.w_elements = nn.Parameter(w_elements, requires_grad=False)
            self.w_tensor_meta = w_tensor_meta
        else:
            assert weight is not None
            self.weight = nn.Parameter(weight.to(dtype=dtype, device=device), requires_grad=False)

        if "Bq" in layer_type:
            if bias is not None or b_scales is not None:
                if b_scales is None:
                    b_scales, b_elements, b_tensor_meta = MXFP_F.extract_mxfp_components(
                        bias, block_dim=0, mxfp_meta=b_mxfp_meta)
                self.b_scales = nn.Parameter(b_scales, requires_grad=False)
                self.b_elements = nn.Parameter(b_elements, requires_grad=False)
                self.b_tensor_meta = b_tensor_meta
        elif bias is not None:
            self.bias = nn.Parameter(bias.to(dtype=dtype, device=device), requires_grad=False)

    def _apply(self, fn, recurse=True):
        before = {n: getattr(self, n).dtype for n in self._CODE_PARAMS if getattr(self, n) is not None}
        result = super()._apply(fn, recurse)
        for name, dt in before.items():
            now = getattr(self, name).dtype
            if now != dt:
                raise ChangeDtypeError(f"Changing dtype of {name} from {dt} to {now} is not allowed.")
        if self.w_tensor_meta is not None and self.w_scales is not None:
            self.w_tensor_meta = self.w_tensor_meta.create(device=self.w_scales.device)
        if self.b_tensor_meta is not None and self.b_scales is not None:
            self.b_tensor_meta = self.b_tensor_meta.create(device=self.b_scales.device)
        return result

    def invalidate_weight_operand(self) -> None:
        """Drop the cached block-scaled form of the weight.  Writes to ``w_scales`` / ``w_elements`` that torch records
        (``copy_`` under ``no_grad``, ``load_state_dict``, moving the module) are noticed without this call; writes
        through ``.data`` are not."""
        self._scaled_w = self._scaled_w_key = self._fast_sig = None

    def _takes_scaled_route(self, input: Tensor) -> bool:
        """Does ``forward(input)`` run on the block-scaled GEMM?"""
        from .functional import linear as L

        if self.backend in ("separate", "fused_bf16") or not self.layer_type.startswith("XqWq") or input.device.type != "cuda":
            return False
        rows = input.numel() // input.shape[-1] if input.numel() else 0
        bias = self.bias if not self.layer_type.endswith("Bq") else None
        return ((self.backend == "fused_scaled" or L.takes_scaled_route(rows, True))
                and L._scaled_eligible(input, self.x_mxfp_meta, self.w_tensor_meta, bias))

    def _weight_operand(self, input: Tensor):
        """The weight in the block-scaled GEMM's form when this call has a kernel that reads it (the block-scaled GEMM for
        quantised bfloat16 activations, the large-tile bf16 kernel from 512 rows on), else None."""
        from . import kernels
        from .functional import linear as L

        if self.backend == "separate" or "Wq" not in self.layer_type or input.device.type != "cuda":
            return None
        rows = input.numel() // input.shape[-1] if input.numel() else 0
        scaled = self._takes_scaled_route(input)
        if not scaled:
            tm = self.w_tensor_meta
            bf16 = (self.backend != "fused_scaled" and len(tm.shape) == 2 and kernels.scaled_format_supported(tm.meta) and tm.block_dim % 2 == 1
                    and input.dtype == torch.bfloat16 and getattr(torch, tm.dtype) == input.dtype
                    and kernels.prepared_w_shape_supported(rows, tm.shape[0], tm.shape[1]))
            if not bf16:
                return None
        key = (self.w_elements.data_ptr(), self.w_elements._version, self.w_scales.data_ptr(), self.w_scales._version)
        if self._scaled_w is None or self._scaled_w_key != key:
            self._scaled_w = L.scaled_weight_operand(self.w_scales, self.w_elements, self.w_tensor_meta)
            self._scaled_w_key = key
        return self._scaled_w

    def _call_signature(self, input: Tensor) -> tuple:
        return (input.shape, input.dtype, input.device, self.backend, self.layer_type, self.x_mxfp_meta)

    @torch.no_grad()
    def forward(self, input: Tensor) -> Tensor:
        # A call that looks like the last one that ran on the block-scaled GEMM with the kept weight operand, the weight
        # unchanged since, goes straight to the two kernels: the checks below cost more host time than a decode-sized
        # product takes on the GPU.
        if self._fast_sig is not None and self._fast_sig == self._call_signature(input):
            w_elements, w_scales = self.w_elements, self.w_scales
            if self._scaled_w_key == (w_elements.data_ptr(), w_elements._version, w_scales.data_ptr(), w_scales._version):
                from . import kernels

                x2 = input.reshape(-1, self.in_features)
                bias = None if self.layer_type.endswith("Bq") else self.bias
                meta = self.x_mxfp_meta
                if x2.is_contiguous() and x2.data_ptr() % 16 == 0 and x2.shape[0] > 0 and (bias is None or bias.is_contiguous()):
                    y = kernels.linear_scaled(x2, meta.element_exp_bits, meta.element_frac_bits, False, self._scaled_w, bias)
                else:
                    y = kernels.mxfp_gemm_scaled(kernels.scaled_operand_from_dense(x2, meta), self._scaled_w, bias, input.dtype)
                return y.view(*input.shape[:-1], self.out_features)
        w_operand = self._weight_operand(input)
        self._fast_sig = self._call_signature(input) if w_operand is not None and self._takes_scaled_route(input) else None
        return MXFP_F.mxfp_linear(
            x=input, x_meta=self.x_mxfp_meta, w=self.weight, w_scales=self.w_scales, w_elements=self.w_elements,
            w_tensor_meta=self.w_tensor_meta, b=self.bias, b_scales=self.b_scales, b_elements=self.b_elements,
            b_tensor_meta=self.b_tensor_meta, layer_type=self.layer_type, backend=self.backend,
            w_operand=w_operand)

    @torch.no_grad()
    def forward_swiglu(self, gate: Tensor, up: Tensor) -> Tensor:
        """``self(silu(gate) * up)``, the down projection of a SwiGLU block (not in the reference, where the caller writes
        that expression).  On the block-scaled route the activation, the product and the quantisation of the result run
        in one kernel that reads ``gate`` and ``up`` (e.g. the two halves of a stacked gate / up layer's output, as
        views) and writes FP8 codes: the bfloat16 product never goes to memory.  Each of the two operations is rounded to
        bfloat16 as torch rounds it, so the result equals the expression's up to the last bit of the SiLU's exponential.
        Everywhere else this is the expression."""
        from . import kernels

        if (gate.shape == up.shape and gate.dtype == up.dtype and gate.device == up.device and gate.shape[-1] == self.in_features
                and self.layer_type == "XqWqB" and self._takes_scaled_route(gate)):
            w_op = self._weight_operand(gate)
            a_op = kernels.scaled_operand_from_swiglu(gate.reshape(-1, self.in_features) if gate.ndim != 2 else gate,
                                                      up.reshape(-1, self.in_features) if up.ndim != 2 else up, self.x_mxfp_meta)
            y = kernels.mxfp_gemm_scaled(a_op, w_op, self.bias, gate.dtype)
            return y.view(*gate.shape[:-1], self.out_features)
        return self.forward(torch.nn.functional.silu(gate) * up)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"layer_type={self.layer_type}, w_mxfp_meta={self.w_mxfp_meta}, x_mxfp_meta={self.x_mxfp_meta}, "
                f"b_mxfp_meta={self.b_mxfp_meta}")

    @classmethod
    def from_linear(cls, layer: nn.Linear, x_mxfp_meta: MXFPMeta | None, w_mxfp_meta: MXFPMeta | None,
                    b_mxfp_meta: MXFPMeta | None, layer_type: LayerType, backend: Literal["separate", "fused", "fused_bf16", "fused_scaled"]):
        """Quantise a trained ``nn.Linear``."""
        assert isinstance(layer, nn.Linear), "layer must be an instance of nn.Linear"
        with torch.no_grad():
            return cls(weight=layer.weight.clone(), bias=None if layer.bias is None else layer.bias.clone(),
                       x_mxfp_meta=x_mxfp_meta, w_mxfp_meta=w_mxfp_meta, b_mxfp_meta=b_mxfp_meta,
                       layer_type=layer_type, backend=backend)

    def export_quantized(self) -> dict:
        """Everything needed to rebuild the layer, as tensors, strings and integers only (safe to
        ``torch.save`` and to load with ``weights_only=True``): element codes bit-packed, tensor
        metas as plain dicts.  Quantised-weight layer types only."""
        from . import packing

        assert self.w_scales is not None, "export_quantized needs a quantised weight (Wq layer types)"
        d = {"format": "mase_hip.mxfp.linear/1", "layer_type": self.layer_type,
             "x_mxfp_meta": None if self.x_mxfp_meta is None else packing.meta_to_dict(self.x_mxfp_meta),
             "w": packing.export_components(self.w_scales, self.w_elements, self.w_tensor_meta),
             "b": None, "bias": None if self.bias is None else self.bias.detach().clone()}
        if self.b_scales is not None:
            d["b"] = {"scales": self.b_scales.detach().reshape(-1).clone(), "elements": self.b_elements.detach().clone(),
                      "tensor_meta": packing.tensor_meta_to_dict(self.b_tensor_meta)}
        return d

    @classmethod
    def from_exported(cls, d: dict, backend: Literal["separate", "fused", "fused_bf16", "fused_scaled"] = "fused", device=None):
        """Inverse of :meth:`export_quantized`."""
        from . import packing

        assert d.get("format") == "mase_hip.mxfp.linear/1", "not an exported MXFP linear layer"
        w_scales, w_elements, w_tm = packing.import_components(d["w"], device=device)
        b_scales = b_elements = b_tm = None
        if d["b"] is not None:
            b_tm = packing.tensor_meta_from_dict(d["b"]["tensor_meta"], device=device)
            b_scales, b_elements = d["b"]["scales"].view(-1, 1), d["b"]["elements"]
            if device is not None:
                b_scales, b_elements = b_scales.to(device), b_elements.to(device)
        bias = d["bias"]
        if bias is not None and device is not None:
            bias = bias.to(device)
        x_meta = None if d["x_mxfp_meta"] is None else packing.meta_from_dict(d["x_mxfp_meta"])
        return cls.from_quantized(w_scales, w_elements, w_tm, bias, b_scales, b_elements, b_tm, x_meta, d["layer_type"], backend)

    @classmethod
    def from_quantized(cls, w_scales: Tensor | None, w_elements: Tensor | None, w_tensor_meta: MXFPTensorMeta | None,
                       bias: Tensor | None, b_scales: Tensor | None, b_elements: Tensor | None,
                       b_tensor_meta: MXFPTensorMeta | None, x_mxfp_meta: MXFPMeta | None,
                       layer_type: Literal["XWqB", "XWqBq", "XqWqB", "XqWqBq"],
                       backend: Literal["separate", "fused", "fused_bf16", "fused_scaled"]):
        """Re-hydrate from stored components (tensor metas are not part of ``state_dict``)."""
        assert w_scales is not None and w_elements is not None and w_tensor_meta is not None
        return cls(weight=None, bias=bias, x_mxfp_meta=x_mxfp_meta, w_mxfp_meta=None, b_mxfp_meta=None,
                   layer_type=layer_type, backend=backend, dtype=getattr(torch, w_tensor_meta.dtype),
                   device=torch.device(w_tensor_meta.device), w_scales=w_scales, w_elements=w_elements,
                   w_tensor_meta=w_tensor_meta, b_scales=b_scales, b_elements=b_elements,
                   b_tensor_meta=b_tensor_meta)
