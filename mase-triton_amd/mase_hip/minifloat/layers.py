"""Post-training-quantised linear layer with minifloat operands
(API of src/mase_triton/minifloat/layers.py:11-188)."""
from __future__ import annotations

from typing import Literal

import torch
from torch import Tensor, nn

from ..utils.qlayer import ChangeDtypeError
from . import functional as MinifloatF
from .meta import MinifloatMeta, MinifloatTensorMeta

LayerType = Literal["XWB", "XWBq", "XWqB", "XWqBq", "XqWB", "XqWBq", "XqWqB", "XqWqBq"]


class MinifloatLinearPTQ(nn.Module):
    """``y = x W^T + b`` with any of x / W / b held or rounded in a minifloat format.

    Quantised weights and biases are stored as uint16 code tensors (``w_element``,
    ``b_element``) registered as frozen parameters; their dtype may never change, which
    ``.to(dtype=...)`` would otherwise do, hence the check in ``_apply``.
    """

    in_features: int
    out_features: int
    _CODE_PARAMS = ("w_element", "b_element")

    def __init__(
        self,
        weight: Tensor | None,
        bias: Tensor | None,
        x_minifloat_meta: MinifloatMeta | None,
        w_minifloat_meta: MinifloatMeta | None,
        b_minifloat_meta: MinifloatMeta | None,
        layer_type: LayerType,
        backend: Literal["separate", "fused", "fused_bf16", "fused_scaled"] = "fused",
        dtype: torch.dtype | None = None,
        device: torch.device | None = None,
        w_element: Tensor | None = None,
        w_tensor_meta: MinifloatTensorMeta | None = None,
        b_element: Tensor | None = None,
        b_tensor_meta: MinifloatTensorMeta | None = None,
    ):
        super().__init__()
        assert weight is None or weight.ndim == 2
        assert bias is None or bias.ndim == 1
        have_w_codes = w_element is not None and w_tensor_meta is not None
        assert (weight is not None) ^ have_w_codes
        if bias is not None and b_element is not None and b_tensor_meta is not None:
            raise ValueError("Either bias or b_element, b_tensor_meta must be None, not both.")
        if weight is None:
            out_features, in_features = w_tensor_meta.shape
        else:
            out_features, in_features = weight.shape
        assert bias is None or bias.shape[0] == out_features

        self.in_features, self.out_features = in_features, out_features
        self.x_minifloat_meta = x_minifloat_meta
        self.w_minifloat_meta = w_minifloat_meta
        self.b_minifloat_meta = b_minifloat_meta
        self.layer_type = layer_type
        self.backend = backend
        self.dtype, self.device = dtype, device

        self.weight = self.bias = None
        self.w_element = self.w_tensor_meta = None
        self.b_element = self.b_tensor_meta = None
        self._narrowed = self._narrowed_key = None
        self._scaled_w = self._scaled_w_key = None
        self._fast_sig = None   # what the last call on the block-scaled route looked like (see forward)

        if "Wq" in layer_type:
            if w_element is None:
                w_element, w_tensor_meta = MinifloatF.extract_minifloat_component(weight, w_minifloat_meta)
            self.w_element = nn.Parameter(w_element, requires_grad=False)
            self.w_tensor_meta = w_tensor_meta
        else:
            assert weight is not None
            self.weight = nn.Parameter(weight.to(dtype=dtype, device=device), requires_grad=False)

        if "Bq" in layer_type:
            if bias is not None or b_element is not None:
                if b_element is None:
                    b_element, b_tensor_meta = MinifloatF.extract_minifloat_component(bias, b_minifloat_meta)
                self.b_element = nn.Parameter(b_element, requires_grad=False)
                self.b_tensor_meta = b_tensor_meta
        elif bias is not None:
            self.bias = nn.Parameter(bias.to(dtype=dtype, device=device), requires_grad=False)

    def _apply(self, fn, recurse=True):
        before = {n: getattr(self, n).dtype for n in self._CODE_PARAMS if getattr(self, n) is not None}
        result = super()._apply(fn, recurse)
        self._narrowed = self._narrowed_key = None
        self._scaled_w = self._scaled_w_key = self._fast_sig = None
        for name, dt in before.items():
            now = getattr(self, name).dtype
            if now != dt:
                raise ChangeDtypeError(f"Changing dtype of {name} from {dt} to {now} is not allowed.")
        if self.w_tensor_meta is not None and self.w_element is not None:
            self.w_tensor_meta = self.w_tensor_meta.create(device=self.w_element.device)
        if self.b_tensor_meta is not None and self.b_element is not None:
            self.b_tensor_meta = self.b_tensor_meta.create(device=self.b_element.device)
        return result

    def _narrowed_weight(self):
        """One-byte copy of the weight codes for the fused GEMM (not part of ``state_dict``),
        rebuilt when ``w_element`` is replaced, written in place or moved."""
        w = self.w_element
        if (self.backend == "separate" or w is None or w.device.type != "cuda"
                or not MinifloatF.gemm_weight_eligible(self.w_tensor_meta)):
            return None
        key = (w.data_ptr(), w._version, w.device)
        if self._narrowed_key != key:
            self._narrowed = MinifloatF.narrow_weight_codes(w, self.w_tensor_meta)
            self._narrowed_key = key
        return self._narrowed

    def _weight_operand(self, input: Tensor):
        """The weight in the block-scaled GEMM's form when this call takes that GEMM (quantised bfloat16 activations, see
        ``minifloat_linear``), else None.  Not part of ``state_dict``; rebuilt like the one-byte copy."""
        from ..mxfp.functional.linear import takes_scaled_route
        from .functional import linear as L

        w = self.w_element
        if self.backend in ("separate", "fused_bf16") or w is None or not self.layer_type.startswith("XqWq") or input.device.type != "cuda":
            return None
        rows = input.numel() // input.shape[-1] if input.numel() else 0
        bias = self.bias if not self.layer_type.endswith("Bq") else None
        if not ((self.backend == "fused_scaled" or takes_scaled_route(rows, True))
                and L._scaled_eligible(input, self.x_minifloat_meta, self.w_tensor_meta, bias)):
            return None
        key = (w.data_ptr(), w._version, w.device)
        if self._scaled_w_key != key:
            self._scaled_w = L.scaled_weight_operand(w, self.w_tensor_meta, self._narrowed_weight())
            self._scaled_w_key = key
        return self._scaled_w

    def _call_signature(self, input: Tensor) -> tuple:
        return (input.shape, input.dtype, input.device, self.backend, self.layer_type, self.x_minifloat_meta)

    @torch.no_grad()
    def forward(self, input: Tensor) -> Tensor:
        # A call that looks like the last one that ran on the block-scaled GEMM with the kept weight operand, the codes
        # unchanged since, goes straight to the two kernels: the checks below cost more host time than a decode-sized
        # product takes on the GPU.
        if self._fast_sig is not None and self._fast_sig == self._call_signature(input):
            w = self.w_element
            if self._scaled_w_key == (w.data_ptr(), w._version, w.device):
                from ..mxfp import kernels

                xm = self.x_minifloat_meta
                x2 = input.reshape(-1, self.in_features)
                bias = None if self.layer_type.endswith("Bq") else self.bias
                if x2.is_contiguous() and x2.data_ptr() % 16 == 0 and x2.shape[0] > 0 and (bias is None or bias.is_contiguous()):
                    y = kernels.linear_scaled(x2, xm.exp_bits, xm.frac_bits, True, self._scaled_w, bias)
                else:
                    y = kernels.mxfp_gemm_scaled(kernels.scaled_operand_from_dense_minifloat(x2, xm.exp_bits, xm.frac_bits), self._scaled_w, bias, input.dtype)
                return y.view(*input.shape[:-1], self.out_features)
        w_operand = self._weight_operand(input)
        self._fast_sig = self._call_signature(input) if w_operand is not None else None
        return MinifloatF.minifloat_linear(
            x=input, x_meta=self.x_minifloat_meta, w=self.weight, w_element=self.w_element,
            w_tensor_meta=self.w_tensor_meta, b=self.bias, b_element=self.b_element,
            b_tensor_meta=self.b_tensor_meta, layer_type=self.layer_type, backend=self.backend,
            _narrowed=self._narrowed_weight(), _w_operand=w_operand)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"layer_type={self.layer_type}, w_minifloat_meta={self.w_minifloat_meta}, "
                f"x_minifloat_meta={self.x_minifloat_meta}, b_minifloat_meta={self.b_minifloat_meta}")

    @classmethod
    def from_linear(cls, layer: nn.Linear, x_minifloat_meta: MinifloatMeta | None,
                    w_minifloat_meta: MinifloatMeta | None, b_minifloat_meta: MinifloatMeta | None,
                    layer_type: LayerType, backend: Literal["separate", "fused"]):
        """Quantise a trained ``nn.Linear``."""
        assert isinstance(layer, nn.Linear), "layer must be an instance of nn.Linear"
        with torch.no_grad():
            return cls(weight=layer.weight.clone(), bias=None if layer.bias is None else layer.bias.clone(),
                       x_minifloat_meta=x_minifloat_meta, w_minifloat_meta=w_minifloat_meta,
                       b_minifloat_meta=b_minifloat_meta, layer_type=layer_type, backend=backend)

    @classmethod
    def from_quantized(cls, w_element: Tensor | None, w_tensor_meta: MinifloatTensorMeta | None,
                       bias: Tensor | None, b_element: Tensor | None, b_tensor_meta: MinifloatTensorMeta | None,
                       x_minifloat_meta: MinifloatMeta | None,
                       layer_type: Literal["XWqB", "XWqBq", "XqWqB", "XqWqBq"],
                       backend: Literal["separate", "fused"]):
        """Re-hydrate from stored codes (tensor metas are not part of ``state_dict``)."""
        assert w_element is not None and w_tensor_meta is not None
        return cls(weight=None, bias=bias, x_minifloat_meta=x_minifloat_meta, w_minifloat_meta=None,
                   b_minifloat_meta=None, layer_type=layer_type, backend=backend,
                   dtype=getattr(torch, w_tensor_meta.dtype), device=torch.device(w_tensor_meta.device),
                   w_element=w_element, w_tensor_meta=w_tensor_meta, b_element=b_element,
                   b_tensor_meta=b_tensor_meta)
