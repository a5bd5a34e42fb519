"""String/tuple normalisers used by the tensor-meta dataclasses
(same contract as src/mase_triton/utils/meta.py:4-25)."""
import torch


def device_str(device) -> str:
    return device if isinstance(device, str) else str(device)


def dtype_str(dtype) -> str:
    return dtype if isinstance(dtype, str) else str(dtype).removeprefix("torch.")


def shape_tuple(shape) -> tuple:
    return tuple(shape) if isinstance(shape, torch.Size) else shape
