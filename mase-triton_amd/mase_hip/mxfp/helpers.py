"""Layout helpers (API of src/mase_triton/mxfp/helpers.py:4-47): blocks are always taken along
the last axis of a flat array, so the block axis is rotated to the end before quantising and
rotated back after dequantising."""
from torch import Tensor


def flatten_for_quantize(tensor: Tensor, block_dim: int) -> Tensor:
    """Rotate ``block_dim`` to the last position, then flatten (copies unless already last)."""
    axes = list(range(tensor.ndim))
    axes.append(axes.pop(block_dim % tensor.ndim))
    return tensor.permute(axes).flatten()


def permute_for_dequantize(flatten_tensor: Tensor, ori_shape: tuple[int, ...], block_dim: int) -> Tensor:
    """Inverse of :func:`flatten_for_quantize`; returns a view (non-contiguous unless
    ``block_dim`` is the last axis)."""
    ndim = len(ori_shape)
    block_dim %= ndim
    rotated = list(ori_shape)
    rotated.append(rotated.pop(block_dim))
    back = list(range(ndim))
    back.insert(block_dim, back.pop())
    return flatten_tensor.reshape(rotated).permute(back)
