"""torch dtype -> dtype code of the C ABI (counterpart of the reference's torch -> Triton dtype
table, src/mase_triton/dtype.py:5-17, restricted to what the HIP kernels read and write)."""
import torch

TORCH_DTYPE_TO_CODE = {
    torch.float32: 0,
    torch.float16: 1,
    torch.bfloat16: 2,
}

ROUND_MODE_TO_CODE = {"rn": 0, "ru": 1, "rd": 2, "rz": 3}
