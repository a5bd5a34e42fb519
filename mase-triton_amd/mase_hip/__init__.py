"""mase_hip - MXFP / minifloat quantisation and the MXFP GEMM on AMD MI355X (gfx950).

Mirrors the module layout of ``mase_triton`` for this path, so that

    import mase_hip.mxfp.functional as MXFP_F
    from mase_hip.mxfp.layers import MXFPLinearPTQ

read like their ``mase_triton`` counterparts.  ``alias_as_mase_triton()`` additionally
registers the sub-packages under the ``mase_triton`` name for code that imports that name.

Every numerical entry point runs hand-written HIP kernels from ``lib/libmase_hip.so`` through
its C ABI.  There is no CPU implementation in this package: tensors that are not on a GPU, or
a missing library, raise an error.
"""
from __future__ import annotations

import importlib
import sys

__version__ = "0.1.0"

_SUBMODULES = (
    "dtype", "manager", "utils", "utils.meta", "utils.qlayer",
    "minifloat", "minifloat.meta", "minifloat.kernels", "minifloat.functional", "minifloat.layers",
    "mxfp", "mxfp.meta", "mxfp.helpers", "mxfp.kernels", "mxfp.functional", "mxfp.layers",
)


def alias_as_mase_triton(name: str = "mase_triton") -> None:
    """Make ``import mase_triton.mxfp.functional`` (etc.) resolve to this package."""
    if name in sys.modules and sys.modules[name] is not sys.modules[__name__]:
        raise RuntimeError(f"a different module named {name!r} is already imported")
    sys.modules[name] = sys.modules[__name__]
    for sub in _SUBMODULES:
        sys.modules[f"{name}.{sub}"] = importlib.import_module(f"{__name__}.{sub}")
