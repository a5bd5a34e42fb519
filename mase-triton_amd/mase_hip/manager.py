"""Kernel configuration switch, API-compatible with src/mase_triton/manager.py:7-32.

The reference toggles Triton autotuning and reloads its kernel modules.  The HIP kernels
have fixed launch shapes, so the flag is only recorded."""
import logging

logger = logging.getLogger(__name__)


class KernelManager:
    _autotune_is_enabled = False

    @classmethod
    def enable_autotune(cls):
        cls._autotune_is_enabled = True
        logger.info("Autotune enabled (no effect: HIP kernels use fixed launch shapes)")

    @classmethod
    def disable_autotune(cls):
        cls._autotune_is_enabled = False
        logger.info("Autotune disabled")

    @classmethod
    def autotune_is_enabled(cls):
        return cls._autotune_is_enabled
